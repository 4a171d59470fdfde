"""fp32 restatement of the reference's torch path for the MXFP4 fused-MoE layer.

Test infrastructure only (see ``oracle/__init__.py``).

Restates
  * end-to-end semantics (w1 = gate rows then up rows, silu(x Wg^T) * (x Wu^T) Wd^T, times the
    routing weight, summed per token): tests/contrib/moe/test_moe.py:73-118 (``get_torch_ref``)
  * the a4w4 variant, where activations are MXFP4 as well and both operands are dequantised to
    fp32 before ``src.float() @ w.t().float()``: src/contrib/moe_gemm_ref.py:93-142 and
    tests/contrib/moe/test_mxfp4.py:102-236; stage-1 output is rounded to bf16 and re-quantised
    before stage 2 (tests/contrib/moe/test_moe.py:732-744); stage-2 output is ``bf16(acc * w)`` per
    (token, slot) (src/contrib/moe_gemm_mxfp4.py:1291-1333)
  * top-k reduction ``bf16(sum_slot f32(in[t, slot, :]))``, slots in index order:
    src/contrib/moe_gemm_mxfp4.py:199-282
  * the w4a16 variant (bf16 activations, only weights dequantised): src/contrib/moe.py:362-787 as
    driven by tests/contrib/moe/test_moe.py:347-374.

Pins: the matmuls are ``torch.matmul`` in fp32 on exactly-dequantised operands (a library
routine); SiLU is ``torch.nn.functional.silu``; tests/test_oracle_moe.py checks the whole
function against an independent dense formulation (one-hot routing matrix, einsum) and against
hand-computable cases (identity-like weights, single expert, zero routing weight).
"""
import numpy as np
import torch

from . import mxfp4


def _t(x):
    return torch.from_numpy(np.ascontiguousarray(x))


def silu(x):
    return torch.nn.functional.silu(_t(np.asarray(x, dtype=np.float32))).numpy()


def act_quant_dequant(x):
    """bf16-valued float32 rows -> what the MXFP4 activation path feeds the GEMM (float32)."""
    q, s = mxfp4.quantize_mxfp4(x)
    return mxfp4.dequantize_mxfp4(q, s)


def expert_weights_f32(wq, ws):
    """(uint8 [N, K/2] plain row-major, uint8 [N, K/32]) -> float32 [N, K]"""
    return mxfp4.dequantize_mxfp4(wq, ws)


def swiglu(gate, up, limit=None):
    """gpt-oss's gated activation as the reference states it (tests/contrib/moe/test_moe.py:76-81): the gate is
    clamped from above only, the up projection from both sides, limit 7.0 when none is given."""
    limit = float(limit) if limit else 7.0
    g = _t(np.asarray(gate, dtype=np.float32)).clamp(max=limit)
    u = _t(np.asarray(up, dtype=np.float32)).clamp(min=-limit, max=limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)).numpy()


def gateup_ref(x, w1, bias1=None, activation="silu", swiglu_limit=None):
    """x f32 [n, H], w1 f32 [2I, H] -> bf16-rounded silu(gate) * up (or swiglu(gate, up)), f32 [n, I]"""
    acc = torch.matmul(_t(x), _t(w1).t()).numpy()
    if bias1 is not None:
        acc = acc + np.asarray(bias1, dtype=np.float32)[None, :]
    I = w1.shape[0] // 2
    if activation == "swiglu":
        return mxfp4.bf16_round(swiglu(acc[:, :I], acc[:, I:], swiglu_limit))
    assert activation == "silu"
    return mxfp4.bf16_round(silu(acc[:, :I]) * acc[:, I:])


def down_ref(a2, w2, weight, bias2=None):
    """a2 f32 [n, I], w2 f32 [H, I], weight f32 [n] -> bf16-rounded (acc (+bias)) * weight, f32 [n, H]"""
    acc = torch.matmul(_t(a2), _t(w2).t()).numpy()
    if bias2 is not None:
        acc = acc + np.asarray(bias2, dtype=np.float32)[None, :]
    return mxfp4.bf16_round(acc * np.asarray(weight, dtype=np.float32)[:, None])


def moe_ref(hidden, w1q, w1s, w2q, w2s, topk_weight, topk_ids, *, act="a4",
            bias1=None, bias2=None, experts=None, return_parts=False, activation="silu", swiglu_limit=None):
    """Whole layer.

    hidden      float32 [T, H] holding bf16 values
    w1q, w1s    uint8 [E, 2I, H/2], uint8 [E, 2I, H/32]   (plain row-major, not shuffled)
    w2q, w2s    uint8 [E, H, I/2],  uint8 [E, H, I/32]
    act         "a4": activations go through MXFP4 before each GEMM; "a16": bf16 activations
    experts     optional iterable restricting the experts that are evaluated (bounded CPU baseline)
    -> float32 [T, H] (the f32 slot sum), and its bf16 rounding via ``mxfp4.bf16_round``.
    """
    hidden = np.asarray(hidden, dtype=np.float32)
    T, H = hidden.shape
    topk_ids = np.asarray(topk_ids)
    topk_weight = np.asarray(topk_weight, dtype=np.float32)
    k = topk_ids.shape[1]
    E = w1q.shape[0]
    I = w1q.shape[1] // 2
    x_in = act_quant_dequant(hidden) if act == "a4" else hidden
    per_slot = np.zeros((T, k, H), dtype=np.float32)
    a2_all = np.zeros((T, k, I), dtype=np.float32)
    for e in (range(E) if experts is None else experts):
        tok, slot = np.nonzero(topk_ids == e)
        if tok.size == 0:
            continue
        w1 = expert_weights_f32(w1q[e], w1s[e])
        w2 = expert_weights_f32(w2q[e], w2s[e])
        a2 = gateup_ref(x_in[tok], w1, None if bias1 is None else bias1[e], activation, swiglu_limit)
        a2_all[tok, slot] = a2
        a2_in = act_quant_dequant(a2) if act == "a4" else a2
        per_slot[tok, slot] = down_ref(a2_in, w2, topk_weight[tok, slot],
                                       None if bias2 is None else bias2[e])
    out = np.zeros((T, H), dtype=np.float32)
    for s in range(k):                       # slots added in index order, f32
        out += per_slot[:, s]
    if return_parts:
        return out, a2_all, per_slot
    return out
