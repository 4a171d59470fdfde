"""Pins for oracle/moe.py, oracle/routing.py and oracle/metrics.py: an independent dense
formulation, hand-computable special cases, closed forms."""
import numpy as np
import pytest
import torch

from oracle import mxfp4, moe, routing, metrics


def _layer(rng, E, T, k, H, I):
    hidden = mxfp4.bf16_round(rng.standard_normal((T, H)).astype(np.float32))
    w1 = (rng.standard_normal((E, 2 * I, H)) * 0.02).astype(np.float32)
    w2 = (rng.standard_normal((E, H, I)) * 0.02).astype(np.float32)
    w1q, w1s = mxfp4.quantize_mxfp4(w1)
    w2q, w2s = mxfp4.quantize_mxfp4(w2)
    tw, ti = routing.softmax_topk(rng.standard_normal((T, E)), k)
    return hidden, w1q, w1s, w2q, w2s, tw, ti


@pytest.mark.parametrize("act", ["a4", "a16"])
def test_against_dense_formulation(act):
    rng = np.random.default_rng(0)
    E, T, k, H, I = 4, 9, 2, 64, 32
    hidden, w1q, w1s, w2q, w2s, tw, ti = _layer(rng, E, T, k, H, I)
    out, a2, per_slot = moe.moe_ref(hidden, w1q, w1s, w2q, w2s, tw, ti, act=act, return_parts=True)
    # independent: every token through every expert in float64, combined with a dense routing matrix
    W1 = mxfp4.dequantize_mxfp4(w1q, w1s).astype(np.float64)
    W2 = mxfp4.dequantize_mxfp4(w2q, w2s).astype(np.float64)
    qd = (lambda v: mxfp4.dequantize_mxfp4(*mxfp4.quantize_mxfp4(v.astype(np.float32))).astype(np.float64)) \
        if act == "a4" else (lambda v: v.astype(np.float64))
    x = qd(hidden)
    gu = np.einsum("th,enh->etn", x, W1)
    g, u = gu[..., :I], gu[..., I:]
    a = mxfp4.bf16_round((g / (1 + np.exp(-g)) * u).astype(np.float32))
    y = np.einsum("eti,ehi->eth", qd(a.reshape(E * T, I)).reshape(E, T, I), W2)
    dense = np.zeros((T, H))
    for t in range(T):
        for s in range(k):
            dense[t] += mxfp4.bf16_round((y[ti[t, s], t] * tw[t, s]).astype(np.float32))
    # float64 vs float32 matmul can flip single bf16 / e2m1 roundings; the bulk must agree tightly
    assert metrics.cosine(out, dense) > 0.99999
    assert np.median(np.abs(out - dense)) < 1e-3 * np.sqrt(np.mean(dense ** 2))
    assert a2.shape == (T, k, I) and per_slot.shape == (T, k, H)


def test_single_expert_identity_weights():
    # one expert, w1 = [4*I_H ; 4*I_H] (gate = up = 4x), w2 = identity -> out = silu(4x) * 4x * weight
    H = I = 32
    eye = np.eye(H, dtype=np.float32)
    w1q, w1s = mxfp4.quantize_mxfp4(np.concatenate([4 * eye, 4 * eye])[None])
    w2q, w2s = mxfp4.quantize_mxfp4(eye[None])
    assert (mxfp4.dequantize_mxfp4(w1q, w1s)[0, :H] == 4 * eye).all()
    x = mxfp4.bf16_round(np.linspace(-1, 1, 3 * H, dtype=np.float32).reshape(3, H))
    tw = np.array([[1.0], [0.5], [0.0]], dtype=np.float32)
    ti = np.zeros((3, 1), dtype=np.int32)
    out = moe.moe_ref(x, w1q, w1s, w2q, w2s, tw, ti, act="a16")
    g = 4 * x
    expect = mxfp4.bf16_round(mxfp4.bf16_round(g / (1 + np.exp(-g)) * g) * tw)
    np.testing.assert_allclose(out, expect, rtol=2 ** -7, atol=1e-6)
    assert (out[2] == 0).all()


def test_bias_and_expert_subset():
    rng = np.random.default_rng(1)
    E, T, k, H, I = 4, 6, 2, 64, 32
    hidden, w1q, w1s, w2q, w2s, tw, ti = _layer(rng, E, T, k, H, I)
    b1 = (rng.standard_normal((E, 2 * I)) * 0.01).astype(np.float32)
    b2 = (rng.standard_normal((E, H)) * 0.01).astype(np.float32)
    full = moe.moe_ref(hidden, w1q, w1s, w2q, w2s, tw, ti, bias1=b1, bias2=b2)
    parts = sum(moe.moe_ref(hidden, w1q, w1s, w2q, w2s, tw, ti, bias1=b1, bias2=b2, experts=[e]) for e in range(E))
    np.testing.assert_allclose(full, parts, rtol=1e-6, atol=1e-7)
    nob = moe.moe_ref(hidden, w1q, w1s, w2q, w2s, tw, ti)
    assert np.abs(full - nob).max() > 0


def test_routers():
    rng = np.random.default_rng(2)
    logits = rng.standard_normal((50, 64))
    w, ids = routing.softmax_topk(logits, 4)
    assert np.allclose(w.sum(1), 1, atol=1e-6) and all(len(set(r)) == 4 for r in ids.tolist())
    assert (ids[:, 0] == logits.argmax(1)).all()
    w, ids = routing.grouped_sigmoid_topk(logits, 8, n_group=8, topk_group=4)
    assert np.allclose(w.sum(1), 1, atol=1e-6)
    for t in range(50):
        assert len(set(ids[t].tolist())) == 8
        assert len(set((ids[t] // 8).tolist())) <= 4
        # brute force: best 4 groups by the sum of their two best sigmoids, then best 8 inside
        s = 1 / (1 + np.exp(-logits[t]))
        gs = [np.sort(s[g * 8:(g + 1) * 8])[-2:].sum() for g in range(8)]
        groups = sorted(range(8), key=lambda g: -gs[g])[:4]
        cand = sorted([e for g in groups for e in range(g * 8, g * 8 + 8)], key=lambda e: -s[e])[:8]
        assert sorted(cand) == sorted(ids[t].tolist())


def test_metrics_closed_forms():
    x = np.arange(1, 9, dtype=np.float32)
    assert metrics.calc_diff(x, x) == 0 and abs(metrics.calc_diff(x, -x) - 2) < 1e-12
    assert abs(metrics.calc_diff(x, 0 * x) - 1) < 1e-12
    assert abs(metrics.calc_diff(x, 3 * x) - (1 - 6 / 10)) < 1e-12      # 1 - 2c/(1+c^2)
    assert abs(metrics.cosine(x, 5 * x) - 1) < 1e-12
    assert abs(metrics.max_err_over_rms(x + 0.5, x) - 0.5 / np.sqrt(np.mean(x.astype(np.float64) ** 2))) < 1e-12


def test_swiglu_pins():
    """gpt-oss's gated activation (tests/contrib/moe/test_moe.py:76-81) against the formula in float64 and against
    the cases that tell its clamps apart: the gate is clamped from above ONLY, the up projection from both sides,
    the limit defaults to 7."""
    rng = np.random.default_rng(5)
    g = rng.uniform(-6, 6, 1000).astype(np.float32)
    u = rng.uniform(-6, 6, 1000).astype(np.float32)
    g64, u64 = g.astype(np.float64), u.astype(np.float64)
    np.testing.assert_allclose(moe.swiglu(g, u), g64 / (1 + np.exp(-1.702 * g64)) * (u64 + 1), rtol=2e-6, atol=1e-6)

    def closed(gv, uv):
        return gv / (1 + np.exp(-1.702 * gv)) * (uv + 1)
    one = np.ones(1, np.float32)
    np.testing.assert_allclose(moe.swiglu(100 * one, 2 * one), closed(7.0, 2.0), rtol=1e-6)            # gate clamped above
    assert abs(float(moe.swiglu(-100 * one, 2 * one)[0])) < 1e-30                                      # ... not below
    assert abs(closed(-7.0, 2.0)) > 1e-5                                                               # (a symmetric clamp would show)
    np.testing.assert_allclose(moe.swiglu(one, 100 * one), closed(1.0, 7.0), rtol=1e-6)                # up clamped above
    np.testing.assert_allclose(moe.swiglu(one, -100 * one), closed(1.0, -7.0), rtol=1e-6)              # ... and below
    np.testing.assert_allclose(moe.swiglu(3 * one, 3 * one, 0.5), closed(0.5, 0.5), rtol=1e-6)         # explicit limit
    np.testing.assert_allclose(moe.swiglu(3 * one, 3 * one, None), moe.swiglu(3 * one, 3 * one, 7.0))  # default 7
    assert float(moe.swiglu(0 * one, 0 * one)[0]) == 0.0                                               # zero padding stays zero
    # through the gate_up restatement: identity-like weights, gate = 4x, up = 2x
    H = I = 32
    eye = np.eye(H, dtype=np.float32)
    w1 = np.concatenate([4 * eye, 2 * eye])
    x = mxfp4.bf16_round(np.linspace(-3, 3, 2 * H, dtype=np.float32).reshape(2, H))
    got = moe.gateup_ref(x, w1, activation="swiglu", swiglu_limit=5.0)
    gv, uv = np.minimum(4 * x.astype(np.float64), 5.0), np.clip(2 * x.astype(np.float64), -5.0, 5.0)
    np.testing.assert_allclose(got, mxfp4.bf16_round(closed(gv, uv).astype(np.float32)), rtol=2 ** -7, atol=1e-6)
    assert np.abs(got - moe.gateup_ref(x, w1)).max() > 0.1                                             # differs from SiLU


@pytest.mark.parametrize("act", ["a4", "a16"])
def test_shared_expert_as_an_extra_slot_is_routed_plus_dense(act):
    """A shared expert appended as slot k (pyhip_amd.routing.append_shared_experts) gives the routed experts' sum plus
    the shared expert applied to every token: checked on the oracle by evaluating the two halves separately."""
    from pyhip_amd.routing import append_shared_experts
    rng = np.random.default_rng(5)
    E, T, k, H, I = 4, 11, 2, 64, 32
    hidden, w1q, w1s, w2q, w2s, _, _ = _layer(rng, E + 1, T, k, H, I)
    tw, ti = routing.softmax_topk(rng.standard_normal((T, E)), k)          # routed experts 0 .. E-1 only
    tw2, ti2 = append_shared_experts(torch.from_numpy(tw), torch.from_numpy(ti), E, 1, shared_weight=0.5)
    assert tw2.dtype == torch.float32 and ti2.dtype == torch.int32 and tw2.shape == ti2.shape == (T, k + 1)
    assert (ti2[:, :k].numpy() == ti).all() and (ti2[:, k] == E).all()
    assert (tw2[:, :k].numpy() == tw).all() and (tw2[:, k] == 0.5).all()
    both = moe.moe_ref(hidden, w1q, w1s, w2q, w2s, tw2.numpy(), ti2.numpy(), act=act)
    routed = moe.moe_ref(hidden, w1q[:E], w1s[:E], w2q[:E], w2s[:E], tw, ti, act=act)
    x = moe.act_quant_dequant(hidden) if act == "a4" else hidden
    a2 = moe.gateup_ref(x, moe.expert_weights_f32(w1q[E], w1s[E]))
    a2 = moe.act_quant_dequant(a2) if act == "a4" else a2
    shared = moe.down_ref(a2, moe.expert_weights_f32(w2q[E], w2s[E]), np.full(T, 0.5, np.float32))
    assert (both == routed + shared).all()           # the shared slot is added last, in fp32: the same operations
    # two shared experts
    tw3, ti3 = append_shared_experts(torch.from_numpy(tw), torch.from_numpy(ti), E - 1, 2)
    assert (ti3[:, k:] == torch.tensor([E - 1, E], dtype=torch.int32)).all() and (tw3[:, k:] == 1.0).all()
