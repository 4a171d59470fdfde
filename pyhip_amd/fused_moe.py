"""``fused_moe``: MXFP4 fused Mixture-of-Experts layer on MI355X.

Same call surface as the reference's ``fused_moe`` (src/contrib/fused_moe.py:128-155): routing weights
and top-k ids in, per-token bf16 hidden states out.  Weights are MXFP4 (``quant_type=QuantType.per_1x32``):
``w1`` [E, 2*I, H/2] (gate rows then up rows) and ``w2`` [E, H, I/2] as uint8 / float4_e2m1fn_x2 in the
pre-shuffled layout, ``w1_scale`` / ``w2_scale`` e8m0 in the shuffled layout (see ``pyhip_amd.mxfp4``).

Pipeline (all launches on the current torch stream, no host synchronisation):
  sort -> quantise activations to MXFP4 -> gate_up GEMM + SiLU*up (+ re-quantisation) -> down GEMM * routing
  weight -> top-k reduction.

``method="w4a16"`` keeps the activations in bf16 (weights are expanded to bf16 in registers), the variant the
reference runs for few tokens (src/contrib/moe.py:362-787); ``method="a4w4"`` forces the MXFP4-activation path;
``method="auto"`` takes w4a16 for the very smallest calls (see ``pick_w4a16``) and a4w4 above.
"""
import torch

from . import _lib
from .enums import ActivationType, QuantType
from .moe_sorting import moe_sorting, max_blocks

__all__ = ["fused_moe", "fused_moe_routed"]


def _as_u8(t):
    if t is None:
        return None
    return t if t.dtype == torch.uint8 else t.view(torch.uint8)


def _require(cond, msg, exc=ValueError):
    """argument checks raise (an ``assert`` would vanish under ``python -O``)"""
    if not cond:
        raise exc("fused_moe: " + msg)


def _is_shuffled(w):
    """the reference's convention (src/contrib/fused_moe.py:198-206): an ``nn.Parameter`` counts as pre-shuffled
    (wrapping drops the attribute), otherwise the tensor attribute ``is_shuffled`` says so, default False"""
    if isinstance(w, torch.nn.parameter.Parameter):
        return True
    return bool(getattr(w, "is_shuffled", False))


_shuffle_cache = {}          # id(source storage) -> {view key: (tensor version, re-tiled copy)}
_SHUFFLE_CACHE_STORAGES = 8  # plain-layout weight storages remembered at once (each entry holds a full re-tiled copy)


def _shuffled_u8(w):
    """uint8 view of an MXFP4 weight tensor in the pre-shuffled layout the kernels read.  Plain-layout weights
    ([E, N, K/2] row-major, ``is_shuffled`` unset) are shuffled once and remembered (the reference's kernels take both
    layouts, src/contrib/fused_moe.py:410,480; here the plain layout costs one re-tiling pass on first use and a second
    copy of the weights).  An entry belongs to the source tensor's storage object: it is dropped by a finalizer when that
    storage is freed, so a new tensor that lands at the same address never finds a stale copy, and an in-place change
    of the source (its version counter) invalidates it."""
    wu = _as_u8(w)
    if _is_shuffled(w):
        return wu
    import weakref
    from .mxfp4 import shuffle_weight
    storage = wu.untyped_storage()
    sid = id(storage)            # the storage's Python object lives exactly as long as the storage
    views = _shuffle_cache.get(sid)
    if views is None:
        while len(_shuffle_cache) >= _SHUFFLE_CACHE_STORAGES:
            _shuffle_cache.pop(next(iter(_shuffle_cache)))      # oldest first
        views = _shuffle_cache[sid] = {}
        weakref.finalize(storage, _shuffle_cache.pop, sid, None)
    key = (wu.storage_offset(), tuple(wu.shape), tuple(wu.stride()))
    hit = views.get(key)
    if hit is not None and hit[0] == wu._version:
        return hit[1]
    out = shuffle_weight(wu.contiguous())
    views[key] = (wu._version, out)
    return out


def pick_block_m(tokens, topk, experts, hidden=0, w4a16=False):
    """M-tile (= sort block size), from the expected rows per expert ``est = tokens * topk / experts``: 16 rows below 4,
    32 below 12, 64 up to 32, 128 above (layers with fewer than 32 experts: the smallest of 16 / 32 / 64 that holds
    twice ``est``).  Every extra row block of an expert streams the expert's weights once more,
    routing is uneven enough that a tile of just the mean size overflows for about half of the experts, and the rows a
    larger tile leaves empty fetch nothing (DS-V3 shape: T = 1024: 64-row tiles 1.20 ms against 1.27 ms with 32;
    T = 2048: 128-row tiles 1.27 ms against 1.39 ms with 64).  The ladder sits one step above "twice the mean" at decode
    sizes so that routers with uneven expert loads do not pay for it: that costs 1-2 % under an even router and saves
    11-17 % under a Zipf(1.1) one (the numbers are quoted beside ``pyhip_moe_pick_block_m``).

    The tiles of 160, 192, 256 and 288 rows (one wave per SIMD, slower per FLOP) are taken where they save whole passes
    over the weights: where a 128-row tile needs two or three blocks for most experts and the taller tile one, read with
    non-temporal loads (100-132 expected rows per expert: 160 rows; up to 172: 192; up to 236: 256; up to 276: 288).
    Their long epilogue pays most with a long K loop: DS-V3 (hidden 7168) T = 4096 / 6144: 1.36 / 1.64 ms against
    1.70 / 1.92 ms with 128 rows, T = 8192: 1.95 ms with 288 rows against 2.26; at hidden 3072 / 4096 only the 160-row step
    is taken (100-132 expected rows per expert: gpt-oss shape T = 4096 0.50 against 0.56 ms, Mixtral shape T = 512 0.19
    against 0.21; a router that loads its experts unevenly loses with it: Qwen3 shape, Zipf, T = 2048 0.42 against 0.40)."""
    return int(_lib.load().pyhip_moe_pick_block_m(tokens, topk, experts, hidden, 1 if w4a16 else 0))


def pick_w4a16(tokens, topk, experts, hidden):
    """``method="auto"``: True selects the bf16-activation kernels (the reference switches to its w4a16 split-K
    kernel for few tokens, src/contrib/moe.py:362-787).  They win in two regimes (measured on all five benchmark
    shapes, quoted next to the rule in pyhip_moe_pick_w4a16): when at most one expert in eight gets a row at all
    (DeepSeek-V3 shape up to 4 tokens), and in layers with so few experts that the down GEMM of the MXFP4-activation
    path, one workgroup per (row block, 256 output channels), cannot fill the GPU while the bf16-activation kernel
    splits K over four times as many workgroups (Mixtral shape up to 32 tokens)."""
    return bool(_lib.load().pyhip_moe_pick_w4a16(tokens, topk, experts, hidden))


def act_quant_mxfp4(x, rows_limit=None):
    """bf16 [rows, K] -> (uint8 [rows, K/2], uint8 [rows, ceil(K/512)*16]) in the GEMM's A-operand layout."""
    lib = _lib.load()
    _require(x.dtype == torch.bfloat16 and x.dim() == 2, "act_quant_mxfp4 takes a bf16 matrix", TypeError)
    if x.stride(1) != 1 or x.stride(0) % 8 != 0 or x.data_ptr() % 16 != 0:
        x = x.contiguous()
    rows, K = x.shape
    sk = lib.pyhip_moe_act_scale_stride(K)
    q = torch.empty(rows, K // 2, dtype=torch.uint8, device=x.device)
    s = torch.empty(rows, sk, dtype=torch.uint8, device=x.device)
    rc = lib.pyhip_moe_act_quant_mxfp4(_lib.dptr(x), x.stride(0), rows, K, _lib.dptr(q), _lib.dptr(s),
                                       _lib.dptr(rows_limit), _lib.current_stream())
    _lib.check(rc, "act_quant_mxfp4")
    return q, s


def fused_moe(
    hidden_states,
    w1,  # [E, inter_dim*2, dim/2]  gate rows then up rows
    w2,  # [E, dim, inter_dim/2]
    topk_weight,
    topk_ids,
    expert_mask=None,
    activation=ActivationType.Silu,
    quant_type=QuantType.per_1x32,
    doweight_stage1=False,
    w1_scale=None,
    w2_scale=None,
    a1_scale=None,
    a2_scale=None,
    block_size_M=None,
    num_local_tokens=None,
    moe_sorting_dispatch_policy=0,
    dtype=None,
    hidden_pad=0,
    intermediate_pad=0,
    bias1=None,
    bias2=None,
    splitk=0,
    method="auto",
    return_parts=False,
    stage_events=None,
    swiglu_limit=None,
    topk_reduce="store",
    operand_staging="registers",
):
    """See the module docstring.  Extras beyond the reference signature: ``dtype=torch.float32`` returns
    the fp32 top-k sum without the final bf16 rounding; ``return_parts=True`` also returns the
    intermediate buffers; ``stage_events`` (a list) receives ``(name, start_event, end_event)`` per stage;
    ``activation=ActivationType.Swiglu`` selects gpt-oss's clamped SwiGLU with ``swiglu_limit`` (default 7.0, as
    tests/contrib/moe/test_moe.py:76-81); ``topk_reduce="atomic"`` (MXFP4-activation path, row block 16 or 128,
    bf16 output) lets the down GEMM add its results into the output with packed bf16 atomics, the reference's atomic
    variant (src/contrib/moe_gemm_mxfp4.py:1334-1398), instead of the deterministic store + reduction;
    ``topk_reduce="last_arriver"`` (MXFP4-activation path, row block 16, 128 or 288) keeps the stores and lets the
    workgroup of the down GEMM that stores a token's last slot sum the slots, in the order and arithmetic of the
    reduction kernel: the same bits, one launch less;
    ``operand_staging="lds"`` (MXFP4-activation path, 256-row blocks, at most 512 experts) runs both GEMMs on the
    eight-wave tile whose weights, too, are staged through LDS (the tile shape of the reference's prefill kernel,
    src/contrib/moe_gemm_mxfp4.py:318-637) instead of the tiles that load weights straight into registers:
    bit-identical results, measured slower, never chosen automatically."""
    lib = _lib.load()
    _require(activation in (ActivationType.Silu, ActivationType.Swiglu), "SiLU- or SwiGLU-gated experts only")
    act = 1 if activation == ActivationType.Swiglu else 0
    limit = float(swiglu_limit) if swiglu_limit else 7.0
    _require(quant_type == QuantType.per_1x32, "this operator is the MXFP4 (per_1x32) path")
    _require(not doweight_stage1, "doweight_stage1 is not supported (the reference rejects it as well)")
    _require(a1_scale is None and a2_scale is None, "activations are quantised dynamically: a1_scale / a2_scale must be None")
    _require(splitk in (0, 1, 4, 16, 32), "splitk: 0 = automatic, 1 = off, 4 / 16 = split K over that many waves of a workgroup, "
             "32 = sixteen waves on 32-row weight tiles in the down GEMM (w4a16 path only)")
    _require(w1_scale is not None and w2_scale is not None, "w1_scale and w2_scale (e8m0, shuffled) are required")
    _require(hidden_states.is_cuda and hidden_states.dtype == torch.bfloat16 and hidden_states.dim() == 2,
             "hidden_states must be a bf16 matrix on the GPU", TypeError)
    out_dtype = hidden_states.dtype if dtype is None else dtype
    _require(out_dtype in (torch.bfloat16, torch.float32), "dtype must be bfloat16 or float32", TypeError)
    _require(method in ("auto", "a4w4", "w4a16", "jit", "gluon"), "method=%r" % (method,))
    _require(topk_reduce in ("store", "atomic", "last_arriver"), "topk_reduce=%r" % (topk_reduce,))
    _require(operand_staging in ("registers", "lds"), "operand_staging=%r" % (operand_staging,))

    # weights in the plain layout (no ``is_shuffled`` mark) are re-tiled once; the scales always come e8m0-shuffled,
    # as the reference passes them (tests/contrib/moe/test_moe.py:167-189)
    w1u, w2u, w1s, w2s = _shuffled_u8(w1), _shuffled_u8(w2), _as_u8(w1_scale), _as_u8(w2_scale)
    _require(w1u.dim() == 3 and w2u.dim() == 3, "w1 [E, 2*inter, hidden/2] and w2 [E, hidden, inter/2] expected")
    # hidden_pad / intermediate_pad: the weights arrive zero-padded to the kernels' tile multiples and the last
    # hidden_pad (intermediate_pad) channels are padding.  The activations may come at the padded width (the
    # reference's convention) or at the true width, in which case they are widened here and the result is
    # returned at the true width.  The MXFP4-activation GEMMs are told the pads and leave the weights' padding unfetched.
    _require(0 <= hidden_pad < w1u.shape[2] * 2 and 0 <= intermediate_pad < w1u.shape[1] // 2, "bad hidden_pad / intermediate_pad")
    narrow = hidden_pad > 0 and hidden_states.shape[1] == w1u.shape[2] * 2 - hidden_pad
    if narrow:
        hidden_states = torch.nn.functional.pad(hidden_states, (0, hidden_pad))
    T, H = hidden_states.shape
    _require(topk_ids.dim() == 2 and topk_ids.shape[0] == T and tuple(topk_weight.shape) == tuple(topk_ids.shape),
             "topk_ids / topk_weight must be [tokens, topk]")
    k = topk_ids.shape[1]
    E, N1, Hb = w1u.shape
    I = N1 // 2
    _require(Hb * 2 == H and tuple(w2u.shape) == (E, H, I // 2),
             "shapes do not fit: hidden %d, w1 %s, w2 %s" % (H, tuple(w1u.shape), tuple(w2u.shape)))
    _require(w1u.is_contiguous() and w2u.is_contiguous() and w1s.is_contiguous() and w2s.is_contiguous(),
             "weights and scales must be contiguous")
    global_E = E if expert_mask is None else expert_mask.numel()
    dev = hidden_states.device
    if T == 0:
        return torch.zeros(0, H, dtype=out_dtype, device=dev)

    def _mark(name, start=None):
        if stage_events is None:
            return None
        ev = torch.cuda.Event(enable_timing=True)
        ev.record()
        if start is not None:
            stage_events.append((name, start, ev))
        return ev

    topk_ids = topk_ids.to(torch.int32).contiguous()
    topk_weight = topk_weight.to(torch.float32).contiguous()
    # "auto" (and the reference's "jit" / "gluon", which name its own back ends): see pick_w4a16
    w4a16 = method == "w4a16" or (method != "a4w4" and pick_w4a16(T, k, global_E, H))
    bm = block_size_M if block_size_M is not None else pick_block_m(T, k, global_E, H, w4a16)
    if w4a16:
        bm = min(bm, 64)
    if bias1 is not None:
        bias1 = bias1.to(torch.bfloat16).contiguous()
        _require(tuple(bias1.shape) == (E, 2 * I), "bias1 must be [E, 2*inter]")
    if bias2 is not None:
        bias2 = bias2.to(torch.bfloat16).contiguous()
        _require(tuple(bias2.shape) == (E, H), "bias2 must be [E, hidden]")

    if expert_mask is not None:
        expert_mask = expert_mask.to(device=dev, dtype=torch.int32).contiguous()
    if num_local_tokens is not None:
        _require(num_local_tokens.is_cuda and num_local_tokens.dtype == torch.int32,
                 "num_local_tokens must be an int32 scalar tensor on the GPU", TypeError)

    lds_tile = operand_staging == "lds"
    if lds_tile:
        _require(not w4a16 and block_size_M in (None, 256) and topk_reduce == "store",
                 "operand_staging='lds' needs the MXFP4-activation path, 256-row blocks and topk_reduce='store'")
        bm = 256
    atomic = topk_reduce == "atomic"
    if atomic:
        _require(not w4a16 and bm in (16, 128) and out_dtype == torch.bfloat16,
                 "topk_reduce='atomic' needs the MXFP4-activation path, a row block of 16 or 128 and bf16 output")

    arriver = topk_reduce == "last_arriver"
    if arriver:
        _require(not w4a16 and bm in (16, 128, 288) and not lds_tile,
                 "topk_reduce='last_arriver' needs the MXFP4-activation path and a row block of 16, 128 or 288")

    if not return_parts and stage_events is None and not atomic and not lds_tile and not arriver:
        # the whole layer in one library call, intermediates in one workspace: two allocations and one foreign call
        # per layer instead of a dozen of each (the host side is what bounds small layers when they are not replayed
        # from a graph)
        x = hidden_states
        # the kernels read 16-byte pieces of a row: views with an odd row stride or base (a column slice) are copied
        if x.stride(1) != 1 or (w4a16 and x.stride(0) != H) or x.stride(0) % 8 != 0 or x.data_ptr() % 16 != 0:
            x = x.contiguous()
        ws_bytes = lib.pyhip_moe_forward_workspace_bytes(T, k, global_E, H, I, bm, 1 if w4a16 else 0)
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
        out = torch.empty(T, H, dtype=out_dtype, device=dev)
        rc = lib.pyhip_moe_forward(_lib.dptr(x), x.stride(0), _lib.dptr(w1u), _lib.dptr(w1s), _lib.dptr(w2u),
                                   _lib.dptr(w2s), _lib.dptr(bias1), _lib.dptr(bias2), _lib.dptr(topk_ids),
                                   _lib.dptr(topk_weight), _lib.dptr(expert_mask), _lib.dptr(num_local_tokens),
                                   _lib.dptr(out), 1 if out_dtype == torch.float32 else 0, T, k, global_E, H, I,
                                   hidden_pad, intermediate_pad, bm, 1 if w4a16 else 0, splitk, act, limit,
                                   _lib.dptr(ws), ws_bytes, _lib.current_stream())
        _lib.check(rc, "moe_forward")
        return out[:, : H - hidden_pad] if narrow else out

    ev = _mark("start")
    # MXFP4-activation path: the input quantisation rides in the sort's launches (independent work, one dispatch less)
    qin = None
    if not w4a16:
        qin = hidden_states if hidden_states.stride(1) == 1 else hidden_states.contiguous()
    res = moe_sorting(topk_ids, topk_weight, global_E, H, out_dtype, bm, expert_mask, num_local_tokens,
                      moe_sorting_dispatch_policy, alloc_moe_out=False, return_schedule=True, quant_input=qin)
    sorted_ids, sorted_w, sorted_e, num_valid, _, sched = res[:6]
    ev = _mark("sort", ev)
    n_blk = sorted_e.numel()
    stream = _lib.current_stream()

    def _reduce(out3, out):
        # slots the sort dropped (ids outside [0, E), masked experts, tokens past the local count) were never
        # written by the down GEMM: the reduction reads the routing and leaves them out
        return lib.pyhip_moe_topk_reduce_routed(_lib.dptr(out3), _lib.dptr(out), T, k, H,
                                                1 if out_dtype == torch.float32 else 0, _lib.dptr(topk_ids), global_E,
                                                _lib.dptr(expert_mask), _lib.dptr(num_local_tokens), stream)

    if w4a16:
        hs = hidden_states.contiguous()
        a2 = torch.empty(n_blk * bm, I, dtype=torch.bfloat16, device=dev)
        rc = lib.pyhip_moe_gemm1_w4a16(_lib.dptr(hs), _lib.dptr(w1u), _lib.dptr(w1s), _lib.dptr(bias1),
                                       _lib.dptr(sorted_ids), _lib.dptr(sorted_e), _lib.dptr(num_valid),
                                       _lib.dptr(a2), T, k, global_E, H, I, bm, n_blk, splitk, act, limit, stream)
        _lib.check(rc, "moe_gemm1_w4a16")
        ev = _mark("gemm1", ev)
        out3 = torch.empty(T, k, H, dtype=torch.bfloat16, device=dev)
        rc = lib.pyhip_moe_gemm2_w4a16(_lib.dptr(a2), _lib.dptr(w2u), _lib.dptr(w2s), _lib.dptr(bias2),
                                       _lib.dptr(sorted_ids), _lib.dptr(sorted_w), _lib.dptr(sorted_e),
                                       _lib.dptr(num_valid), _lib.dptr(out3), T, k, global_E, H, I, bm, n_blk, splitk, stream)
        _lib.check(rc, "moe_gemm2_w4a16")
        ev = _mark("gemm2", ev)
        out = torch.empty(T, H, dtype=out_dtype, device=dev)
        rc = _reduce(out3, out)
        _lib.check(rc, "moe_topk_reduce")
        _mark("reduce", ev)
        if narrow:
            out = out[:, : H - hidden_pad]
        if return_parts:
            return out, dict(sorted_ids=sorted_ids, sorted_weights=sorted_w, sorted_expert_ids=sorted_e,
                             num_valid_ids=num_valid, a2=a2, out3=out3, block_m=bm)
        return out

    a1_q, a1_s = res[6]
    # the stage-1 kernel writes its result already quantised for stage 2; the bf16 copy is only produced on request
    a2 = torch.empty(n_blk * bm, I, dtype=torch.bfloat16, device=dev) if return_parts else None
    a2_q = torch.empty(n_blk * bm, I // 2, dtype=torch.uint8, device=dev)
    a2_s = torch.empty(n_blk * bm, lib.pyhip_moe_act_scale_stride(I), dtype=torch.uint8, device=dev)
    if lds_tile:
        rc = lib.pyhip_moe_gemm1_mxfp4_lds(_lib.dptr(a1_q), _lib.dptr(a1_s), _lib.dptr(w1u), _lib.dptr(w1s),
                                           _lib.dptr(bias1), _lib.dptr(sorted_ids), _lib.dptr(sorted_e),
                                           _lib.dptr(num_valid), _lib.dptr(sched), _lib.dptr(a2), _lib.dptr(a2_q),
                                           _lib.dptr(a2_s), T, k, global_E, H, I, n_blk, act, limit, stream)
    else:
        rc = lib.pyhip_moe_gemm1_mxfp4(_lib.dptr(a1_q), _lib.dptr(a1_s), _lib.dptr(w1u), _lib.dptr(w1s),
                                       _lib.dptr(bias1), _lib.dptr(sorted_ids), _lib.dptr(sorted_e),
                                       _lib.dptr(num_valid), _lib.dptr(sched), _lib.dptr(a2), _lib.dptr(a2_q),
                                       _lib.dptr(a2_s), T, k, global_E, H, I, hidden_pad, intermediate_pad, bm, n_blk,
                                       act, limit, stream)
    _lib.check(rc, "moe_gemm1_mxfp4")
    ev = _mark("gemm1", ev)
    if atomic:
        out3 = None
        out = torch.empty(T, H, dtype=out_dtype, device=dev)
        _lib.check(lib.pyhip_moe_zero_fill(_lib.dptr(out), out.numel() * 2, stream), "moe_zero_fill")
        rc = lib.pyhip_moe_gemm2_mxfp4_atomic(_lib.dptr(a2_q), _lib.dptr(a2_s), _lib.dptr(w2u), _lib.dptr(w2s),
                                              _lib.dptr(bias2), _lib.dptr(sorted_ids), _lib.dptr(sorted_w),
                                              _lib.dptr(sorted_e), _lib.dptr(num_valid), _lib.dptr(sched), _lib.dptr(out),
                                              T, k, global_E, H, I, bm, n_blk, stream)
        _lib.check(rc, "moe_gemm2_mxfp4_atomic")
        _mark("gemm2", ev)
    elif arriver:
        # the down GEMM whose workgroups also sum a token's slots (whoever stores the last one): no reduction launch
        out3 = torch.empty(T, k, H, dtype=torch.bfloat16, device=dev)
        out = torch.empty(T, H, dtype=out_dtype, device=dev)
        arrive = torch.empty(T * (H // 256), dtype=torch.int32, device=dev)
        rc = lib.pyhip_moe_gemm2_mxfp4_reduce(_lib.dptr(a2_q), _lib.dptr(a2_s), _lib.dptr(w2u), _lib.dptr(w2s),
                                              _lib.dptr(bias2), _lib.dptr(sorted_ids), _lib.dptr(sorted_w),
                                              _lib.dptr(sorted_e), _lib.dptr(num_valid), _lib.dptr(sched), _lib.dptr(out3),
                                              _lib.dptr(topk_ids), _lib.dptr(expert_mask), _lib.dptr(num_local_tokens),
                                              _lib.dptr(arrive), _lib.dptr(out), 1 if out_dtype == torch.float32 else 0,
                                              T, k, global_E, H, I, bm, n_blk, stream)
        _lib.check(rc, "moe_gemm2_mxfp4_reduce")
        _mark("gemm2", ev)
    else:
        out3 = torch.empty(T, k, H, dtype=torch.bfloat16, device=dev)
        if lds_tile:
            rc = lib.pyhip_moe_gemm2_mxfp4_lds(_lib.dptr(a2_q), _lib.dptr(a2_s), _lib.dptr(w2u), _lib.dptr(w2s),
                                               _lib.dptr(bias2), _lib.dptr(sorted_ids), _lib.dptr(sorted_w),
                                               _lib.dptr(sorted_e), _lib.dptr(num_valid), _lib.dptr(sched),
                                               _lib.dptr(out3), T, k, global_E, H, I, n_blk, stream)
        else:
            rc = lib.pyhip_moe_gemm2_mxfp4(_lib.dptr(a2_q), _lib.dptr(a2_s), _lib.dptr(w2u), _lib.dptr(w2s),
                                           _lib.dptr(bias2), _lib.dptr(sorted_ids), _lib.dptr(sorted_w),
                                           _lib.dptr(sorted_e), _lib.dptr(num_valid), _lib.dptr(sched), _lib.dptr(out3),
                                           T, k, global_E, H, I, hidden_pad, intermediate_pad, bm, n_blk, stream)
        _lib.check(rc, "moe_gemm2_mxfp4")
        ev = _mark("gemm2", ev)
        out = torch.empty(T, H, dtype=out_dtype, device=dev)
        rc = _reduce(out3, out)
        _lib.check(rc, "moe_topk_reduce")
        _mark("reduce", ev)
    if narrow:
        out = out[:, : H - hidden_pad]
    if return_parts:
        return out, dict(sorted_ids=sorted_ids, sorted_weights=sorted_w, sorted_expert_ids=sorted_e,
                         num_valid_ids=num_valid, a1_q=a1_q, a1_s=a1_s, a2=a2, a2_q=a2_q, a2_s=a2_s,
                         out3=out3, block_m=bm)
    return out


def fused_moe_routed(hidden_states, w1, w2, gating_output, topk, renormalize=True, num_expert_group=0, topk_group=0,
                     w1_scale=None, w2_scale=None, expert_mask=None, activation=ActivationType.Silu,
                     block_size_M=None, num_local_tokens=None, dtype=None, bias1=None, bias2=None, splitk=0,
                     method="auto", swiglu_limit=None, return_routing=False, hidden_pad=0, intermediate_pad=0):
    """``fused_topk`` (or ``grouped_topk`` when ``num_expert_group > 0``) followed by ``fused_moe``, as the reference's
    callers chain them (tests/contrib/moe/test_fused_moe.py:38-60), in one library call: for up to 64 tokens the
    router runs inside the sort's launch.  ``gating_output`` f32 [T, E], E a multiple of 64 (use ``fused_topk`` +
    ``fused_moe`` otherwise).  ``hidden_pad`` / ``intermediate_pad`` as for ``fused_moe``, with the activations at the
    padded width.  -> out, or (out, topk_weights, topk_ids) with ``return_routing``."""
    lib = _lib.load()
    _require(activation in (ActivationType.Silu, ActivationType.Swiglu), "SiLU- or SwiGLU-gated experts only")
    act = 1 if activation == ActivationType.Swiglu else 0
    limit = float(swiglu_limit) if swiglu_limit else 7.0
    _require(w1_scale is not None and w2_scale is not None, "w1_scale and w2_scale (e8m0, shuffled) are required")
    _require(hidden_states.is_cuda and hidden_states.dtype == torch.bfloat16 and hidden_states.dim() == 2,
             "hidden_states must be a bf16 matrix on the GPU", TypeError)
    out_dtype = hidden_states.dtype if dtype is None else dtype
    _require(out_dtype in (torch.bfloat16, torch.float32), "dtype must be bfloat16 or float32", TypeError)
    _require(method in ("auto", "a4w4", "w4a16"), "method=%r" % (method,))
    w1u, w2u, w1s, w2s = _shuffled_u8(w1), _shuffled_u8(w2), _as_u8(w1_scale), _as_u8(w2_scale)
    T, H = hidden_states.shape
    E, N1, Hb = w1u.shape
    I = N1 // 2
    _require(Hb * 2 == H and tuple(w2u.shape) == (E, H, I // 2), "shapes do not fit")
    global_E = E if expert_mask is None else expert_mask.numel()
    _require(gating_output.is_cuda and tuple(gating_output.shape) == (T, global_E) and global_E % 64 == 0,
             "gating_output must be [tokens, experts] on the GPU with experts a multiple of 64")
    g = gating_output.float().contiguous()
    dev = hidden_states.device
    if expert_mask is not None:
        expert_mask = expert_mask.to(device=dev, dtype=torch.int32).contiguous()
    w4a16 = method == "w4a16" or (method != "a4w4" and pick_w4a16(T, topk, global_E, H))
    bm = block_size_M if block_size_M is not None else pick_block_m(T, topk, global_E, H, w4a16)
    if w4a16:
        bm = min(bm, 64)
    if bias1 is not None:
        bias1 = bias1.to(torch.bfloat16).contiguous()
    if bias2 is not None:
        bias2 = bias2.to(torch.bfloat16).contiguous()
    x = hidden_states
    if x.stride(1) != 1 or (w4a16 and x.stride(0) != H) or x.stride(0) % 8 != 0 or x.data_ptr() % 16 != 0:
        x = x.contiguous()
    ws_bytes = lib.pyhip_moe_forward_workspace_bytes(T, topk, global_E, H, I, bm, 1 if w4a16 else 0)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    out = torch.empty(T, H, dtype=out_dtype, device=dev)
    tw = torch.empty(T, topk, dtype=torch.float32, device=dev)
    ti = torch.empty(T, topk, dtype=torch.int32, device=dev)
    rc = lib.pyhip_moe_forward_routed(_lib.dptr(x), x.stride(0), _lib.dptr(w1u), _lib.dptr(w1s), _lib.dptr(w2u),
                                      _lib.dptr(w2s), _lib.dptr(bias1), _lib.dptr(bias2), _lib.dptr(g),
                                      int(num_expert_group), int(topk_group), 1 if renormalize else 0, _lib.dptr(ti),
                                      _lib.dptr(tw), _lib.dptr(expert_mask), _lib.dptr(num_local_tokens), _lib.dptr(out),
                                      1 if out_dtype == torch.float32 else 0, T, topk, global_E, H, I, int(hidden_pad),
                                      int(intermediate_pad), bm, 1 if w4a16 else 0, splitk, act, limit, _lib.dptr(ws),
                                      ws_bytes, _lib.current_stream())
    _lib.check(rc, "moe_forward_routed")
    return (out, tw, ti) if return_routing else out
