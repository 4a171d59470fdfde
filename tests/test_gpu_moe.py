"""GPU parity of the MXFP4 fused-MoE hot path through the C ABI.

Tolerance (floating point): against the oracle's fp32 path on identical seeded inputs (see _end_to_end),
max|err| <= 1e-2 * rms(ref) and cosine >= 0.999 on the operator's fp32 output; its bf16 output may
differ from the fp32 reference by half a bf16 ulp of the value on top of that (the output quantum).
Integer/byte stages (activation quantisation, sort) are bit-exact.
"""
import numpy as np
import pytest
import torch

from oracle import metrics, moe, mxfp4 as om
from pyhip_amd import fused_moe
from pyhip_amd.fused_moe import act_quant_mxfp4
import cases

pytestmark = pytest.mark.gpu

TOL_MAX = 1e-2
TOL_COS = 0.999


def _f(t):
    return t.float().cpu().numpy()


def test_act_quant_bit_exact():
    g = torch.Generator().manual_seed(0)
    rows, K = 37, 1024
    x = torch.randn(rows, K, generator=g) * torch.exp(torch.randn(rows, 1, generator=g) * 3)
    x[0, :32] = 0                                                     # all-zero block
    ties = torch.tensor([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0, 4.0, -0.25, -0.75, -1.25, -1.75, -2.5, -3.5, -5.0, 6.0])
    x[1, :16] = ties                                                  # exact ties, block scale 1
    x[1, 16:32] = 0
    x[2, :32] = torch.linspace(-7.9, 7.9, 32)                         # saturation range (scale 1)
    x[3, :64] = torch.randn(64, generator=g) * 1e-30                  # tiny exponents
    x[4, :64] = torch.randn(64, generator=g) * 1e30
    xb = x.to(torch.bfloat16)
    print("act_quant case rows=37 K=1024", flush=True)
    q, s = act_quant_mxfp4(xb.cuda())
    torch.cuda.synchronize()
    oq, os_ = om.quantize_mxfp4(xb.float().numpy())
    got_s = cases.untranspose_act_scales(s.cpu().numpy(), K)
    assert (got_s == os_).all(), np.argwhere(got_s != os_)[:10]
    bad = np.argwhere(q.cpu().numpy() != oq)
    assert bad.size == 0, (bad[:10], q.cpu().numpy()[tuple(bad[0])], oq[tuple(bad[0])])


class _Flips(tuple):
    """(stage-1, stage-2) counts of roundings that went the other way, plus ``moved_tokens`` (bool [T])"""


def _stage_checks(L, parts, bm):
    """stage-by-stage comparison; every stage is fed the KERNEL's previous output.
    -> (worst stage-1 error, worst stage-2 error, the oracle's layer output given the kernel's stage-1 result,
        numbers of stage-1 / stage-2 values whose bf16 rounding went the other way than the oracle's; that pair
        carries ``moved_tokens``: the tokens with a stage-1 row whose re-quantised MXFP4 form differs from the
        oracle's, i.e. where such a rounding also crossed an e2m1 or block-scale boundary)"""
    so = parts["sorted_ids"].cpu().numpy().view(np.uint32)
    se = parts["sorted_expert_ids"].cpu().numpy().view(np.uint32)
    sw = parts["sorted_weights"].cpu().numpy()
    nv = int(parts["num_valid_ids"][0])
    x = om.dequantize_mxfp4(*om.quantize_mxfp4(_f(L.hidden)))
    a2 = _f(parts["a2"])
    out3 = _f(parts["out3"])
    a2q = om.dequantize_mxfp4(*om.quantize_mxfp4(a2[:nv]))
    worst1 = worst2 = 0.0
    nflip1 = nflip2 = ntot1 = ntot2 = 0
    per_slot = np.zeros((L.T, L.k, out3.shape[2]), np.float32)
    moved_tokens = np.zeros(L.T, bool)
    for b in range(nv // bm):
        e = int(se[b])
        ids = so[b * bm:(b + 1) * bm]
        tok, slot = (ids & 0xFFFFFF).astype(np.int64), (ids >> 24).astype(np.int64)
        ok = slot < L.k
        w1 = moe.expert_weights_f32(L.w1q[e], L.w1s[e])
        w2 = moe.expert_weights_f32(L.w2q[e], L.w2s[e])
        b1 = None if L.bias1 is None else _f(L.bias1[e])
        b2 = None if L.bias2 is None else _f(L.bias2[e])
        ref1 = moe.gateup_ref(x[tok[ok]], w1, b1)
        got1 = a2[b * bm:(b + 1) * bm][ok]
        rms1 = np.sqrt(np.mean(ref1 ** 2)) + 1e-30
        # both sides are bf16 roundings of nearly equal fp32 values: allow one bf16 ulp of the value
        worst1 = max(worst1, (np.maximum(np.abs(got1 - ref1) - np.abs(ref1) * 2.0 ** -7, 0)).max() / rms1)
        nflip1 += int((got1 != ref1).sum())
        ntot1 += got1.size
        if (got1 != ref1).any():
            moved = (om.dequantize_mxfp4(*om.quantize_mxfp4(ref1)) != a2q[b * bm:(b + 1) * bm][ok]).any(axis=1)
            moved_tokens[tok[ok][moved]] = True
        assert (a2[b * bm:(b + 1) * bm][~ok] == 0).all()
        ref2 = moe.down_ref(a2q[b * bm:(b + 1) * bm][ok], w2, sw[b * bm:(b + 1) * bm][ok], b2)
        got2 = out3[tok[ok], slot[ok]]
        per_slot[tok[ok], slot[ok]] = ref2
        rms2 = np.sqrt(np.mean(ref2 ** 2)) + 1e-30
        worst2 = max(worst2, (np.maximum(np.abs(got2 - ref2) - np.abs(ref2) * 2.0 ** -7, 0)).max() / rms2)
        nflip2 += int((got2 != ref2).sum())
        ntot2 += got2.size
    # one-ulp disagreements must stay rare
    assert nflip1 <= 0.02 * ntot1 and nflip2 <= 0.02 * ntot2, (nflip1, ntot1, nflip2, ntot2)
    ref_out = np.zeros((L.T, out3.shape[2]), np.float32)
    for s in range(L.k):
        ref_out += per_slot[:, s]
    print(f"  stage outputs that differ from the oracle's by a rounding: stage 1 {nflip1} of {ntot1}, "
          f"stage 2 {nflip2} of {ntot2}; worst beyond one bf16 ulp: {worst1:.2e} / {worst2:.2e} of the rms", flush=True)
    flips = _Flips((nflip1, nflip2))
    flips.moved_tokens = moved_tokens
    return worst1, worst2, ref_out, flips


def _end_to_end(got32, ref, ref_given_a2, nflip1):
    """The layer output against the oracle.  Both sides round the stage-1 result to bf16 and re-quantise it to
    MXFP4; two correct fp32 evaluation orders can round a value that sits on a bf16 boundary differently, and
    when that value also sits on an e2m1 boundary the re-quantised activation moves by a whole e2m1 step,
    which shows as an isolated outlier in one output row.  So: the strict bound (max|err| <= 1e-2 * rms,
    cosine >= 0.999) is asserted against the oracle evaluated from the kernel's own stage-1 result (whose
    one-ulp agreement with the oracle's is asserted separately), and against the pure oracle the same bound
    must hold for all but 2e-3 of the elements (one moved activation touches every output channel of its
    row) with no error above 0.1 * rms, and every element beyond the strict bound must belong to a token that
    has such a moved activation (``nflip1.moved_tokens``: the re-quantised stage-1 row differs from the
    oracle's); all other tokens meet the strict bound.  When no stage output was rounded the other way
    (nflip1 == (0, 0)) there is nothing to excuse, and the strict bound is asserted against the pure oracle as well.  The reference's own
    metric, calc_diff <= 0.01 for the MXFP4-activation path (tests/contrib/moe/test_mxfp4.py:286-299), is asserted
    in every case."""
    err_a2, cos_a2 = metrics.max_err_over_rms(got32, ref_given_a2), metrics.cosine(got32, ref_given_a2)
    err, cos = metrics.max_err_over_rms(got32, ref), metrics.cosine(got32, ref)
    rms = np.sqrt(np.mean(ref.astype(np.float64) ** 2))
    frac = float((np.abs(got32 - ref) > TOL_MAX * rms).mean())
    print(f"  vs oracle: max|err|/rms={err:.3e} cosine={cos:.8f} beyond-bound fraction={frac:.2e}; "
          f"given the kernel's a2: max|err|/rms={err_a2:.3e} cosine={cos_a2:.8f}", flush=True)
    cd = metrics.calc_diff(got32, ref)
    print(f"  calc_diff={cd:.3e}; strict bound against the pure oracle "
          f"{'asserted (no stage rounding differs)' if not any(nflip1) else 'relaxed (%d stage-1, %d stage-2 roundings differ): worst %.3e of the 0.1 allowed, fraction %.2e of the 2e-3 allowed' % (nflip1[0], nflip1[1], err, frac)}",
          flush=True)
    assert err_a2 <= TOL_MAX and cos_a2 >= TOL_COS
    assert cd <= 0.01
    if not any(nflip1):
        assert err <= TOL_MAX and cos >= TOL_COS
    else:
        assert cos >= TOL_COS and frac <= 2e-3 and err <= 0.1
        moved = getattr(nflip1, "moved_tokens", None)
        if moved is not None:
            beyond = (np.abs(got32 - ref) > TOL_MAX * rms).any(axis=1)
            print(f"  tokens with a moved activation: {int(moved.sum())}; tokens beyond the strict bound: {int(beyond.sum())}", flush=True)
            assert not (beyond & ~moved).any(), "an outlier in a token whose stage-1 rows re-quantise as the oracle's"
    return err


@pytest.mark.parametrize("name,T,bm,bias", [
    ("tiny", 64, None, False),        # the tiny layer: E=8, top-2, T=64, H=1024, I=512
    ("tiny", 64, 16, False),
    ("tiny", 64, 32, True),
    ("tiny", 5, 16, False),
    ("tiny", 300, 64, False),
    ("tiny", 300, 128, True),
    ("tiny", 300, 256, True),         # 256-row tile: accumulators in hand-numbered accumulation registers
    ("mixtral_s", 700, 256, False),
    # 288-row tile: 72 accumulator tiles (8 of them in ordinary registers), ids ring of two, schedule read from global
    # memory; "odd" has three K-groups in gate_up (persistent) and two in down (one workgroup per tile)
    ("mixtral_s", 700, 288, False), ("odd", 640, 288, True), ("longk_s", 330, 288, True), ("tiny", 300, 288, True),
    ("mixtral_s", 700, 160, False), ("odd", 640, 192, True), ("longk_s", 330, 160, True),
    ("mixtral_s", 33, 32, False),
    ("qwen3_s", 64, 16, False),
    ("qwen3_s", 257, 64, False),
    ("dsv3_s", 16, 16, False),
    ("dsv3_s", 128, None, False),
    ("odd", 77, 32, True),
    ("odd", 500, None, False),
])
def test_fused_moe_matches_oracle(name, T, bm, bias):
    L = cases.make_layer(name, T, seed=0, bias=bias)
    w1, w1s, w2, w2s = cases.device_weights(L)
    tw, ti = torch.from_numpy(L.topk_w).cuda(), torch.from_numpy(L.topk_ids).cuda()
    b1 = None if L.bias1 is None else L.bias1.cuda()
    b2 = None if L.bias2 is None else L.bias2.cuda()
    print(f"fused_moe case {name} T={T} bm={bm} bias={bias}", flush=True)
    out32, parts = fused_moe(L.hidden.cuda(), w1, w2, tw, ti, w1_scale=w1s, w2_scale=w2s, block_size_M=bm,
                             bias1=b1, bias2=b2, dtype=torch.float32, return_parts=True, method="a4w4")
    out16 = fused_moe(L.hidden.cuda(), w1, w2, tw, ti, w1_scale=w1s, w2_scale=w2s, block_size_M=bm,
                      bias1=b1, bias2=b2, method="a4w4")
    torch.cuda.synchronize()
    assert out16.dtype == torch.bfloat16 and out16.shape == (T, L.H)

    # activation quantisation: bit-exact
    oq, os_ = om.quantize_mxfp4(_f(L.hidden))
    assert (parts["a1_q"].cpu().numpy() == oq).all()
    assert (cases.untranspose_act_scales(parts["a1_s"].cpu().numpy(), L.H) == os_).all()

    # the quantised copy of the stage-1 result written by the GEMM epilogue is what the stand-alone quantiser
    # makes of the bf16 copy, bit for bit
    nv = int(parts["num_valid_ids"][0])
    q2, s2 = act_quant_mxfp4(parts["a2"][:nv].contiguous())
    assert torch.equal(parts["a2_q"][:nv], q2) and torch.equal(parts["a2_s"][:nv], s2)
    oq2, os2 = om.quantize_mxfp4(_f(parts["a2"][:nv]))
    assert (q2.cpu().numpy() == oq2).all() and (cases.untranspose_act_scales(s2.cpu().numpy(), L.I) == os2).all()

    # stage-wise, each stage fed the kernel's own previous output
    w1e, w2e, ref_a2, nflip1 = _stage_checks(L, parts, parts["block_m"])
    assert w1e <= TOL_MAX, f"stage 1 (max|err| - ulp)/rms = {w1e}"
    assert w2e <= TOL_MAX, f"stage 2 (max|err| - ulp)/rms = {w2e}"

    # end to end
    ref = moe.moe_ref(_f(L.hidden), L.w1q, L.w1s, L.w2q, L.w2s, L.topk_w, L.topk_ids, act="a4",
                      bias1=None if L.bias1 is None else _f(L.bias1), bias2=None if L.bias2 is None else _f(L.bias2))
    rms = np.sqrt(np.mean(ref.astype(np.float64) ** 2))
    got32 = _f(out32)
    _end_to_end(got32, ref, ref_a2, nflip1)
    half_ulp = np.abs(ref_a2) * 2.0 ** -8
    assert (np.abs(_f(out16) - ref_a2) <= TOL_MAX * rms + half_ulp).all()
    # the bf16 output is the rounding of the fp32 output
    assert (_f(out16) == om.bf16_round(got32)).all()


@pytest.mark.parametrize("T,bm,bias", [(48, 16, True), (400, 128, True), (129, None, False)])
def test_padded_shape_matches_oracle(T, bm, bias):
    """hidden = inter = 1440 (gpt-oss / 2): weights zero-padded to 1536, hidden_pad / intermediate_pad passed
    as the reference's signature defines them; the oracle runs on the unpadded problem."""
    L = cases.make_layer("gptoss_s", T, seed=3, bias=bias)
    w1, w1s, w2, w2s, b1, b2, hp, ip = cases.padded_device_weights(L)
    assert (hp, ip) == (96, 96)
    tw, ti = torch.from_numpy(L.topk_w).cuda(), torch.from_numpy(L.topk_ids).cuda()
    print(f"padded case T={T} bm={bm} bias={bias}", flush=True)
    kw = dict(w1_scale=w1s, w2_scale=w2s, block_size_M=bm, bias1=b1, bias2=b2, hidden_pad=hp, intermediate_pad=ip,
              dtype=torch.float32, method="a4w4")
    out_narrow, parts = fused_moe(L.hidden.cuda(), w1, w2, tw, ti, return_parts=True, **kw)   # activations at the true width
    wide = torch.nn.functional.pad(L.hidden, (0, hp)).cuda()
    out_wide = fused_moe(wide, w1, w2, tw, ti, **kw)                                    # the reference's convention
    torch.cuda.synchronize()
    assert out_narrow.shape == (T, L.H) and out_wide.shape == (T, L.H + hp)
    assert (_f(out_wide)[:, L.H:] == 0).all()                                           # padded channels stay zero
    assert (_f(out_wide)[:, :L.H] == _f(out_narrow)).all()
    ref = moe.moe_ref(_f(L.hidden), L.w1q, L.w1s, L.w2q, L.w2s, L.topk_w, L.topk_ids, act="a4",
                      bias1=None if L.bias1 is None else _f(L.bias1), bias2=None if L.bias2 is None else _f(L.bias2))
    # stage-wise on the unpadded part of the intermediates (the padded columns must be exactly zero)
    nv = int(parts["num_valid_ids"][0])                   # rows past the padded total are never written
    assert (_f(parts["a2"])[:nv, L.I:] == 0).all() and (_f(parts["out3"])[:, :, L.H:] == 0).all()
    view = dict(parts, a2=parts["a2"][:, :L.I], out3=parts["out3"][:, :, :L.H])
    w1e, w2e, ref_a2, nflip1 = _stage_checks(L, view, parts["block_m"])
    assert w1e <= TOL_MAX and w2e <= TOL_MAX
    _end_to_end(_f(out_narrow), ref, ref_a2, nflip1)


@pytest.mark.parametrize("T,bm", [(24, 16), (90, 32), (150, 64), (300, 128), (500, 288)])
def test_padding_is_left_unfetched_and_changes_nothing(T, bm):
    """hidden 1376 and inter 1312 padded to 1536: the last K-step of 128 columns is all padding in both GEMMs, and so are
    whole waves' weight rows.  Told the pads, the GEMMs leave that part of the weights unfetched (the 16- and 32-row tiles
    also the K-step); the padding being zeros, the result must equal, bit for bit, the one computed with the padded
    sizes passed off as real ones (pads 0, everything fetched), in the one-call path and step by step, and must match
    the oracle on the unpadded problem."""
    L = cases.make_layer("gptoss_s", T, seed=5, bias=True, H=1376, I=1312)
    w1, w1s, w2, w2s, b1, b2, hp, ip = cases.padded_device_weights(L)
    assert (hp, ip) == (160, 224)
    tw, ti = torch.from_numpy(L.topk_w).cuda(), torch.from_numpy(L.topk_ids).cuda()
    print(f"unfetched-padding case T={T} bm={bm}", flush=True)
    kw = dict(w1_scale=w1s, w2_scale=w2s, block_size_M=bm, bias1=b1, bias2=b2, dtype=torch.float32, method="a4w4")
    wide = torch.nn.functional.pad(L.hidden, (0, hp)).cuda()
    told = fused_moe(wide, w1, w2, tw, ti, hidden_pad=hp, intermediate_pad=ip, **kw)
    told_steps, parts = fused_moe(wide, w1, w2, tw, ti, hidden_pad=hp, intermediate_pad=ip, return_parts=True, **kw)
    untold = fused_moe(wide, w1, w2, tw, ti, **kw)
    torch.cuda.synchronize()
    assert told.shape == (T, L.H + hp) and torch.equal(told, untold) and torch.equal(told_steps, untold)
    assert (_f(told)[:, L.H:] == 0).all()
    nv = int(parts["num_valid_ids"][0])
    assert (_f(parts["a2"])[:nv, L.I:] == 0).all() and (_f(parts["out3"])[:, :, L.H:] == 0).all()
    ref = moe.moe_ref(_f(L.hidden), L.w1q, L.w1s, L.w2q, L.w2s, L.topk_w, L.topk_ids, act="a4", bias1=_f(L.bias1),
                      bias2=_f(L.bias2))
    view = dict(parts, a2=parts["a2"][:, :L.I], out3=parts["out3"][:, :, :L.H])
    w1e, w2e, ref_a2, nflip1 = _stage_checks(L, view, parts["block_m"])
    assert w1e <= TOL_MAX and w2e <= TOL_MAX
    _end_to_end(_f(told)[:, :L.H], ref, ref_a2, nflip1)


@pytest.mark.parametrize("T,bm", [(24, 16), (300, 128), (500, 288)])
def test_padded_weight_rows_are_not_read(T, bm):
    """Whether the kernels really leave the padding alone: hidden 1408 (22 x 64) and inter 1312 (41 x 32) padded to
    1536, and the weight rows of the padding (whole waves' worth in both GEMMs) filled with ones instead of zeros,
    which a caller must not do.  Told the pads, the GEMMs do not fetch those rows: the padded columns of a2, out3 and
    the output are exact zeros and everything equals the run on clean weights.  Not told, the ones show up."""
    from oracle import layout
    from pyhip_amd import mxfp4 as pm
    L = cases.make_layer("gptoss_s", T, seed=6, H=1408, I=1312)
    t = torch.from_numpy
    w1q, w1s, w2q, w2s, _, _, hp, ip = pm.pad_layer_weights(t(L.w1q), t(L.w1s), t(L.w2q), t(L.w2s))
    assert (hp, ip) == (128, 224)
    E, H, I, Hp, Ip = L.E, L.H, L.I, L.H + hp, L.I + ip

    def device(w1q, w1s, w2q, w2s):
        w1 = t(layout.shuffle_weight(w1q.numpy())).cuda()
        w2 = t(layout.shuffle_weight(w2q.numpy())).cuda()
        s1 = t(layout.e8m0_shuffle(w1s.numpy().reshape(E * 2 * Ip, Hp // 32))).cuda()
        s2 = t(layout.e8m0_shuffle(w2s.numpy().reshape(E * Hp, Ip // 32))).cuda()
        w1.is_shuffled = w2.is_shuffled = True
        return w1, s1, w2, s2

    clean = device(w1q, w1s, w2q, w2s)
    d1q, d1s, d2q, d2s = w1q.clone(), w1s.clone(), w2q.clone(), w2s.clone()
    for lo, hi in ((I, Ip), (Ip + I, 2 * Ip)):            # the padding rows of the gate half and of the up half
        d1q[:, lo:hi, : H // 2] = 0x22                      # e2m1 pairs (1.0, 1.0), over the real columns
        d1s[:, lo:hi, : H // 32] = 127                      # scale 2^0
    d2q[:, H:, : I // 2] = 0x22
    d2s[:, H:, : I // 32] = 127
    dirty = device(d1q, d1s, d2q, d2s)
    tw, ti = t(L.topk_w).cuda(), t(L.topk_ids).cuda()
    wide = torch.nn.functional.pad(L.hidden, (0, hp)).cuda()
    print(f"unread-padding case T={T} bm={bm}", flush=True)

    def run(w, **pads):
        w1, s1, w2, s2 = w
        return fused_moe(wide, w1, w2, tw, ti, w1_scale=s1, w2_scale=s2, block_size_M=bm, dtype=torch.float32, method="a4w4",
                         return_parts=True, **pads)

    want, pw = run(clean, hidden_pad=hp, intermediate_pad=ip)
    got, pg = run(dirty, hidden_pad=hp, intermediate_pad=ip)
    seen, ps = run(dirty)
    one_call = fused_moe(wide, dirty[0], dirty[2], tw, ti, w1_scale=dirty[1], w2_scale=dirty[3], block_size_M=bm,
                         dtype=torch.float32, method="a4w4", hidden_pad=hp, intermediate_pad=ip)
    torch.cuda.synchronize()
    nv = int(pg["num_valid_ids"][0])
    assert torch.equal(got, want) and torch.equal(one_call, want)
    assert (got[:, H:] == 0).all() and (_f(pg["a2"])[:nv, I:] == 0).all() and (_f(pg["out3"])[:, :, H:] == 0).all()
    assert torch.equal(pg["a2"][:nv], pw["a2"][:nv]) and torch.equal(pg["out3"], pw["out3"])
    # the poison is there to be seen by kernels that fetch everything
    assert (_f(ps["a2"])[:nv, I:] != 0).any() and (seen[:, H:] != 0).any()
    assert torch.equal(seen[:, :H], want[:, :H])


@pytest.mark.parametrize("name,T,bm,bias,splitk", [
    ("tiny", 64, 16, False, 1), ("tiny", 5, 16, True, 0), ("tiny", 200, 64, False, 1), ("mixtral_s", 33, 32, False, 1),
    ("qwen3_s", 64, 16, False, 1), ("dsv3_s", 16, None, False, 1), ("dsv3_s", 128, None, True, 1),
    ("tiny", 64, 16, True, 4), ("tiny", 200, 64, False, 4), ("mixtral_s", 33, 32, False, 4), ("dsv3_s", 16, None, False, 4),
    ("gptoss_s1", 20, 16, True, 4),
    ("odd", 9, 16, False, 0), ("odd", 77, 32, True, 1),
    ("longk_s", 3, 16, True, 16), ("longk_s", 40, 16, False, 16), ("longk_s", 3, 16, False, 4),
    ("longk_s", 3, 16, True, 32), ("longk_s", 40, 16, False, 32), ("verylongk_s", 2, 16, True, 32), ("verylongk_s", 1, 16, False, 0),
    ("verylongk_s", 20, 16, True, 0),
])
def test_w4a16_matches_oracle(name, T, bm, bias, splitk):
    """bf16 activations x MXFP4 weights (method="w4a16") against the oracle's "a16" path:
    max|err| <= 1e-2 * rms(ref), cosine >= 0.999; the stage-1 result within one bf16 ulp."""
    L = cases.make_layer(name, T, seed=1, bias=bias)
    w1, w1s, w2, w2s = cases.device_weights(L)
    tw, ti = torch.from_numpy(L.topk_w).cuda(), torch.from_numpy(L.topk_ids).cuda()
    b1 = None if L.bias1 is None else L.bias1.cuda()
    b2 = None if L.bias2 is None else L.bias2.cuda()
    print(f"w4a16 case {name} T={T} bm={bm} bias={bias} splitk={splitk}", flush=True)
    out32, parts = fused_moe(L.hidden.cuda(), w1, w2, tw, ti, w1_scale=w1s, w2_scale=w2s, block_size_M=bm,
                             bias1=b1, bias2=b2, dtype=torch.float32, method="w4a16", return_parts=True, splitk=splitk)
    torch.cuda.synchronize()
    ref, a2_ref, slot_ref = moe.moe_ref(_f(L.hidden), L.w1q, L.w1s, L.w2q, L.w2s, L.topk_w, L.topk_ids, act="a16",
                                 bias1=None if L.bias1 is None else _f(L.bias1),
                                 bias2=None if L.bias2 is None else _f(L.bias2), return_parts=True)
    # stage 1: a2[sorted position] against the oracle's a2[token, slot]
    so = parts["sorted_ids"].cpu().numpy().view(np.uint32)
    nv = int(parts["num_valid_ids"][0])
    tok, slot = (so[:nv] & 0xFFFFFF).astype(np.int64), (so[:nv] >> 24).astype(np.int64)
    okm = slot < L.k
    got_a2 = _f(parts["a2"])[:nv]
    want = a2_ref[tok[okm], slot[okm]]
    rms1 = np.sqrt(np.mean(want.astype(np.float64) ** 2))
    assert (np.abs(got_a2[okm] - want) <= TOL_MAX * rms1 + np.abs(want) * 2.0 ** -7).all()
    assert (got_a2[~okm] == 0).all()
    # every (token, slot) output is rounded to bf16 before the slots are summed (the kernel's and the oracle's
    # fp32 values differ in the last bits, so a rounding may go the other way): one bf16 ulp of each slot value
    # on top of the bound
    rms = np.sqrt(np.mean(ref.astype(np.float64) ** 2))
    ulp = np.abs(slot_ref).sum(axis=1) * 2.0 ** -7
    excess = np.maximum(np.abs(_f(out32) - ref) - ulp, 0).max() / rms
    err, cos = metrics.max_err_over_rms(_f(out32), ref), metrics.cosine(_f(out32), ref)
    # The allowance is needed because a slot value near 3 * rms carries a bf16 ulp of 2^-7 * 3 * rms = 2.3e-2 * rms
    # by itself: one rounding that goes the other way already exceeds 1e-2 * rms, with both sides correct.  It is
    # only ever used by a vanishing fraction of the elements, which is asserted (and printed) here.
    beyond = float((np.abs(_f(out32) - ref) > TOL_MAX * rms).mean())
    cd = metrics.calc_diff(_f(out32), ref)
    print(f"  max|err|/rms={err:.3e} (beyond the rounding allowance: {excess:.3e}; fraction of elements beyond the "
          f"strict bound: {beyond:.2e}) cosine={cos:.8f} calc_diff={cd:.3e}", flush=True)
    assert excess <= TOL_MAX and cos >= TOL_COS and beyond <= 1e-3 and cd <= 0.01


@pytest.mark.parametrize("method,limit,T", [("a4w4", None, 300), ("a4w4", 1.0, 37), ("w4a16", None, 20), ("w4a16", 0.5, 20)])
def test_swiglu_matches_oracle(method, limit, T):
    """gpt-oss's clamped SwiGLU (activation=ActivationType.Swiglu) with biases on the gpt-oss-like padded shape,
    against the oracle: stage-1 result within 1e-2 * rms + one bf16 ulp, layer output max|err| <= 1e-2 * rms(ref)
    beyond the bf16 rounding allowance of the slot values, cosine >= 0.999.  A small limit puts most values on
    the clamps."""
    from pyhip_amd.enums import ActivationType
    L = cases.make_layer("gptoss_s", T, seed=4, bias=True)
    w1, w1s, w2, w2s, b1, b2, hp, ip = cases.padded_device_weights(L)
    tw, ti = torch.from_numpy(L.topk_w).cuda(), torch.from_numpy(L.topk_ids).cuda()
    print(f"swiglu case method={method} limit={limit} T={T}", flush=True)
    out32, parts = fused_moe(L.hidden.cuda(), w1, w2, tw, ti, w1_scale=w1s, w2_scale=w2s, bias1=b1, bias2=b2,
                             hidden_pad=hp, intermediate_pad=ip, dtype=torch.float32, method=method,
                             activation=ActivationType.Swiglu, swiglu_limit=limit, return_parts=True)
    torch.cuda.synchronize()
    ref, a2_ref, slot_ref = moe.moe_ref(_f(L.hidden), L.w1q, L.w1s, L.w2q, L.w2s, L.topk_w, L.topk_ids,
                                        act="a4" if method == "a4w4" else "a16", bias1=_f(L.bias1), bias2=_f(L.bias2),
                                        return_parts=True, activation="swiglu", swiglu_limit=limit)
    silu_ref = moe.moe_ref(_f(L.hidden), L.w1q, L.w1s, L.w2q, L.w2s, L.topk_w, L.topk_ids,
                           act="a4" if method == "a4w4" else "a16", bias1=_f(L.bias1), bias2=_f(L.bias2))
    so = parts["sorted_ids"].cpu().numpy().view(np.uint32)
    nv = int(parts["num_valid_ids"][0])
    tok, slot = (so[:nv] & 0xFFFFFF).astype(np.int64), (so[:nv] >> 24).astype(np.int64)
    okm = slot < L.k
    got_a2 = _f(parts["a2"])[:nv]
    assert (got_a2[:, L.I:] == 0).all() and (got_a2[~okm] == 0).all()          # padded channels and rows stay zero
    want = a2_ref[tok[okm], slot[okm]]
    rms1 = np.sqrt(np.mean(want.astype(np.float64) ** 2))
    assert (np.abs(got_a2[okm][:, :L.I] - want) <= TOL_MAX * rms1 + np.abs(want) * 2.0 ** -7).all()
    rms = np.sqrt(np.mean(ref.astype(np.float64) ** 2))
    got = _f(out32)
    cos = metrics.cosine(got, ref)
    if method == "w4a16":
        ulp = np.abs(slot_ref).sum(axis=1) * 2.0 ** -7
        excess = np.maximum(np.abs(got - ref) - ulp, 0).max() / rms
        print(f"  beyond the rounding allowance: {excess:.3e} cosine={cos:.8f}", flush=True)
        assert excess <= TOL_MAX
    else:
        # the MXFP4 re-quantisation of the stage-1 result can flip a code where kernel and oracle differ in the
        # last bit: a few isolated outliers, bounded
        err = np.abs(got - ref) / rms
        print(f"  max|err|/rms={err.max():.3e} outliers={np.mean(err > TOL_MAX):.2e} cosine={cos:.8f}", flush=True)
        assert np.mean(err > TOL_MAX) <= 2e-3 and err.max() <= 0.1
    assert cos >= TOL_COS
    assert metrics.cosine(got, silu_ref) < 0.99                                 # and it is not SiLU
    if method == "a4w4":
        # the eight-wave tile with both operands through LDS has its own instance of this epilogue: same bits
        kw = dict(w1_scale=w1s, w2_scale=w2s, bias1=b1, bias2=b2, hidden_pad=hp, intermediate_pad=ip, dtype=torch.float32,
                  method=method, activation=ActivationType.Swiglu, swiglu_limit=limit)
        assert torch.equal(fused_moe(L.hidden.cuda(), w1, w2, tw, ti, operand_staging="lds", **kw), out32)


def test_prepared_weight_file_feeds_the_operator(tmp_path):
    """pyhip_amd.prepare_weights: float weights -> file -> operator arguments; same bytes and same output as the
    weights the other tests build by hand (padded gpt-oss-like shape with biases)."""
    from pyhip_amd import prepare_weights as pw
    L = cases.make_layer("gptoss_s", 20, seed=6, bias=True)
    w1f = torch.from_numpy(om.dequantize_mxfp4(L.w1q, L.w1s))          # exactly representable: quantising again is the identity
    w2f = torch.from_numpy(om.dequantize_mxfp4(L.w2q, L.w2s))
    path = str(tmp_path / "layer.safetensors")
    pw.save(path, *pw.convert(w1f, w2f, L.bias1, L.bias2))
    tensors, meta = pw.load(path, device="cuda")
    (w1, w2), kw = pw.fused_moe_kwargs(tensors, meta)
    r1, r1s, r2, r2s, b1, b2, hp, ip = cases.padded_device_weights(L)
    assert (hp, ip) == (meta["hidden_pad"], meta["intermediate_pad"])
    assert torch.equal(w1, r1) and torch.equal(w2, r2) and torch.equal(kw["w1_scale"], r1s) and torch.equal(kw["w2_scale"], r2s)
    tw, ti = torch.from_numpy(L.topk_w).cuda(), torch.from_numpy(L.topk_ids).cuda()
    print("prepared-weights case gptoss_s T=20", flush=True)
    out = fused_moe(L.hidden.cuda(), w1, w2, tw, ti, **kw)
    ref = fused_moe(L.hidden.cuda(), r1, r2, tw, ti, w1_scale=r1s, w2_scale=r2s, bias1=b1, bias2=b2, hidden_pad=hp,
                    intermediate_pad=ip)
    torch.cuda.synchronize()
    assert torch.equal(out, ref) and torch.isfinite(out.float()).all()


def test_auto_dispatch():
    """method="auto": bf16 activations for the smallest calls (see pick_w4a16), MXFP4 activations above"""
    L = cases.make_layer("dsv3_s", 1, seed=2)             # 8 pairs over 64 experts
    w1, w1s, w2, w2s = cases.device_weights(L)
    tw, ti = torch.from_numpy(L.topk_w).cuda(), torch.from_numpy(L.topk_ids).cuda()
    kw = dict(w1_scale=w1s, w2_scale=w2s)
    auto = fused_moe(L.hidden.cuda(), w1, w2, tw, ti, **kw)
    assert torch.equal(auto, fused_moe(L.hidden.cuda(), w1, w2, tw, ti, method="w4a16", **kw))
    L = cases.make_layer("tiny", 64, seed=2)              # 64 * 2 / 8 = 16 rows per expert
    w1, w1s, w2, w2s = cases.device_weights(L)
    tw, ti = torch.from_numpy(L.topk_w).cuda(), torch.from_numpy(L.topk_ids).cuda()
    kw = dict(w1_scale=w1s, w2_scale=w2s)
    auto = fused_moe(L.hidden.cuda(), w1, w2, tw, ti, **kw)
    assert torch.equal(auto, fused_moe(L.hidden.cuda(), w1, w2, tw, ti, method="a4w4", **kw))


@pytest.mark.parametrize("name,T,method", [("dsv3_s", 16, "w4a16"), ("tiny", 300, "a4w4"), ("dsv3_s", 1, "w4a16")])
def test_graph_capture_replays(name, T, method):
    """The whole layer is enqueue-only (no host synchronisation, no memset nodes), so it can be captured in a
    HIP graph; every replay, with the inputs rewritten in place and eager work in between, must reproduce the
    eager result bit for bit."""
    L = cases.make_layer(name, T, seed=4)
    w1, w1s, w2, w2s = cases.device_weights(L)
    hidden = L.hidden.cuda()
    tw, ti = torch.from_numpy(L.topk_w).cuda(), torch.from_numpy(L.topk_ids).cuda()
    kw = dict(w1_scale=w1s, w2_scale=w2s, method=method)
    print(f"graph case {name} T={T} method={method}", flush=True)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):                       # warm-up outside the capture
        fused_moe(hidden, w1, w2, tw, ti, **kw)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out_g = fused_moe(hidden, w1, w2, tw, ti, **kw)
    g = torch.Generator().manual_seed(11)
    for rep in range(3):
        hidden.copy_((torch.randn(T, L.H, generator=g)).to(torch.bfloat16))
        perm = torch.randperm(T, generator=g)
        # a different routing on every replay (one token: its experts shifted, which keeps them distinct)
        ti.copy_((torch.from_numpy(L.topk_ids)[perm] + (3 * (rep + 1) if T == 1 else 0)) % L.E)
        tw.copy_(torch.from_numpy(L.topk_w)[perm])
        graph.replay()
        torch.cuda.synchronize()
        got = out_g.clone()
        eager = fused_moe(hidden, w1, w2, tw, ti, **kw)  # eager work between the replays
        torch.cuda.synchronize()
        assert torch.equal(got, eager), f"replay {rep}"


@pytest.mark.parametrize("method,T", [("a4w4", 200), ("w4a16", 6)])
def test_expert_mask_and_local_tokens(method, T):
    """Expert-parallel use of the call surface (src/contrib/fused_moe.py:134): with ``expert_mask`` a rank holds
    the weights of its experts only and the sort hands out local expert ids; slots routed elsewhere contribute
    nothing.  Every (token, slot) a rank owns must come out bit for bit as in the run that holds all experts,
    and the ranks' fp32 outputs must add up to the full output.  ``num_local_tokens`` (a device scalar) limits
    the tokens that take part without changing any launch shape."""
    L = cases.make_layer("dsv3_s", T, seed=5)
    w1, w1s, w2, w2s = cases.device_weights(L)
    hidden = L.hidden.cuda()
    tw, ti = torch.from_numpy(L.topk_w).cuda(), torch.from_numpy(L.topk_ids).cuda()
    E, N1, I = L.E, w1.shape[1], L.I
    print(f"expert-mask case dsv3_s T={T} method={method}", flush=True)
    full, pf = fused_moe(hidden, w1, w2, tw, ti, w1_scale=w1s, w2_scale=w2s, dtype=torch.float32,
                         return_parts=True, method=method, block_size_M=16)
    total = torch.zeros_like(full)
    # scale rows are grouped per expert: [E * N, ...] with N a multiple of 32, so an expert's rows can be selected
    s1 = w1s.view(E, -1)
    s2 = w2s.view(E, -1)
    for parity in (0, 1):
        mask = torch.tensor([(e % 2) == parity for e in range(E)], dtype=torch.int32, device="cuda")
        keep = mask.bool()
        w1k, w2k = w1[keep].contiguous(), w2[keep].contiguous()
        w1k.is_shuffled = w2k.is_shuffled = True
        out, p = fused_moe(hidden, w1k, w2k, tw, ti, expert_mask=mask,
                           w1_scale=s1[keep].contiguous().view(-1, w1s.shape[-1]),
                           w2_scale=s2[keep].contiguous().view(-1, w2s.shape[-1]),
                           dtype=torch.float32, return_parts=True, method=method, block_size_M=16)
        torch.cuda.synchronize()
        mine = keep[ti.long()]                                   # [T, k]
        assert torch.equal(p["out3"][mine], pf["out3"][mine])      # (slots owned elsewhere are never written nor read)
        total += out
    assert torch.allclose(total, full, rtol=1e-5, atol=1e-6)

    n_local = T // 2 + 1
    nl = torch.tensor([n_local], dtype=torch.int32, device="cuda")
    out = fused_moe(hidden, w1, w2, tw, ti, w1_scale=w1s, w2_scale=w2s, dtype=torch.float32, num_local_tokens=nl,
                    method=method, block_size_M=16)
    torch.cuda.synchronize()
    assert torch.equal(out[:n_local], full[:n_local])
    assert (out[n_local:] == 0).all()


@pytest.mark.parametrize("name,bias,swiglu", [("mixtral_s", False, False), ("dsv3_s", True, False), ("tiny", True, True),
                                              ("longk_s", False, False), ("verylongk_s", True, False)])
def test_single_token_skips_the_sort(name, bias, swiglu):
    """One token with bf16 activations: the layer call runs no sort, the GEMMs read topk_ids / topk_weights themselves
    (pyhip_moe_gemm{1,2}_w4a16_token).  The result must equal the sorted, step-by-step path bit for bit (which the
    other tests hold against the oracle): plain, with an out-of-range id, under an expert mask with the rank's own
    weights only (local expert numbering), and with num_local_tokens 0 and 1; also on poisoned intermediates."""
    from pyhip_amd.enums import ActivationType
    L = cases.make_layer(name, 1, seed=41, bias=bias)
    w1, w1s, w2, w2s = cases.device_weights(L)
    hidden = L.hidden.cuda()
    tw = torch.from_numpy(L.topk_w).cuda()
    b1 = None if L.bias1 is None else L.bias1.cuda()
    b2 = None if L.bias2 is None else L.bias2.cuda()
    act = dict(activation=ActivationType.Swiglu, swiglu_limit=7.0) if swiglu else {}
    E = L.E
    s1, s2 = w1s.view(E, -1), w2s.view(E, -1)
    print(f"single-token case {name} bias={bias} swiglu={swiglu}", flush=True)
    ids_plain = L.topk_ids.copy()
    ids_hole = ids_plain.copy()
    ids_hole[0, 0] = E + 3                                      # a slot whose expert lives elsewhere
    ran = 0
    for ids in (ids_plain, ids_hole):
        ti = torch.from_numpy(ids).cuda()
        for masked in (False, True):
            kw = dict(w1_scale=w1s, w2_scale=w2s, bias1=b1, bias2=b2, method="w4a16", **act)
            wa, wb = w1, w2
            if masked:
                # the rank holds every expert but the one of the token's last slot, and none beyond the 3/4 mark
                mask = torch.ones(E, dtype=torch.int32)
                mask[int(L.topk_ids[0, -1])] = 0
                mask[(3 * E) // 4:] = 0
                if int(mask[torch.from_numpy(ids_plain[0]).long().clamp(0, E - 1)].sum()) == 0:
                    mask[int(L.topk_ids[0, 0])] = 1
                keep = mask.bool().cuda()
                wa, wb = w1[keep].contiguous(), w2[keep].contiguous()
                wa.is_shuffled = wb.is_shuffled = True
                kw.update(expert_mask=mask.cuda(), w1_scale=s1[keep].contiguous().view(-1, w1s.shape[-1]),
                          w2_scale=s2[keep].contiguous().view(-1, w2s.shape[-1]),
                          bias1=None if b1 is None else b1[keep].contiguous(), bias2=None if b2 is None else b2[keep].contiguous())
            for nl in (None, 1, 0):
                if nl is not None:
                    kw["num_local_tokens"] = torch.tensor([nl], dtype=torch.int32, device="cuda")
                for dt in (torch.float32, torch.bfloat16):
                    want = fused_moe(hidden, wa, wb, tw, ti, dtype=dt, return_parts=True, **kw)[0]
                    _poison_allocator(8 << 20)
                    got = fused_moe(hidden, wa, wb, tw, ti, dtype=dt, **kw)
                    torch.cuda.synchronize()
                    assert torch.isfinite(got.float()).all() and torch.equal(got, want), (masked, nl, dt)
                    if nl == 0:
                        assert (got == 0).all()
                    ran += 1
    assert ran == 24


@pytest.mark.parametrize("method", ["a4w4", "w4a16"])
def test_strided_hidden_states(method):
    """hidden_states may be a column slice of a wider tensor (row stride larger than the hidden size): the result
    is that of the contiguous copy, bit for bit"""
    L = cases.make_layer("tiny", 40, seed=9)
    w1, w1s, w2, w2s = cases.device_weights(L)
    tw, ti = torch.from_numpy(L.topk_w).cuda(), torch.from_numpy(L.topk_ids).cuda()
    wide = torch.zeros(40, L.H + 256, dtype=torch.bfloat16, device="cuda")
    wide[:, :L.H] = L.hidden.cuda()
    view = wide[:, :L.H]
    assert not view.is_contiguous()
    print(f"strided hidden case method={method}", flush=True)
    a = fused_moe(view, w1, w2, tw, ti, w1_scale=w1s, w2_scale=w2s, method=method)
    b = fused_moe(view.contiguous(), w1, w2, tw, ti, w1_scale=w1s, w2_scale=w2s, method=method)
    torch.cuda.synchronize()
    assert torch.equal(a, b)


@pytest.mark.parametrize("name,T,method,bias", [("tiny", 64, "a4w4", True), ("tiny", 5, "w4a16", True),
                                                ("dsv3_s", 300, "a4w4", False), ("odd", 40, "auto", False)])
def test_one_call_path_equals_the_step_by_step_path(name, T, method, bias):
    """Without ``return_parts`` / ``stage_events`` the operator is a single pyhip_moe_forward call with one workspace;
    with them it runs the entry points one by one with separate buffers.  Same kernels, same order: same bits, with
    and without an expert mask and a local token count."""
    L = cases.make_layer(name, T, seed=12, bias=bias)
    w1, w1s, w2, w2s = cases.device_weights(L)
    tw, ti = torch.from_numpy(L.topk_w).cuda(), torch.from_numpy(L.topk_ids).cuda()
    b1 = None if L.bias1 is None else L.bias1.cuda()
    b2 = None if L.bias2 is None else L.bias2.cuda()
    kw = dict(w1_scale=w1s, w2_scale=w2s, bias1=b1, bias2=b2, method=method)
    print(f"one-call case {name} T={T} method={method} bias={bias}", flush=True)
    hidden = L.hidden.cuda()
    for dt in (None, torch.float32):
        a = fused_moe(hidden, w1, w2, tw, ti, dtype=dt, **kw)
        b, _ = fused_moe(hidden, w1, w2, tw, ti, dtype=dt, return_parts=True, **kw)
        torch.cuda.synchronize()
        assert torch.equal(a, b)
    nl = torch.tensor([T // 2], dtype=torch.int32, device="cuda")
    a = fused_moe(hidden, w1, w2, tw, ti, num_local_tokens=nl, **kw)
    b, _ = fused_moe(hidden, w1, w2, tw, ti, num_local_tokens=nl, return_parts=True, **kw)
    torch.cuda.synchronize()
    assert torch.equal(a, b) and (a[T // 2:] == 0).all()


def _poison_allocator(nbytes):
    """NaN patterns into memory the caching allocator will hand out next, so that anything read without having
    been written shows"""
    junk = torch.full((nbytes // 2,), float("nan"), dtype=torch.bfloat16, device="cuda")
    torch.cuda.synchronize()
    del junk


@pytest.mark.parametrize("method,T,one_call", [("a4w4", 90, True), ("a4w4", 90, False), ("w4a16", 7, True), ("w4a16", 7, False)])
def test_dropped_pairs_contribute_exactly_zero(method, T, one_call):
    """Ids outside [0, E) (a -1 or E sentinel for experts held elsewhere, the router's 0x7FFFFFFF for a NaN row) are
    dropped by the sort, with no expert mask given: their slots are never written by the down GEMM and must
    contribute exactly nothing, whatever the intermediate buffers held before.  The result equals the run in which
    those slots carry a valid id and weight 0 ... except that no product is formed at all: compare with the
    oracle, and bit for bit with the same call on buffers that held other garbage."""
    L = cases.make_layer("dsv3_s", T, seed=21)
    w1, w1s, w2, w2s = cases.device_weights(L)
    ids = L.topk_ids.copy()
    rng = np.random.default_rng(5)
    drop = rng.random(ids.shape) < 0.3
    ids[drop] = rng.choice(np.array([-1, L.E, L.E + 7, 0x7FFFFFFF], dtype=np.int64), size=int(drop.sum())).astype(np.int32)
    ids[0, :] = -1                                               # a token with no expert at all: a zero row
    tw, ti = torch.from_numpy(L.topk_w).cuda(), torch.from_numpy(ids).cuda()
    print(f"dropped-pairs case dsv3_s T={T} method={method} one_call={one_call}", flush=True)
    kw = dict(w1_scale=w1s, w2_scale=w2s, dtype=torch.float32, method=method, block_size_M=16)
    outs = []
    for fill in (0, 1):
        _poison_allocator(64 << 20) if fill else torch.zeros(32 << 20, dtype=torch.uint8, device="cuda")
        o = fused_moe(L.hidden.cuda(), w1, w2, tw, ti, **kw) if one_call else \
            fused_moe(L.hidden.cuda(), w1, w2, tw, ti, return_parts=True, **kw)[0]
        torch.cuda.synchronize()
        outs.append(o.clone())
    assert torch.isfinite(outs[1]).all() and torch.equal(outs[0], outs[1])
    assert (outs[1][0] == 0).all()
    ref = moe.moe_ref(_f(L.hidden), L.w1q, L.w1s, L.w2q, L.w2s, L.topk_w, ids, act="a4" if method == "a4w4" else "a16")
    rms = np.sqrt(np.mean(ref.astype(np.float64) ** 2))
    err = np.abs(_f(outs[1]) - ref) / rms
    print(f"  max|err|/rms={err.max():.3e} beyond-bound fraction={np.mean(err > TOL_MAX):.2e}", flush=True)
    assert np.mean(err > TOL_MAX) <= 2e-3 and err.max() <= 0.1 and metrics.cosine(_f(outs[1]), ref) >= TOL_COS


@pytest.mark.parametrize("name,T,method,bm", [("tiny", 300, "a4w4", None), ("dsv3_s", 40, "a4w4", 16), ("dsv3_s", 6, "w4a16", None)])
def test_shared_expert_as_an_extra_slot(name, T, method, bm):
    """A shared expert stored behind the routed ones and appended to the routing as slot k
    (pyhip_amd.routing.append_shared_experts): one more expert to the kernels, one that receives every token and so
    spans many row blocks, against the oracle on the same extended routing."""
    from oracle import routing as oroute
    from pyhip_amd.routing import append_shared_experts
    E0 = cases.CONFIGS[name]["E"]
    L = cases.make_layer(name, T, seed=11, E=E0 + 1, router="softmax")
    g = np.random.default_rng(12)
    tw0, ti0 = oroute.softmax_topk(g.standard_normal((T, E0)), L.k)        # the router sees the routed experts only
    tw, ti = append_shared_experts(torch.from_numpy(tw0).cuda(), torch.from_numpy(ti0).cuda(), E0, 1)
    assert ti.shape == (T, L.k + 1) and int(ti.max()) == E0
    w1, w1s, w2, w2s = cases.device_weights(L)
    print(f"shared-expert case {name} T={T} method={method} bm={bm}", flush=True)
    out = fused_moe(L.hidden.cuda(), w1, w2, tw, ti, w1_scale=w1s, w2_scale=w2s, block_size_M=bm, dtype=torch.float32,
                    method=method)
    torch.cuda.synchronize()
    ref = moe.moe_ref(_f(L.hidden), L.w1q, L.w1s, L.w2q, L.w2s, tw.cpu().numpy(), ti.cpu().numpy(),
                      act="a4" if method == "a4w4" else "a16")
    got = _f(out)
    rms = np.sqrt(np.mean(ref.astype(np.float64) ** 2))
    err, cos = metrics.max_err_over_rms(got, ref), metrics.cosine(got, ref)
    frac = float((np.abs(got - ref) > TOL_MAX * rms).mean())
    print(f"  vs oracle: max|err|/rms={err:.3e} cosine={cos:.8f} beyond-bound fraction={frac:.2e}", flush=True)
    # the bound of _end_to_end's relaxed branch (a stage-1 value rounded the other way may move one activation by an e2m1 step)
    assert cos >= TOL_COS and metrics.calc_diff(got, ref) <= 0.01 and frac <= 2e-3 and err <= 0.1


@pytest.mark.parametrize("method,T", [("a4w4", 50), ("w4a16", 5)])
def test_plain_layout_weights(method, T):
    """Weights without the ``is_shuffled`` mark are in the plain [E, N, K/2] layout (the reference's kernels take
    both, src/contrib/fused_moe.py:198-206,410,480): the operator re-tiles them once and gives the same bits."""
    L = cases.make_layer("tiny", T, seed=13)
    w1, w1s, w2, w2s = cases.device_weights(L)
    p1, _, p2, _ = cases.plain_device_weights(L)
    assert not getattr(p1, "is_shuffled", False)
    tw, ti = torch.from_numpy(L.topk_w).cuda(), torch.from_numpy(L.topk_ids).cuda()
    print(f"plain-layout case tiny T={T} method={method}", flush=True)
    a = fused_moe(L.hidden.cuda(), w1, w2, tw, ti, w1_scale=w1s, w2_scale=w2s, method=method)
    b = fused_moe(L.hidden.cuda(), p1, p2, tw, ti, w1_scale=w1s, w2_scale=w2s, method=method)
    c = fused_moe(L.hidden.cuda(), torch.nn.Parameter(w1.clone(), requires_grad=False),
                  torch.nn.Parameter(w2.clone(), requires_grad=False), tw, ti, w1_scale=w1s, w2_scale=w2s, method=method)
    torch.cuda.synchronize()
    assert torch.equal(a, b) and torch.equal(a, c)


def test_odd_views_of_hidden_states_are_copied():
    """a column slice at an odd element offset (base not 16-byte aligned, row stride not a multiple of 8) is made
    contiguous instead of being refused"""
    L = cases.make_layer("tiny", 12, seed=14)
    w1, w1s, w2, w2s = cases.device_weights(L)
    tw, ti = torch.from_numpy(L.topk_w).cuda(), torch.from_numpy(L.topk_ids).cuda()
    wide = torch.zeros(12, L.H + 5, dtype=torch.bfloat16, device="cuda")
    wide[:, 3:3 + L.H] = L.hidden.cuda()
    view = wide[:, 3:3 + L.H]
    for method in ("a4w4", "w4a16"):
        a = fused_moe(view, w1, w2, tw, ti, w1_scale=w1s, w2_scale=w2s, method=method)
        b = fused_moe(view.contiguous(), w1, w2, tw, ti, w1_scale=w1s, w2_scale=w2s, method=method)
        torch.cuda.synchronize()
        assert torch.equal(a, b)


@pytest.mark.parametrize("name,T,bm", [("dsv3_s", 16, 16), ("tiny", 300, 128), ("odd", 200, 128)])
def test_atomic_topk_reduce_variant(name, T, bm):
    """topk_reduce="atomic": the down GEMM adds bf16(acc * routing weight) into the output with packed bf16 atomics
    (the reference's atomic variant, src/contrib/moe_gemm_mxfp4.py:1334-1398).  Every addition rounds to bf16 and the
    slots arrive in no fixed order, so the comparison with the deterministic result allows one bf16 rounding (half an
    ulp, 2^-8 relative) of a running sum no larger than the sum of the slot magnitudes per addition."""
    L = cases.make_layer(name, T, seed=17)
    w1, w1s, w2, w2s = cases.device_weights(L)
    tw, ti = torch.from_numpy(L.topk_w).cuda(), torch.from_numpy(L.topk_ids).cuda()
    print(f"atomic-reduce case {name} T={T} bm={bm}", flush=True)
    kw = dict(w1_scale=w1s, w2_scale=w2s, block_size_M=bm, method="a4w4")
    ref32, parts = fused_moe(L.hidden.cuda(), w1, w2, tw, ti, dtype=torch.float32, return_parts=True, **kw)
    got = fused_moe(L.hidden.cuda(), w1, w2, tw, ti, topk_reduce="atomic", **kw)
    torch.cuda.synchronize()
    assert got.dtype == torch.bfloat16 and torch.isfinite(got.float()).all()
    mag = parts["out3"].float().abs().sum(dim=1)                      # sum over slots of |slot value|
    assert ((got.float() - ref32).abs() <= mag * L.k * 2.0 ** -8 + 1e-30).all()
    rms = ref32.pow(2).mean().sqrt().item()
    err = (got.float() - ref32).abs().max().item() / rms
    print(f"  max|atomic - deterministic fp32 sum| / rms = {err:.3e}", flush=True)
    assert metrics.cosine(_f(got), _f(ref32)) >= 0.9999


@pytest.mark.parametrize("name,T,bm,bias", [("dsv3_s", 16, 16, False), ("dsv3_s", 200, 16, False), ("tiny", 300, 128, True),
                                            ("mixtral_s", 700, 288, False), ("odd", 640, 288, True), ("qwen3_s", 257, 128, False)])
def test_last_arriver_topk_reduce_variant(name, T, bm, bias):
    """topk_reduce="last_arriver": the down GEMM's workgroups do the top-k reduction themselves, the one that stores a
    token's last slot for a weight tile sums the slots in slot order.  Same arithmetic as the reduction kernel, so the
    output must equal the default path's bit for bit, in bf16 and in fp32, whatever the arrival order (three runs), and
    also where the sort drops pairs (expert mask, local token count): a token all of whose pairs are dropped comes
    out as zeros."""
    L = cases.make_layer(name, T, seed=21, bias=bias)
    w1, w1s, w2, w2s = cases.device_weights(L)
    tw, ti = torch.from_numpy(L.topk_w).cuda(), torch.from_numpy(L.topk_ids).cuda()
    kw = dict(w1_scale=w1s, w2_scale=w2s, block_size_M=bm, method="a4w4", bias1=None if L.bias1 is None else L.bias1.cuda(),
              bias2=None if L.bias2 is None else L.bias2.cuda())
    hidden = L.hidden.cuda()
    print(f"last-arriver case {name} T={T} bm={bm} bias={bias}", flush=True)
    for dt in (torch.bfloat16, torch.float32):
        want = fused_moe(hidden, w1, w2, tw, ti, dtype=dt, **kw)
        for rep in range(3):
            got, parts = fused_moe(hidden, w1, w2, tw, ti, dtype=dt, topk_reduce="last_arriver", return_parts=True, **kw)
            torch.cuda.synchronize()
            assert torch.equal(got, want), f"dtype {dt} run {rep}"
    # out3 is still written in full (callers may want the per-slot results)
    _, parts0 = fused_moe(hidden, w1, w2, tw, ti, return_parts=True, **kw)
    assert torch.equal(parts["out3"], parts0["out3"])
    # dropped pairs: every other expert masked out, and only the first two thirds of the tokens take part
    E = L.E
    mask = torch.tensor([e % 2 for e in range(E)], dtype=torch.int32, device="cuda")
    keep = mask.bool()
    w1k, w2k = w1[keep].contiguous(), w2[keep].contiguous()
    w1k.is_shuffled = w2k.is_shuffled = True
    kwm = dict(kw, w1_scale=w1s.view(E, -1)[keep].contiguous().view(-1, w1s.shape[-1]),
               w2_scale=w2s.view(E, -1)[keep].contiguous().view(-1, w2s.shape[-1]), expert_mask=mask,
               num_local_tokens=torch.tensor([max(1, 2 * T // 3)], dtype=torch.int32, device="cuda"),
               bias1=None if L.bias1 is None else L.bias1.cuda()[keep].contiguous(),
               bias2=None if L.bias2 is None else L.bias2.cuda()[keep].contiguous())
    want = fused_moe(hidden, w1k, w2k, tw, ti, **kwm)
    got = fused_moe(hidden, w1k, w2k, tw, ti, topk_reduce="last_arriver", **kwm)
    torch.cuda.synchronize()
    assert torch.equal(got, want)
    assert (got[max(1, 2 * T // 3):] == 0).all()


def test_mfma_stream_probe_runs():
    """the measurement probe behind bench.py --frontier: every variant launches, finishes and reports the CU count;
    bad arguments are refused before anything is launched"""
    import ctypes
    from pyhip_amd import _lib
    lib = _lib.load()
    buf = torch.zeros((1 << 30) + (16 << 20), dtype=torch.uint8, device="cuda")
    sink = torch.zeros(4, dtype=torch.int32, device="cuda")
    wgs = ctypes.c_int(0)
    for v in range(10):
        print(f"probe variant {v}", flush=True)
        _lib.check(lib.pyhip_moe_probe_mfma_stream(v, 20, _lib.dptr(buf), buf.numel(), _lib.dptr(sink), 2, ctypes.byref(wgs),
                                                   _lib.current_stream()), "probe")
        torch.cuda.synchronize()
    assert wgs.value == 2 * torch.cuda.get_device_properties(0).multi_processor_count     # (the last variants: two per CU)
    assert (sink == 0).all()
    assert lib.pyhip_moe_probe_mfma_stream(10, 20, _lib.dptr(buf), buf.numel(), _lib.dptr(sink), 1, None, None) == 1
    assert lib.pyhip_moe_probe_mfma_stream(2, 20, _lib.dptr(buf), 1 << 30, _lib.dptr(sink), 1, None, None) == 1
    assert b"buffer" in lib.pyhip_moe_last_error()


@pytest.mark.parametrize("T", [2, 3, 7, 31, 63, 128, 200, 255, 256, 768, 2048])
def test_reference_style_inputs(T):
    """The reference's own accuracy sweep (tests/contrib/moe/test_moe.py:949-1035) draws its inputs differently from
    the benchmark: hidden states (x + 1) * 0.001 (small, non-zero mean, :145), expert ids from tiled random
    permutations (every token's slots distinct, loads balanced, :264-272) and routing weights ~N(0,1), negative ones
    included (:264); batch sizes 2..63, 128..255 and multiples of 256.  Same bar as there plus this suite's:
    calc_diff <= 0.01 against the fp32 oracle, cosine >= 0.999, outliers bounded."""
    E, k, H, I = 64, 8, 1024, 512
    g = torch.Generator().manual_seed(1000 + T)
    L = cases.make_layer("dsv3_s", T, seed=3)
    L.hidden = ((torch.randn(T, H, generator=g) + 1.0) * 0.001).to(torch.bfloat16)
    L.topk_ids = torch.stack([torch.randperm(E, generator=g)[:k] for _ in range(T)]).to(torch.int32).numpy()
    L.topk_w = torch.randn(T, k, generator=g).float().numpy()
    w1, w1s, w2, w2s = cases.device_weights(L)
    tw, ti = torch.from_numpy(L.topk_w).cuda(), torch.from_numpy(L.topk_ids).cuda()
    print(f"reference-style case T={T}", flush=True)
    for method in ("a4w4", "w4a16"):
        if method == "w4a16" and T > 256:
            continue
        out = fused_moe(L.hidden.cuda(), w1, w2, tw, ti, w1_scale=w1s, w2_scale=w2s, dtype=torch.float32, method=method)
        torch.cuda.synchronize()
        ref = moe.moe_ref(_f(L.hidden), L.w1q, L.w1s, L.w2q, L.w2s, L.topk_w, L.topk_ids,
                          act="a4" if method == "a4w4" else "a16")
        got = _f(out)
        rms = np.sqrt(np.mean(ref.astype(np.float64) ** 2))
        err = np.abs(got - ref) / rms
        cd = metrics.calc_diff(got, ref)
        print(f"  {method}: max|err|/rms={err.max():.3e} beyond-bound fraction={np.mean(err > TOL_MAX):.2e} "
              f"cosine={metrics.cosine(got, ref):.8f} calc_diff={cd:.2e}", flush=True)
        assert np.isfinite(got).all() and cd <= 0.01 and metrics.cosine(got, ref) >= TOL_COS
        assert np.mean(err > TOL_MAX) <= 2e-3 and err.max() <= 0.1


@pytest.mark.parametrize("T,bm", [(48, 16), (300, 128)])
def test_more_experts_than_the_tile_schedule_holds(T, bm):
    """720 experts: the MXFP4 GEMMs keep their tile schedule in LDS for up to 704 and otherwise start one workgroup
    per tile.  (The 720 experts are 45 copies of 16 drawn ones, so that building the case stays cheap; every token's
    experts are distinct.)  Same bounds as the other end-to-end cases; and the result must equal, bit for bit, the
    one the 16-expert layer gives for the ids folded back, which takes the scheduled path."""
    base = cases.make_layer("tiny", T, seed=11, E=16, k=4, bias=True)
    rep = 45
    L = cases.Layer()
    L.E, L.k, L.H, L.I, L.T = base.E * rep, base.k, base.H, base.I, T
    L.hidden, L.topk_w = base.hidden, base.topk_w
    L.w1q, L.w1s = np.tile(base.w1q, (rep, 1, 1)), np.tile(base.w1s, (rep, 1, 1))
    L.w2q, L.w2s = np.tile(base.w2q, (rep, 1, 1)), np.tile(base.w2s, (rep, 1, 1))
    L.bias1, L.bias2 = base.bias1.repeat(rep, 1), base.bias2.repeat(rep, 1)
    rng = np.random.default_rng(5)
    L.topk_ids = (base.topk_ids + base.E * rng.integers(0, rep, size=base.topk_ids.shape)).astype(base.topk_ids.dtype)
    assert L.topk_ids.max() >= 704
    outs = []
    for lay in (L, base):
        w1, w1s, w2, w2s = cases.device_weights(lay)
        tw, ti = torch.from_numpy(lay.topk_w).cuda(), torch.from_numpy(lay.topk_ids).cuda()
        print(f"many-experts case E={lay.E} T={T} bm={bm}", flush=True)
        outs.append(fused_moe(lay.hidden.cuda(), w1, w2, tw, ti, w1_scale=w1s, w2_scale=w2s, block_size_M=bm,
                              bias1=lay.bias1.cuda(), bias2=lay.bias2.cuda(), dtype=torch.float32, method="a4w4",
                              return_parts=True))
        torch.cuda.synchronize()
    (out32, parts), (out_base, _) = outs
    assert torch.equal(out32, out_base)
    w1e, w2e, ref_a2, nflip1 = _stage_checks(L, parts, parts["block_m"])
    assert w1e <= TOL_MAX and w2e <= TOL_MAX
    ref = moe.moe_ref(_f(L.hidden), L.w1q, L.w1s, L.w2q, L.w2s, L.topk_w, L.topk_ids, act="a4", bias1=_f(L.bias1),
                      bias2=_f(L.bias2))
    _end_to_end(_f(out32), ref, ref_a2, nflip1)


@pytest.mark.parametrize("name,T,bias", [("mixtral_s", 700, False), ("mixtral_s", 40, True), ("longk_s", 300, True),
                                         ("odd", 520, False), ("gptoss_s1", 260, True)])
def test_tile_with_both_operands_through_lds(name, T, bias):
    """operand_staging="lds": the eight-wave 256-row tile (weights and activations both by LDS-DMA, two wave rows half
    a K-step apart) against the oracle, to the bounds of the other end-to-end cases, and bit for bit against the tiles
    that load weights into registers.  Shapes with two to five K-groups per tile (odd counts change the parity of the
    scale stages from tile to tile), experts with several row blocks and with a nearly empty last one."""
    L = cases.make_layer(name, T, seed=7, bias=bias)
    w1, w1s, w2, w2s = cases.device_weights(L)
    tw, ti = torch.from_numpy(L.topk_w).cuda(), torch.from_numpy(L.topk_ids).cuda()
    b1 = None if L.bias1 is None else L.bias1.cuda()
    b2 = None if L.bias2 is None else L.bias2.cuda()
    kw = dict(w1_scale=w1s, w2_scale=w2s, bias1=b1, bias2=b2, dtype=torch.float32, method="a4w4")
    print(f"lds-tile case {name} T={T} bias={bias}", flush=True)
    out_lds, parts = fused_moe(L.hidden.cuda(), w1, w2, tw, ti, operand_staging="lds", return_parts=True, **kw)
    torch.cuda.synchronize()
    assert parts["block_m"] == 256
    for bm in (256, 128):
        assert torch.equal(out_lds, fused_moe(L.hidden.cuda(), w1, w2, tw, ti, block_size_M=bm, **kw)), bm
    w1e, w2e, ref_a2, nflip1 = _stage_checks(L, parts, 256)
    assert w1e <= TOL_MAX and w2e <= TOL_MAX
    ref = moe.moe_ref(_f(L.hidden), L.w1q, L.w1s, L.w2q, L.w2s, L.topk_w, L.topk_ids, act="a4",
                      bias1=None if L.bias1 is None else _f(L.bias1), bias2=None if L.bias2 is None else _f(L.bias2))
    _end_to_end(_f(out_lds), ref, ref_a2, nflip1)


def test_lds_tile_rejects_what_it_does_not_serve():
    """a down GEMM with a single K-group (inter = 512) has nothing to pipeline: the entry point says so"""
    from pyhip_amd._lib import PyhipError
    L = cases.make_layer("tiny", 40, seed=1)
    w1, w1s, w2, w2s = cases.device_weights(L)
    tw, ti = torch.from_numpy(L.topk_w).cuda(), torch.from_numpy(L.topk_ids).cuda()
    with pytest.raises(PyhipError, match="K >= 1024"):
        fused_moe(L.hidden.cuda(), w1, w2, tw, ti, w1_scale=w1s, w2_scale=w2s, operand_staging="lds")
    with pytest.raises(ValueError):
        fused_moe(L.hidden.cuda(), w1, w2, tw, ti, w1_scale=w1s, w2_scale=w2s, operand_staging="lds", block_size_M=128)
