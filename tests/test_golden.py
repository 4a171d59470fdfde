"""Golden fixtures of tests/golden (written by tests/golden/make_golden.py from the compiled reference
headers and the CPU oracle): the oracle against them on the CPU, the HIP path against them on the GPU."""
import os
import zlib

import numpy as np
import pytest
import torch

from oracle import mxfp4 as om, sorting, moe, metrics
import cases

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _sort_cases():
    z = np.load(os.path.join(GOLD, "sort_ck.npz"))
    for i in range(int(z["n_cases"])):
        T, k, E, unit, masked, n = [int(v) for v in z[f"c{i}_meta"]]
        yield dict(ids=z[f"c{i}_ids"], w=z[f"c{i}_w"], T=T, k=k, E=E, unit=unit, n=n,
                   mask=z[f"c{i}_mask"] if masked else None, so=z[f"c{i}_sorted_ids"], sw=z[f"c{i}_sorted_w"],
                   se=z[f"c{i}_sorted_e"])


def test_oracle_sorter_against_golden():
    for c in _sort_cases():
        so, sw, se, nv = sorting.moe_sorting_ref(c["ids"], c["w"], c["E"], c["unit"], expert_mask=c["mask"])
        n = c["n"]
        assert int(nv[0]) == n and (so[:n] == c["so"]).all() and (sw[:n] == c["sw"]).all()
        assert (se[: n // c["unit"]] == c["se"]).all()


def test_oracle_e2m1_against_golden():
    z = np.load(os.path.join(GOLD, "e2m1_ck.npz"))
    assert (om.E2M1_TABLE16 == z["e2m1_table"]).all()
    xs = z["x_over_scale"]
    for si, sc in enumerate(z["scales"]):
        got = om.e2m1_encode_rne(((xs * sc).astype(np.float32) / sc).astype(np.float32))   # the converter sees x / scale
        # the reference's host converter returns +6 (code 7) for every |v| >= 7, dropping the sign of negative
        # inputs (mxfp_convert.hpp:100-104); the oracle saturates to -6 (code 15) there, as the MX format and the
        # hardware conversion do.  Everything below the saturation branch must agree bit for bit.
        sat_neg = xs <= -7
        assert (got[~sat_neg] == z["codes"][si][~sat_neg]).all(), (sc, xs[got != z["codes"][si]][:8])
        assert (z["codes"][si][sat_neg] == 7).all() and (got[sat_neg] == 15).all()
    # byte 0 is 2^-127 in the MX format; the reference's host conversion returns FLT_MIN = 2^-126 for it
    # (e8m0.hpp:92-95).  It only ever scales all-zero blocks, so the difference is unobservable.
    e8 = z["e8m0_table"]
    mine = om.e8m0_decode(np.arange(255, dtype=np.uint8))
    assert (mine[1:] == e8[1:]).all() and e8[0] == np.float32(2.0 ** -126) and mine[0] == np.float32(2.0 ** -127)


def test_oracle_layer_against_golden():
    z = np.load(os.path.join(GOLD, "tiny_layer.npz"))
    L = cases.make_layer("tiny", 64, seed=0)
    crc = lambda a: np.uint32(zlib.crc32(np.ascontiguousarray(a).tobytes()))
    # the seeded inputs are the ones the fixture was made from
    assert crc(L.hidden.view(dtype=torch.int16).numpy()) == z["crc_hidden"]
    assert crc(L.w1q) == z["crc_w1q"] and crc(L.w1s) == z["crc_w1s"]
    assert crc(L.w2q) == z["crc_w2q"] and crc(L.w2s) == z["crc_w2s"]
    assert (L.topk_ids == z["topk_ids"]).all() and (L.topk_w == z["topk_w"]).all()
    ref = moe.moe_ref(L.hidden.float().numpy(), L.w1q, L.w1s, L.w2q, L.w2s, L.topk_w, L.topk_ids, act="a4")
    # same algorithm, same BLAS: allow only reassociation noise of the fp32 matmul
    assert metrics.max_err_over_rms(ref, z["out"]) < 2e-3
    assert metrics.cosine(ref, z["out"]) > 0.99999


@pytest.mark.gpu
def test_gpu_sorter_against_golden():
    from pyhip_amd.moe_sorting import moe_sorting
    for i, c in enumerate(_sort_cases()):
        print(f"golden sort case {i}: T={c['T']} k={c['k']} E={c['E']} unit={c['unit']}", flush=True)
        mask = None if c["mask"] is None else torch.from_numpy(c["mask"]).cuda()
        so, sw, se, nv, _ = moe_sorting(torch.from_numpy(c["ids"]).cuda(), torch.from_numpy(c["w"]).cuda(), c["E"],
                                        1024, torch.bfloat16, c["unit"], mask, alloc_moe_out=False)
        torch.cuda.synchronize()
        n = c["n"]
        assert int(nv[0]) == n
        assert (so.cpu().numpy().view(np.uint32)[:n] == c["so"]).all()
        assert (sw.cpu().numpy()[:n] == c["sw"]).all()
        assert (se.cpu().numpy().view(np.uint32)[: n // c["unit"]] == c["se"]).all()


@pytest.mark.gpu
def test_gpu_layer_against_golden():
    """tolerance: max|err| <= 1e-2 * rms(ref), cosine >= 0.999"""
    from pyhip_amd import fused_moe
    z = np.load(os.path.join(GOLD, "tiny_layer.npz"))
    L = cases.make_layer("tiny", 64, seed=0)
    w1, w1s, w2, w2s = cases.device_weights(L)
    print("golden layer: tiny T=64", flush=True)
    out = fused_moe(L.hidden.cuda(), w1, w2, torch.from_numpy(L.topk_w).cuda(), torch.from_numpy(L.topk_ids).cuda(),
                    w1_scale=w1s, w2_scale=w2s, dtype=torch.float32)
    torch.cuda.synchronize()
    got = out.cpu().numpy()
    assert metrics.max_err_over_rms(got, z["out"]) <= 1e-2 and metrics.cosine(got, z["out"]) >= 0.999
