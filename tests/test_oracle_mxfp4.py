"""Pins for oracle/mxfp4.py: value tables of the reference's vendored CK headers, the compiled CK
host conversion (oracle/_ref), torch's e8m0 dtype, brute force, and closed-form properties."""
import ctypes

import numpy as np
import pytest
import torch

from oracle import mxfp4
from conftest import ptr


def test_e2m1_table_matches_pk_fp4_header():
    # archive/ck_tile/ck_tile/core/numeric/pk_fp4.hpp:128-129
    expect = [0, 0.5, 1, 1.5, 2, 3, 4, 6, -0.0, -0.5, -1, -1.5, -2, -3, -4, -6]
    assert mxfp4.E2M1_TABLE16.tolist() == expect
    assert np.signbit(mxfp4.E2M1_TABLE16[8])


def test_nibble_order_low_is_even_element(ck_ref):
    packed = np.array([[0x21, 0xF7]], dtype=np.uint8)
    assert mxfp4.e2m1_unpack(packed).tolist() == [[1, 2, 7, 15]]
    assert mxfp4.e2m1_decode(packed).tolist() == [[0.5, 1.0, 6.0, -6.0]]
    assert ck_ref.ck_ref_pack(1, 2) == 0x21                      # pk_fp4.hpp:122-125
    assert (mxfp4.e2m1_pack(mxfp4.e2m1_unpack(packed)) == packed).all()


def test_e8m0_examples_from_header():
    # archive/ck_tile/ck_tile/core/numeric/e8m0.hpp:16-23
    b = np.array([0b01111111, 0b10000000, 0b10000010, 0b10000111, 0b10001110, 0, 254], dtype=np.uint8)
    got = mxfp4.e8m0_decode(b).astype(np.float64)
    assert got.tolist() == [1.0, 2.0, 8.0, 256.0, 32768.0, 2.0 ** -127, 2.0 ** 127]
    assert np.isnan(mxfp4.e8m0_decode(np.uint8(255)))


def test_e8m0_against_torch_dtype():
    b = np.arange(1, 255, dtype=np.uint8)       # 0 is 2^-127, a float32 denormal torch may flush
    t = torch.from_numpy(b.copy()).view(torch.float8_e8m0fnu).to(torch.float32).numpy()
    assert (t == mxfp4.e8m0_decode(b)).all()


def test_e8m0_and_e2m1_decode_against_compiled_ck(ck_ref):
    b = np.arange(1, 255, dtype=np.uint8)       # CK's host code returns FLT_MIN for byte 0 (e8m0.hpp:92-95)
    out = np.zeros(b.size, np.float32)
    ck_ref.ck_ref_e8m0_to_float(ptr(b), out.ctypes.data_as(ctypes.c_void_p), b.size)
    assert (out == mxfp4.e8m0_decode(b)).all()
    codes = np.arange(16, dtype=np.uint8)
    for scale in (1.0, 0.25, 8.0):
        f = np.zeros(16, np.float32)
        ck_ref.ck_ref_e2m1_to_float(ptr(codes), ctypes.c_float(scale), ptr(f), 16)
        assert (f == mxfp4.E2M1_TABLE16 * np.float32(scale)).all()


def _brute_nearest(v):
    """nearest table value; ties -> even code.  Independent of e2m1_encode_rne's thresholds."""
    vals = mxfp4.E2M1_VALUES.astype(np.float64)
    out = []
    for x in np.asarray(v, dtype=np.float64).ravel():
        a = min(abs(x), 1e30)
        d = np.abs(vals - a)
        best = np.flatnonzero(d == d.min())
        c = int(best[0]) if len(best) == 1 else int([b for b in best if b % 2 == 0][0])
        out.append(c | (8 if np.signbit(x) else 0))
    return np.array(out, dtype=np.uint8)


def test_encode_rne_brute_force():
    grid = np.arange(-9.0, 9.0, 1.0 / 64, dtype=np.float32)        # hits every midpoint exactly
    assert (mxfp4.e2m1_encode_rne(grid) == _brute_nearest(grid)).all()
    rng = np.random.default_rng(1)
    x = (rng.standard_normal(20000) * 3).astype(np.float32)
    assert (mxfp4.e2m1_encode_rne(x) == _brute_nearest(x)).all()


def test_encode_rne_against_compiled_ck(ck_ref):
    # CK's saturation branch drops the sign for |v| >= 7 (mxfp_convert.hpp:100-104 returns 0b0111);
    # compare on |v| < 7 where its arithmetic is the RNE conversion.
    grid = np.arange(-6.984375, 7.0, 1.0 / 64, dtype=np.float32)
    rng = np.random.default_rng(2)
    rnd = np.clip(rng.standard_normal(50000) * 2.5, -6.99, 6.99).astype(np.float32)
    for x in (grid, rnd):
        for scale in (1.0, 0.5, 4.0):
            xs = (x * np.float32(scale)).astype(np.float32)
            codes = np.zeros(xs.size, np.uint8)
            ck_ref.ck_ref_float_to_e2m1(ptr(xs), ctypes.c_float(scale), ptr(codes), xs.size)
            mine = mxfp4.e2m1_encode_rne(x)
            # CK encodes -0.0 results of tiny negatives with the sign bit as well
            assert (codes == mine).all(), np.flatnonzero(codes != mine)[:10]


def test_block_scale_closed_form():
    amax = np.array([1.0, 1.5, 2.0, 3.99, 4.0, 0.02, 6.0, 2.0 ** -130, 0.0, 3e38], dtype=np.float32)
    b = mxfp4.block_scale_e8m0(amax)
    for a, bb in zip(amax.astype(np.float64), b):
        if a == 0:
            assert bb == 0
            continue
        e = int(np.floor(np.log2(a))) - 2 + 127
        assert bb == min(max(e, 0), 254)
        if 0 < e < 254:
            assert 4.0 <= a / 2.0 ** (int(bb) - 127) < 8.0          # amax lands in [4, 8) * scale


def test_quantize_properties():
    rng = np.random.default_rng(3)
    x = (rng.standard_normal((64, 256)) * np.exp(rng.standard_normal((64, 1)) * 3)).astype(np.float32)
    x[3, 32:64] = 0                                              # an all-zero block
    q, s = mxfp4.quantize_mxfp4(x)
    assert q.shape == (64, 128) and s.shape == (64, 8) and q.dtype == np.uint8 and s.dtype == np.uint8
    d = mxfp4.dequantize_mxfp4(q, s)
    assert (d[3, 32:64] == 0).all() and s[3, 1] == 0
    # idempotence: the dequantised block has the same amax exponent (values >= 4*scale survive) or,
    # if amax rounded up into the next binade, re-quantises to the same real numbers
    q2, s2 = mxfp4.quantize_mxfp4(d)
    assert (mxfp4.dequantize_mxfp4(q2, s2) == d).all()
    # error bound: half a step of the local e2m1 spacing (<= 1 for values in [4,6], saturation adds
    # up to 2 for scaled values in (6, 8)), in units of the block scale
    scale = np.repeat(mxfp4.e8m0_decode(s), 32, axis=1)
    err = np.abs(x - d) / scale
    assert err.max() <= 2.0
    assert (np.abs(d) <= 6 * scale).all()
    inside = np.abs(x) / scale <= 6
    assert err[inside].max() <= 1.0
    # sign and monotonicity
    assert ((d == 0) | (np.sign(d) == np.sign(x))).all()


def test_bf16_round_against_torch():
    rng = np.random.default_rng(4)
    x = (rng.standard_normal(100000) * 10).astype(np.float32)
    x[:4] = [1.00390625, 1.01171875, -1.00390625, 3.0e38]         # exact ties
    t = torch.from_numpy(x).to(torch.bfloat16).to(torch.float32).numpy()
    assert (mxfp4.bf16_round(x) == t).all()
