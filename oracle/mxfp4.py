"""MXFP4 (OCP microscaling: e2m1 values, one e8m0 scale per 32 elements) on the CPU.

Test infrastructure only (see ``oracle/__init__.py``).  numpy, byte/integer exact.

Restates
  * e2m1 value table and nibble order (low nibble = even element):
    archive/ck_tile/ck_tile/core/numeric/pk_fp4.hpp:122-129,196-203
  * e8m0 decode 2^(b-127), 0xFF = NaN: archive/ck_tile/ck_tile/core/numeric/e8m0.hpp:16-23,85-100
  * round-to-nearest-even float -> e2m1 with saturation at 6:
    archive/ck_tile/ck_tile/core/numeric/mxfp_convert.hpp:61-216
  * per-1x32 quantisation as the reference's tests use it through
    ``aiter.get_torch_quant(QuantType.per_1x32)`` (tests/contrib/moe/test_moe.py:161,175;
    tests/contrib/moe/test_mxfp4.py:46).  aiter is a third-party module that is not in the
    reference tree and has no pinned version; the block-scale rule used here is the closed
    form of the benchmark definition: scale = 2^(floor(log2(amax)) - 2).
  * dequantisation: tests/contrib/moe/test_moe.py:164-166,178-180.

Pins
  * ``e2m1_decode`` / ``e8m0_decode``: the value table of pk_fp4.hpp and the examples of
    e8m0.hpp (tests/test_oracle_mxfp4.py), torch's own float8_e8m0fnu cast, and the compiled
    CK host code in oracle/_ref where it builds.
  * ``e2m1_encode_rne``: compiled CK ``convert_to_type<pk_fp4_t>`` (oracle/_ref) for |v| < 7,
    brute-force nearest-value search with ties-to-even-code over a dense grid.
  * ``quantize_mxfp4``: properties the closed form fixes (amax lands in [4,8)*scale, the
    error bound of half a step, idempotence of quantise(dequantise(.))).  Tie-breaking and
    all-zero-block behaviour of aiter's quantiser itself: **parity unpinned** (aiter absent).
"""
import numpy as np

#: e2m1 magnitudes by 3-bit code (exp:2, mant:1, bias 1); bit 3 is the sign.
E2M1_VALUES = np.array([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0], dtype=np.float32)
E2M1_TABLE16 = np.concatenate([E2M1_VALUES, -E2M1_VALUES]).astype(np.float32)
BLOCK = 32


def e8m0_decode(b):
    """uint8 biased exponent -> float32 2^(b-127); 0xFF -> NaN (e8m0.hpp:16-23)."""
    b = np.asarray(b, dtype=np.uint8)
    out = np.ldexp(np.float32(1.0), np.minimum(b, 254).astype(np.int32) - 127).astype(np.float32)
    return np.where(b == 0xFF, np.float32(np.nan), out)


def e2m1_unpack(packed):
    """uint8[..., K/2] -> uint8 codes[..., K]; low nibble is the even element (pk_fp4.hpp:122-125)."""
    packed = np.asarray(packed, dtype=np.uint8)
    lo = packed & 0x0F
    hi = packed >> 4
    return np.stack([lo, hi], axis=-1).reshape(*packed.shape[:-1], packed.shape[-1] * 2)


def e2m1_pack(codes):
    codes = np.asarray(codes, dtype=np.uint8)
    assert codes.shape[-1] % 2 == 0
    c = codes.reshape(*codes.shape[:-1], codes.shape[-1] // 2, 2)
    return (c[..., 0] & 0x0F) | ((c[..., 1] & 0x0F) << 4)


def e2m1_decode(packed):
    """uint8[..., K/2] -> float32[..., K]."""
    return E2M1_TABLE16[e2m1_unpack(packed)]


def e2m1_encode_rne(v):
    """float32 (already divided by the block scale) -> 4-bit code, round to nearest,
    ties to the even code, |v| > 6 saturates to +-6 (mxfp_convert.hpp:61-216).

    Midpoints between neighbours: .25 .75 1.25 1.75 2.5 3.5 5; the even codes are
    0 (0.0), 2 (1.0), 4 (2.0), 6 (4.0).
    """
    v = np.asarray(v, dtype=np.float32)
    a = np.abs(v)
    # code = number of thresholds passed; ties resolved per midpoint parity
    code = np.zeros(a.shape, dtype=np.uint8)
    #          midpoint, tie goes up?
    for mid, tie_up in ((0.25, False), (0.75, True), (1.25, False), (1.75, True),
                        (2.5, False), (3.5, True), (5.0, False)):
        m = np.float32(mid)
        code += ((a > m) | ((a == m) & tie_up)).astype(np.uint8)
    sign = np.signbit(v).astype(np.uint8) << 3
    return (code | sign).astype(np.uint8)


def block_scale_e8m0(amax):
    """Biased exponent of 2^(floor(log2(amax)) - 2), clamped to [0, 254]; amax == 0 -> 0."""
    amax = np.asarray(amax, dtype=np.float32)
    _, e = np.frexp(amax)              # amax = m * 2^e, m in [0.5, 1)  ->  floor(log2) = e - 1
    fl = e.astype(np.int32) - 1
    b = fl - 2 + 127
    b = np.where(amax > 0, b, 0)
    return np.clip(b, 0, 254).astype(np.uint8)


def quantize_mxfp4(x):
    """float [..., K] (K % 32 == 0) -> (uint8 packed [..., K/2], uint8 e8m0 [..., K/32])."""
    x = np.asarray(x, dtype=np.float32)
    K = x.shape[-1]
    assert K % BLOCK == 0
    xb = x.reshape(*x.shape[:-1], K // BLOCK, BLOCK)
    amax = np.max(np.abs(xb), axis=-1)
    sb = block_scale_e8m0(amax)
    scaled = np.ldexp(xb, (127 - sb.astype(np.int32))[..., None]).astype(np.float32)
    codes = e2m1_encode_rne(scaled).reshape(x.shape)
    return e2m1_pack(codes), sb


def dequantize_mxfp4(packed, scale_e8m0):
    """(uint8 [..., K/2], uint8 [..., K/32]) -> float32 [..., K] (exact: <= 2 mantissa bits)."""
    vals = e2m1_decode(packed)
    K = vals.shape[-1]
    vb = vals.reshape(*vals.shape[:-1], K // BLOCK, BLOCK)
    s = np.asarray(scale_e8m0, dtype=np.uint8)
    assert s.shape == vb.shape[:-1], (s.shape, vb.shape)
    out = np.ldexp(vb, (s.astype(np.int32) - 127)[..., None]).astype(np.float32)
    return out.reshape(vals.shape)


def bf16_round(x):
    """float32 -> nearest bfloat16 (ties to even), returned as float32."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    u = x.view(np.uint32).astype(np.uint64)
    r = ((u + 0x7FFF + ((u >> 16) & 1)) & 0xFFFF0000).astype(np.uint32)
    out = r.view(np.float32).copy()
    nan = np.isnan(x)
    out[nan] = np.nan
    return out.reshape(x.shape)
