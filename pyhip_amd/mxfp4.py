"""Host-side MXFP4 weight preparation in torch (any device): quantise, dequantise and the two
byte re-tilings the kernels consume.

Formats (same as the reference's inputs):
  * values   uint8 [..., K/2], two e2m1 codes per byte, low nibble = even element
  * scales   uint8 [..., K/32], e8m0 = 2^(b-127); scale = 2^(floor(log2 amax) - 2)
  * ``shuffle_weight``: [N, Kb] -> 1 KB blocks of 16 rows x 64 B stored lane-major
    (src/misc.py:116-130 ``pre_shuffle(x, 16)``)
  * ``e8m0_shuffle``  : rows padded to 256, cols to 8, [32 rows x 8 cols] tiles of 256 B
    (tests/contrib/moe/test_fused_moe.py:222-236)
"""
import torch

BLOCK = 32
_E2M1 = [0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0]


def _table(device):
    t = torch.tensor(_E2M1 + [-v for v in _E2M1], dtype=torch.float32, device=device)
    return t


def quantize_mxfp4(x):
    """float tensor [..., K] -> (uint8 [..., K/2], uint8 [..., K/32])"""
    K = x.shape[-1]
    assert K % BLOCK == 0
    xb = x.float().reshape(*x.shape[:-1], K // BLOCK, BLOCK)
    amax = xb.abs().amax(dim=-1)
    _, ex = torch.frexp(amax)                      # amax = m * 2^ex, m in [0.5, 1)
    b = (ex.to(torch.int32) - 1 - 2 + 127)
    b = torch.where(amax > 0, b, torch.zeros_like(b)).clamp_(0, 254)
    a = torch.ldexp(xb.abs(), (127 - b).unsqueeze(-1))
    code = torch.zeros_like(a, dtype=torch.uint8)
    for mid, tie_up in ((0.25, False), (0.75, True), (1.25, False), (1.75, True), (2.5, False), (3.5, True), (5.0, False)):
        code += ((a > mid) | ((a == mid) & tie_up)).to(torch.uint8)
    code |= (torch.signbit(xb).to(torch.uint8) << 3)
    code = code.reshape(*x.shape[:-1], K // 2, 2)
    packed = code[..., 0] | (code[..., 1] << 4)
    return packed.contiguous(), b.to(torch.uint8).contiguous()


def dequantize_mxfp4(packed, scale, dtype=torch.float32):
    lo, hi = packed & 0xF, packed >> 4
    codes = torch.stack([lo, hi], dim=-1).reshape(*packed.shape[:-1], packed.shape[-1] * 2)
    vals = _table(packed.device)[codes.long()]
    K = vals.shape[-1]
    vb = vals.reshape(*vals.shape[:-1], K // BLOCK, BLOCK)
    out = torch.ldexp(vb, (scale.to(torch.int32) - 127).unsqueeze(-1))
    return out.reshape(vals.shape).to(dtype)


def shuffle_weight(w):
    """uint8 [..., N, Kb] -> same shape, MFMA-operand order (one 1 KB block per 16 rows x 64 B)."""
    assert w.dtype == torch.uint8
    *lead, N, Kb = w.shape
    assert N % 16 == 0 and Kb % 64 == 0, (N, Kb)
    x = w.reshape(*lead, N // 16, 16, Kb // 64, 4, 16)
    n = len(lead)
    x = x.permute(*range(n), n + 0, n + 2, n + 3, n + 1, n + 4)
    return x.contiguous().reshape(*lead, N, Kb)


def deshuffle_weight(w):
    assert w.dtype == torch.uint8
    *lead, N, Kb = w.shape
    x = w.reshape(*lead, N // 16, Kb // 64, 4, 16, 16)
    n = len(lead)
    x = x.permute(*range(n), n + 0, n + 3, n + 1, n + 2, n + 4)
    return x.contiguous().reshape(*lead, N, Kb)


def e8m0_shuffle(s):
    """uint8 [R, C] -> uint8 [ceil(R/256)*256, ceil(C/8)*8] in the scaled-MFMA tile order."""
    assert s.dtype == torch.uint8 and s.dim() == 2
    R, C = s.shape
    Rp, Cp = (R + 255) // 256 * 256, (C + 7) // 8 * 8
    p = torch.zeros(Rp, Cp, dtype=torch.uint8, device=s.device)
    p[:R, :C] = s
    p = p.view(Rp // 32, 2, 16, Cp // 8, 2, 4).permute(0, 3, 5, 2, 4, 1).contiguous()
    return p.view(Rp, Cp)


def e8m0_deshuffle(s, rows=None, cols=None):
    Rp, Cp = s.shape
    p = s.view(Rp // 32, Cp // 8, 4, 16, 2, 2).permute(0, 5, 3, 1, 4, 2).contiguous().view(Rp, Cp)
    return p[: (rows or Rp), : (cols or Cp)]


def prepare_expert_weights(w, shuffle=True):
    """float [E, N, K] -> (uint8 [E, N, K/2] (pre-shuffled), uint8 [E*N padded, K/32 padded] (shuffled)).

    The value tensor carries ``is_shuffled = True`` as the reference expects
    (src/contrib/fused_moe.py:198-206)."""
    E, N, K = w.shape
    q, s = quantize_mxfp4(w)
    if shuffle:
        q = shuffle_weight(q)
        q.is_shuffled = True
    return q, e8m0_shuffle(s.reshape(E * N, K // BLOCK))


def pad_to(n, multiple=512):
    return (n + multiple - 1) // multiple * multiple


def pad_layer_weights(w1q, w1s, w2q, w2s, bias1=None, bias2=None, multiple=512):
    """Zero-pad quantised (not yet shuffled) expert weights so that ``hidden`` and ``inter`` become
    multiples of ``multiple``, the way aiter pads gpt-oss weights (hidden 2880 -> 3072): the caller then
    passes ``hidden_pad`` / ``intermediate_pad`` to ``fused_moe`` (reference argument meaning:
    tests/contrib/moe/test_fused_moe.py:92-105 -- the trailing rows/columns of the padded weights are zero).

    w1q uint8 [E, 2I, H/2] (gate rows then up rows), w1s uint8 [E, 2I, H/32], w2q [E, H, I/2], w2s [E, H, I/32].
    Returns (w1q, w1s, w2q, w2s, bias1, bias2, hidden_pad, intermediate_pad) at the padded sizes; gate rows stay
    at [0, I), up rows move to [I_padded, I_padded + I).  A zero byte is the e2m1 pair (0, 0) and a zero
    scale byte multiplies it by 2^-127, so padded rows and columns contribute exactly nothing."""
    E, N1, Hb = w1q.shape
    H, I = Hb * 2, N1 // 2
    Hp, Ip = pad_to(H, multiple), pad_to(I, multiple)
    if (Hp, Ip) == (H, I):
        return w1q, w1s, w2q, w2s, bias1, bias2, 0, 0

    def grow(t, rows_from, rows_to, cols):
        out = torch.zeros(t.shape[0], rows_to, cols, dtype=t.dtype, device=t.device)
        out[:, :rows_from, : t.shape[2]] = t
        return out

    def grow_gate_up(t, cols):
        out = torch.zeros(t.shape[0], 2 * Ip, cols, dtype=t.dtype, device=t.device)
        out[:, :I, : t.shape[2]] = t[:, :I]
        out[:, Ip:Ip + I, : t.shape[2]] = t[:, I:]
        return out

    w1q_p, w1s_p = grow_gate_up(w1q, Hp // 2), grow_gate_up(w1s, Hp // BLOCK)
    w2q_p, w2s_p = grow(w2q, H, Hp, Ip // 2), grow(w2s, H, Hp, Ip // BLOCK)
    if bias1 is not None:
        b = torch.zeros(E, 2 * Ip, dtype=bias1.dtype, device=bias1.device)
        b[:, :I], b[:, Ip:Ip + I] = bias1[:, :I], bias1[:, I:]
        bias1 = b
    if bias2 is not None:
        b = torch.zeros(E, Hp, dtype=bias2.dtype, device=bias2.device)
        b[:, :H] = bias2
        bias2 = b
    return w1q_p, w1s_p, w2q_p, w2s_p, bias1, bias2, Hp - H, Ip - I
