"""Byte-level re-tilings of MXFP4 weights and e8m0 scales (numpy, exact).

Test infrastructure only (see ``oracle/__init__.py``).

Restates
  * ``shuffle_weight``  : src/misc.py:116-130 (``pre_shuffle(x, 16)``; the same permutation as
    ``aiter.ops.shuffle.shuffle_weight(layout=(16,16))`` used at tests/contrib/moe/test_moe.py:169,186)
  * ``deshuffle_weight``: src/contrib/moe_gemm_ref.py:1-22
  * ``e8m0_shuffle``    : algorithm quoted at tests/contrib/moe/test_fused_moe.py:222-236
  * ``e8m0_deshuffle``  : src/contrib/moe_gemm_ref.py:57-64

Pins: forward o inverse = identity on random bytes (the two directions are restated from
different reference files), plus the closed-form byte address each permutation implies
(tests/test_oracle_layout.py checks single bytes through the documented index formula:
weight byte (n, kb) -> ((n/16)*(Kb/64) + kb/64)*1024 + ((kb%64)/16)*256 + (n%16)*16 + kb%16;
scale byte (r, c) -> ((r/32)*(C/8) + c/8)*256 + (c%4)*64 + (r%16)*4 + ((c%8)/4)*2 + (r%32)/16).
"""
import numpy as np


def shuffle_weight(w):
    """uint8 [..., N, Kb] -> same shape, 1 KB blocks of 16 rows x 64 B stored lane-major
    (lane = kgrp*16 + row, 16 B each)."""
    w = np.asarray(w)
    assert w.dtype == np.uint8
    *lead, N, Kb = w.shape
    assert N % 16 == 0 and Kb % 64 == 0, (N, Kb)
    x = w.reshape(*lead, N // 16, 16, Kb // 64, 4, 16)
    nl = len(lead)
    x = np.moveaxis(x, nl + 1, nl + 3)          # [.., N/16, Kb/64, 4, 16, 16]
    return np.ascontiguousarray(x).reshape(*lead, N, Kb)


def deshuffle_weight(w):
    w = np.asarray(w)
    assert w.dtype == np.uint8
    *lead, N, Kb = w.shape
    x = w.reshape(*lead, N // 16, Kb // 64, 4, 16, 16)
    nl = len(lead)
    x = np.moveaxis(x, nl + 3, nl + 1)          # [.., N/16, 16, Kb/64, 4, 16]
    return np.ascontiguousarray(x).reshape(*lead, N, Kb)


def e8m0_shuffle(s):
    """uint8 [R, C] -> uint8 [ceil(R/256)*256, ceil(C/8)*8]; every [32 rows x 8 cols] tile
    becomes 256 B = 64 dwords, dword = (c%4)*16 + r%16, byte = ((c%8)/4)*2 + (r%32)/16."""
    s = np.asarray(s, dtype=np.uint8)
    R, C = s.shape
    Rp, Cp = (R + 255) // 256 * 256, (C + 7) // 8 * 8
    p = np.zeros((Rp, Cp), dtype=np.uint8)
    p[:R, :C] = s
    p = p.reshape(Rp // 32, 2, 16, Cp // 8, 2, 4).transpose(0, 3, 5, 2, 4, 1)
    return np.ascontiguousarray(p).reshape(Rp, Cp)


def e8m0_deshuffle(s, rows=None, cols=None):
    s = np.asarray(s, dtype=np.uint8)
    Rp, Cp = s.shape
    p = s.reshape(Rp // 32, Cp // 8, 4, 16, 2, 2).transpose(0, 5, 3, 1, 4, 2)
    p = np.ascontiguousarray(p).reshape(Rp, Cp)
    return p[: (rows or Rp), : (cols or Cp)]
