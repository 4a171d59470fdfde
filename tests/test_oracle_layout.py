"""Pins for oracle/layout.py: forward o inverse identity (the directions restate different
reference files) and the closed-form byte address of each permutation."""
import numpy as np

from oracle import layout


def test_weight_shuffle_roundtrip_and_address():
    rng = np.random.default_rng(0)
    N, Kb = 64, 256
    w = rng.integers(0, 256, (3, N, Kb), dtype=np.uint8)
    sh = layout.shuffle_weight(w)
    assert (layout.deshuffle_weight(sh) == w).all()
    flat = sh.reshape(3, -1)
    for n, kb in [(0, 0), (1, 0), (0, 16), (17, 70), (63, 255), (32, 129), (15, 63)]:
        addr = ((n // 16) * (Kb // 64) + kb // 64) * 1024 + ((kb % 64) // 16) * 256 + (n % 16) * 16 + kb % 16
        assert (flat[:, addr] == w[:, n, kb]).all()


def test_weight_block_is_mfma_lane_major():
    # one 1 KB block = 16 rows x 64 B; lane l (= kgrp*16 + row) owns bytes [l*16, l*16+16)
    N, Kb = 16, 64
    w = np.arange(N * Kb, dtype=np.uint32).astype(np.uint8).reshape(N, Kb)
    sh = layout.shuffle_weight(w).reshape(64, 16)
    for lane in range(64):
        row, kgrp = lane % 16, lane // 16
        assert (sh[lane] == w[row, kgrp * 16: kgrp * 16 + 16]).all()


def test_scale_shuffle_roundtrip_padding_and_address():
    rng = np.random.default_rng(1)
    R, C = 300, 13
    s = rng.integers(1, 255, (R, C), dtype=np.uint8)
    sh = layout.e8m0_shuffle(s)
    assert sh.shape == (512, 16)
    assert (layout.e8m0_deshuffle(sh, R, C) == s).all()
    full = layout.e8m0_deshuffle(sh)
    assert (full[R:] == 0).all() and (full[:, C:] == 0).all()
    flat = sh.reshape(-1)
    Cp = 16
    for r, c in [(0, 0), (1, 0), (16, 0), (0, 4), (0, 1), (37, 11), (299, 12), (31, 7), (32, 8)]:
        addr = ((r // 32) * (Cp // 8) + c // 8) * 256 + (c % 4) * 64 + (r % 16) * 4 + ((c % 8) // 4) * 2 + (r % 32) // 16
        assert flat[addr] == s[r, c]
