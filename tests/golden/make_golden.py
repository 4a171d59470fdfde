#!/usr/bin/env python3
"""Writes the golden fixtures of this directory.  Run from the repository root:

    make -C oracle/ref_build && python tests/golden/make_golden.py

Sources of the expected values:
  sort_ck.npz   inputs -> outputs of the reference's own C++ statement of the sorter
                (archive/ck_tile/ck_tile/host/reference/reference_moe_sorting.hpp:13-117), compiled from the
                reference tree into oracle/_ref/libck_ref.so
  e2m1_ck.npz   float -> e2m1 codes of the reference's converter (archive/ck_tile/ck_tile/core/numeric/
                mxfp_convert.hpp:61-216) for every tie and neighbourhood at several scales, the code -> float
                table (pk_fp4.hpp:128-129) and the e8m0 byte -> float table (e8m0.hpp:85-100), same library
  tiny_layer.npz  the tiny layer (E=8, top-2, T=64, H=1024, I=512, seed 0): routing, checksums of the seeded
                inputs and the layer output of the CPU oracle (oracle/moe.py, act="a4").  A regression anchor
                for the oracle and the known answer the GPU path is compared with.
The fixtures are data only; no reference source is stored here.
"""
import ctypes
import os
import sys
import zlib

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))


def ptr(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def main():
    from conftest import ck_sort
    lib = ctypes.CDLL(os.path.join(ROOT, "oracle", "_ref", "libck_ref.so"))
    lib.ck_ref_moe_sorting.restype = ctypes.c_int

    # ---- sorter
    rng = np.random.default_rng(2024)
    out = {}
    cases = [(5, 3, 6, 4, False), (37, 3, 11, 16, True), (64, 2, 8, 32, False), (16, 8, 256, 16, False),
             (200, 8, 32, 64, True), (1, 1, 1, 16, False), (129, 4, 16, 128, True)]
    for i, (T, k, E, unit, masked) in enumerate(cases):
        ids = np.stack([rng.permutation(E)[:k] for _ in range(T)]).astype(np.int32)
        w = rng.random((T, k)).astype(np.float32)
        mask = (rng.random(E) < 0.6).astype(np.int32) if masked else None
        so, sw, se, n = ck_sort(lib, ids, w, E, unit, mask)
        out.update({f"c{i}_ids": ids, f"c{i}_w": w, f"c{i}_meta": np.array([T, k, E, unit, int(masked), n]),
                    f"c{i}_mask": mask if masked else np.zeros(0, np.int32),
                    f"c{i}_sorted_ids": so, f"c{i}_sorted_w": sw, f"c{i}_sorted_e": se})
    np.savez_compressed(os.path.join(HERE, "sort_ck.npz"), n_cases=len(cases), **out)

    # ---- e2m1 / e8m0
    grid = [0.0, 0.25, 0.5, 0.75, 1.0, 1.25, 1.5, 1.75, 2.0, 2.5, 3.0, 3.5, 4.0, 5.0, 6.0, 7.0, 8.0, 100.0]
    xs = []
    for g in grid:
        for d in (-1e-3, -1e-6, 0.0, 1e-6, 1e-3):
            xs += [g + d, -(g + d)]
    xs = np.array(xs, np.float32)
    scales = np.array([2.0 ** -10, 0.5, 1.0, 8.0], np.float32)
    codes = np.zeros((len(scales), len(xs)), np.uint8)
    for si, sc in enumerate(scales):
        x = (xs * sc).astype(np.float32)
        c = np.zeros(len(xs), np.uint8)
        lib.ck_ref_float_to_e2m1(ptr(x), ctypes.c_float(float(sc)), ptr(c), len(xs))
        codes[si] = c
    table = np.zeros(16, np.float32)
    allc = np.arange(16, dtype=np.uint8)
    lib.ck_ref_e2m1_to_float(ptr(allc), ctypes.c_float(1.0), ptr(table), 16)
    e8 = np.zeros(255, np.float32)
    b = np.arange(255, dtype=np.uint8)
    lib.ck_ref_e8m0_to_float(ptr(b), ptr(e8), 255)
    np.savez_compressed(os.path.join(HERE, "e2m1_ck.npz"), x_over_scale=xs, scales=scales, codes=codes,
                        e2m1_table=table, e8m0_table=e8)

    # ---- the tiny layer
    import cases as tc
    from oracle import moe
    L = tc.make_layer("tiny", 64, seed=0)
    ref, a2, per_slot = moe.moe_ref(L.hidden.float().numpy(), L.w1q, L.w1s, L.w2q, L.w2s, L.topk_w, L.topk_ids,
                                    act="a4", return_parts=True)
    crc = lambda a: np.uint32(zlib.crc32(np.ascontiguousarray(a).tobytes()))
    np.savez_compressed(os.path.join(HERE, "tiny_layer.npz"), topk_ids=L.topk_ids, topk_w=L.topk_w,
                        crc_hidden=crc(L.hidden.view(dtype=__import__("torch").int16).numpy()), crc_w1q=crc(L.w1q),
                        crc_w1s=crc(L.w1s), crc_w2q=crc(L.w2q), crc_w2s=crc(L.w2s), out=ref.astype(np.float32),
                        a2_row0=a2[0].astype(np.float32))
    for f in sorted(os.listdir(HERE)):
        print(f, os.path.getsize(os.path.join(HERE, f)))


if __name__ == "__main__":
    main()
