"""Pins for oracle/sorting.py: the literal triple loop, the compiled CK host reference, the worked
example of moe_sorting_kernel.hpp:30-97 re-derived through it, and the invariants of
tests/contrib/moe/test_moe_sorting.py:109-125 (reference tree)."""
import numpy as np
import pytest

from oracle import sorting
from conftest import ck_sort


def _rand_case(rng, T, k, E, skew=False):
    if skew:
        p = 1.0 / np.arange(1, E + 1) ** 1.1
        p /= p.sum()
        ids = np.stack([rng.choice(E, size=k, replace=False, p=p) for _ in range(T)])
    else:
        ids = np.stack([rng.permutation(E)[:k] for _ in range(T)])
    w = rng.random((T, k), dtype=np.float32)
    return ids.astype(np.int32), w


CASES = [(1, 1, 1, 4), (5, 3, 6, 4), (64, 2, 8, 16), (33, 8, 256, 16), (7, 4, 128, 32), (200, 8, 32, 64),
         (16, 8, 256, 256), (129, 2, 8, 128)]


@pytest.mark.parametrize("T,k,E,Bm", CASES)
def test_against_triple_loop(T, k, E, Bm):
    rng = np.random.default_rng(T * 131 + k)
    ids, w = _rand_case(rng, T, k, E, skew=(E >= 32 and T > 16))
    so, sw, se, nv = sorting.moe_sorting_ref(ids, w, E, Bm)
    b_ids, b_w, b_e, b_n = sorting.moe_sorting_brute(ids.tolist(), w.tolist(), E, Bm)
    assert nv[0] == b_n and nv[1] == T
    assert so[:b_n].tolist() == b_ids
    assert sw[:b_n].tolist() == b_w
    assert se[: b_n // Bm].tolist() == b_e
    # tail: padding id, weight 0, expert fill
    assert (so[b_n:] == ((k << 24) | T)).all() and (sw[b_n:] == 0).all()
    assert (se[b_n // Bm:] == sorting.EXPERT_ID_FILL).all()
    assert so.size == sorting.max_blocks(T * k, E, Bm) * Bm


@pytest.mark.parametrize("T,k,E,Bm", CASES)
@pytest.mark.parametrize("masked", [False, True])
def test_against_compiled_ck_reference(ck_ref, T, k, E, Bm, masked):
    rng = np.random.default_rng(T * 7 + k + 1000 * masked)
    ids, w = _rand_case(rng, T, k, E)
    mask = None
    if masked:
        mask = (rng.random(E) < 0.6).astype(np.int32)
        mask[rng.integers(E)] = 1
    so, sw, se, nv = sorting.moe_sorting_ref(ids, w, E, Bm, expert_mask=mask)
    c_ids, c_w, c_e, c_n = ck_sort(ck_ref, ids, w, E, Bm, mask)
    assert nv[0] == c_n
    assert (so[:c_n] == c_ids).all()
    assert (sw[:c_n] == c_w).all()
    assert (se[: c_n // Bm] == c_e).all()


def test_worked_example_of_ck_header(ck_ref):
    # moe_sorting_kernel.hpp:30-97: 6 experts, top-3, unit 4, 5 tokens.  The comment's numbers
    # are inconsistent with its own token count, so the expected values come from the compiled
    # reference; the layout facts stated in the comment are asserted explicitly.
    ids = np.array([[0, 3, 5], [2, 3, 5], [1, 3, 5], [1, 2, 3], [1, 3, 5]], dtype=np.int32)
    w = np.arange(15, dtype=np.float32).reshape(5, 3) + 1
    so, sw, se, nv = sorting.moe_sorting_ref(ids, w, 6, 4)
    assert nv[0] == 24                                            # "num_tokens_post_padded_ptr : [24]" with skipping
    assert se[:6].tolist() == [0, 1, 2, 3, 3, 5]                  # "sorted_expert_ids_ptr : [0, 1, 2, 3, 3, 5]"
    assert (so[:24] & 0xFFFFFF).tolist() == [0, 5, 5, 5, 2, 3, 4, 5, 1, 3, 5, 5, 0, 1, 2, 3, 4, 5, 5, 5, 0, 1, 2, 4]
    c_ids, c_w, c_e, c_n = ck_sort(ck_ref, ids, w, 6, 4)
    assert c_n == 24 and (c_ids == so[:24]).all() and (c_w == sw[:24]).all()
    # local expert mask [1,0,1,1,0,1] -> local ids [0,1,2,2,3], padded count 20 (hpp:84-97)
    so, sw, se, nv = sorting.moe_sorting_ref(ids, w, 6, 4, expert_mask=[1, 0, 1, 1, 0, 1])
    assert nv[0] == 20 and se[:5].tolist() == [0, 1, 2, 2, 3]


@pytest.mark.parametrize("T,k,E,Bm", [(256, 8, 256, 32), (1000, 4, 128, 64)])
def test_permutation_invariants(T, k, E, Bm):
    # tests/contrib/moe/test_moe_sorting.py:109-125: every (token, slot) exactly once, under its
    # expert, with its weight; the padded total is a multiple of the block size
    rng = np.random.default_rng(5)
    ids, w = _rand_case(rng, T, k, E, skew=True)
    so, sw, se, nv = sorting.moe_sorting_ref(ids, w, E, Bm)
    n = int(nv[0])
    assert n % Bm == 0
    seen = np.zeros((T, k), dtype=np.int32)
    for p in range(n):
        tok, slot = int(so[p] & 0xFFFFFF), int(so[p] >> 24)
        if slot >= k:
            assert tok == T and sw[p] == 0
            continue
        seen[tok, slot] += 1
        assert ids[tok, slot] == se[p // Bm]
        assert w[tok, slot] == sw[p]
    assert (seen == 1).all()
    assert (np.diff(se[: n // Bm].astype(np.int64)) >= 0).all()


def test_num_local_tokens():
    rng = np.random.default_rng(6)
    ids, w = _rand_case(rng, 40, 4, 16)
    a = sorting.moe_sorting_ref(ids, w, 16, 8, num_local_tokens=25)
    b = sorting.moe_sorting_ref(ids[:25], w[:25], 16, 8)
    n = int(b[3][0])
    assert a[3][0] == n and a[3][1] == 25
    assert (a[0][:n] == b[0][:n]).all() and (a[1][:n] == b[1][:n]).all()
    assert a[0].size == sorting.max_blocks(40 * 4, 16, 8) * 8       # buffers sized for all rows
