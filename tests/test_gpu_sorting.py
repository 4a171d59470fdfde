"""GPU parity of the routing sort through the C ABI: bit-exact against the oracle (whole buffers,
including padding and tail entries)."""
import numpy as np
import pytest
import torch

from oracle import sorting
from pyhip_amd import moe_sorting

pytestmark = pytest.mark.gpu


def _ids(rng, T, k, E, skew):
    if skew:
        p = 1.0 / np.arange(1, E + 1) ** 1.1
        p /= p.sum()
        return np.stack([rng.choice(E, size=k, replace=False, p=p) for _ in range(T)]).astype(np.int32)
    return np.stack([rng.permutation(E)[:k] for _ in range(T)]).astype(np.int32)


def _run(ids, w, E, Bm, mask=None, nloc=None):
    dev = "cuda"
    t_ids, t_w = torch.from_numpy(ids).to(dev), torch.from_numpy(w).to(dev)
    t_mask = None if mask is None else torch.from_numpy(mask).to(dev)
    t_nloc = None if nloc is None else torch.tensor([nloc], dtype=torch.int32, device=dev)
    print(f"sort case T={ids.shape[0]} k={ids.shape[1]} E={E} Bm={Bm} mask={mask is not None} nloc={nloc}", flush=True)
    so, sw, se, nv, out = moe_sorting(t_ids, t_w, E, 64, torch.bfloat16, Bm, t_mask, t_nloc)
    torch.cuda.synchronize()
    r_so, r_sw, r_se, r_nv = sorting.moe_sorting_ref(ids, w, E, Bm, expert_mask=mask, num_local_tokens=nloc)
    assert (nv.cpu().numpy().view(np.uint32) == r_nv).all(), (nv, r_nv)
    assert (so.cpu().numpy().view(np.uint32) == r_so).all()
    assert (sw.cpu().numpy() == r_sw).all()
    assert (se.cpu().numpy().view(np.uint32) == r_se).all()
    assert (out == 0).all() and out.shape == (ids.shape[0], 64)


@pytest.mark.parametrize("T,k,E,Bm,skew", [
    (1, 1, 1, 16, False), (1, 8, 256, 16, False), (16, 8, 256, 16, False), (64, 2, 8, 32, False),
    (33, 8, 256, 32, True), (7, 4, 128, 64, False), (200, 8, 32, 64, True), (129, 2, 8, 128, False),
    (512, 8, 256, 128, True), (513, 8, 256, 128, True),
    (256, 8, 256, 64, True),               # 2048 pairs: the largest single-workgroup case
    (257, 8, 256, 64, True),               # first multi-launch case
    (1024, 8, 256, 64, True), (1025, 8, 256, 64, True),
    (4097, 2, 8, 16, False), (2048, 4, 1024, 16, True),
    (40000, 8, 64, 32, True),              # waves of the multi-launch sort take more than one register-load of pairs
    (4096, 2, 8, 256, False), (8192, 8, 256, 256, True), (3000, 4, 128, 16, True), (5000, 20, 400, 32, False),
])
def test_sort_matches_oracle(T, k, E, Bm, skew):
    rng = np.random.default_rng(T * 31 + k * 7 + E)
    _run(_ids(rng, T, k, E, skew), rng.random((T, k), dtype=np.float32), E, Bm)


@pytest.mark.parametrize("T,k,E,Bm", [(40, 4, 16, 16), (700, 8, 64, 32), (2000, 8, 64, 32), (50000, 6, 64, 32)])
def test_sort_expert_mask_and_local_tokens(T, k, E, Bm):
    rng = np.random.default_rng(T)
    ids, w = _ids(rng, T, k, E, False), rng.random((T, k), dtype=np.float32)
    mask = (rng.random(E) < 0.5).astype(np.int32)
    mask[0] = 1
    _run(ids, w, E, Bm, mask=mask)
    _run(ids, w, E, Bm, nloc=T // 2 + 1)
    _run(ids, w, E, Bm, mask=mask, nloc=T // 3)
    _run(ids, w, E, Bm, nloc=0)


def test_sort_all_tokens_one_expert():
    T, k, E, Bm = 1000, 1, 8, 64
    ids = np.full((T, k), 5, dtype=np.int32)
    _run(ids, np.linspace(0, 1, T * k, dtype=np.float32).reshape(T, k), E, Bm)


@pytest.mark.parametrize("T,k,E,Bm,K", [(16, 8, 256, 16, 7168), (200, 8, 64, 32, 1024), (256, 8, 256, 64, 2880 + 192),
                                        (257, 8, 256, 64, 512), (3000, 4, 128, 128, 4096), (1, 1, 8, 16, 32)])
def test_sort_with_quantisation_equals_the_separate_calls(T, k, E, Bm, K):
    """pyhip_moe_sorting_quant carries the input quantisation in the sort's launches (the single-workgroup sort for
    up to 2048 pairs, the scan launch above that): every output must equal the separate calls' bit for bit."""
    from pyhip_amd.fused_moe import act_quant_mxfp4
    rng = np.random.default_rng(T + K)
    ids, w = _ids(rng, T, k, E, True), rng.random((T, k), dtype=np.float32)
    dev = torch.device("cuda")
    t_ids, t_w = torch.from_numpy(ids).to(dev), torch.from_numpy(w).to(dev)
    x_full = (torch.randn(T, K + 64, generator=torch.Generator().manual_seed(T)) * 3).to(torch.bfloat16).to(dev)
    x = x_full[:, :K]                                   # row stride larger than K
    print(f"sort+quant case T={T} k={k} E={E} Bm={Bm} K={K}", flush=True)
    ref = moe_sorting(t_ids, t_w, E, 64, torch.bfloat16, Bm, alloc_moe_out=False, return_schedule=True)
    q_ref, s_ref = act_quant_mxfp4(x)
    got = moe_sorting(t_ids, t_w, E, 64, torch.bfloat16, Bm, alloc_moe_out=False, return_schedule=True, quant_input=x)
    torch.cuda.synchronize()
    nv = int(ref[3][0])
    assert torch.equal(got[3], ref[3])
    assert torch.equal(got[0][:nv], ref[0][:nv]) and torch.equal(got[1][:nv], ref[1][:nv])
    assert torch.equal(got[0], ref[0]) and torch.equal(got[1], ref[1]) and torch.equal(got[2], ref[2])
    assert torch.equal(got[5], ref[5])
    q, s = got[6]
    assert torch.equal(q, q_ref) and torch.equal(s, s_ref)
