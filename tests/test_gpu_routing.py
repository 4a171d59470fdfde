"""GPU routers against the oracle's routers (float64 on the CPU).  The kernels work in fp32, so a pick may
differ from the oracle's only where two scores are closer than fp32 can tell apart: ids must match wherever
the oracle's k-th and (k+1)-th score and all neighbouring picks differ by more than 1e-5 relative; weights must
match to 1e-5 relative."""
import numpy as np
import pytest
import torch

from oracle import routing as oroute
from pyhip_amd import routing

pytestmark = pytest.mark.gpu


def _check(w, ids, rw, rids, scores):
    w, ids = w.cpu().numpy(), ids.cpu().numpy()
    T, k = rids.shape
    srt = -np.sort(-scores, axis=-1)
    gaps = np.abs(srt[:, :k] - srt[:, 1:k + 1]) / np.maximum(np.abs(srt[:, :k]), 1e-30)
    clear = (gaps > 1e-5).all(axis=-1)                    # rows where fp32 cannot reorder anything
    assert clear.mean() > 0.95
    assert (ids[clear] == rids[clear]).all()
    np.testing.assert_allclose(w[clear], rw[clear], rtol=1e-5, atol=1e-8)
    for t in range(T):                                    # every row: k distinct experts in range
        assert len(set(ids[t].tolist())) == k and ids[t].min() >= 0 and ids[t].max() < scores.shape[1]


@pytest.mark.parametrize("T,E,k,renorm", [(64, 8, 2, True), (33, 128, 8, True), (1000, 256, 8, True), (7, 64, 4, False),
                                          (5, 400, 20, True), (16, 2048, 32, True)])
def test_softmax_topk(T, E, k, renorm):
    g = torch.Generator().manual_seed(T + E)
    logits = torch.randn(T, E, generator=g)
    print(f"router softmax T={T} E={E} k={k}", flush=True)
    w, ids = routing.fused_topk(None, logits.cuda(), k, renorm)
    torch.cuda.synchronize()
    rw, rids = oroute.softmax_topk(logits.numpy(), k, renormalize=renorm)
    x = logits.double().numpy()
    p = np.exp(x - x.max(-1, keepdims=True))
    _check(w, ids, rw, rids, p / p.sum(-1, keepdims=True))


@pytest.mark.parametrize("T,E,k,ng,tg", [(128, 256, 8, 8, 4), (9, 64, 4, 4, 2), (50, 128, 6, 8, 3), (3, 1024, 8, 16, 4)])
def test_grouped_sigmoid_topk(T, E, k, ng, tg):
    g = torch.Generator().manual_seed(T * 3 + E)
    logits = torch.randn(T, E, generator=g)
    print(f"router grouped T={T} E={E} k={k} groups={ng}/{tg}", flush=True)
    w, ids = routing.grouped_topk(logits.cuda(), k, True, ng, tg)
    torch.cuda.synchronize()
    rw, rids = oroute.grouped_sigmoid_topk(logits.numpy(), k, ng, tg)
    s = 1.0 / (1.0 + np.exp(-logits.double().numpy()))
    # masked scores as the oracle ranks them
    gs = np.sort(s.reshape(T, ng, E // ng), axis=-1)[..., -2:].sum(-1)
    gsel = np.argsort(-gs, axis=-1, kind="stable")[:, :tg]
    mask = np.zeros((T, ng), bool)
    np.put_along_axis(mask, gsel, True, axis=-1)
    masked = np.where(np.repeat(mask, E // ng, axis=1), s, 0.0)
    _check(w, ids, rw, rids, masked)
    got_groups = ids.cpu().numpy() // (E // ng)
    for t in range(T):
        assert set(got_groups[t].tolist()) <= set(gsel[t].tolist())


def test_routed_layer_end_to_end():
    """router -> fused_moe on the device equals the same layer with the oracle's routing"""
    import cases
    from pyhip_amd import fused_moe
    L = cases.make_layer("dsv3_s", 40, seed=6)
    g = torch.Generator().manual_seed(6)
    logits = torch.randn(40, L.E, generator=g)
    w, ids = routing.grouped_topk(logits.cuda(), L.k, True, 8, 4)
    rw, rids = oroute.grouped_sigmoid_topk(logits.numpy(), L.k, 8, 4)
    assert (ids.cpu().numpy() == rids).all()
    w1, w1s, w2, w2s = cases.device_weights(L)
    a = fused_moe(L.hidden.cuda(), w1, w2, w, ids, w1_scale=w1s, w2_scale=w2s, method="a4w4", dtype=torch.float32)
    b = fused_moe(L.hidden.cuda(), w1, w2, torch.from_numpy(rw).cuda(), torch.from_numpy(rids).cuda(), w1_scale=w1s,
                  w2_scale=w2s, method="a4w4", dtype=torch.float32)
    torch.cuda.synchronize()
    rms = b.float().pow(2).mean().sqrt().item()
    assert (a - b).abs().max().item() <= 1e-4 * rms          # only the fp32 routing weights differ


@pytest.mark.parametrize("T,router,method", [(1, "grouped", "w4a16"), (16, "grouped", "auto"), (64, "softmax", "a4w4"),
                                             (65, "softmax", "a4w4"), (300, "grouped", "a4w4")])
def test_router_inside_the_layer_call(T, router, method):
    """fused_moe_routed (router + sort + GEMMs + reduce behind one library call; up to 64 tokens the sort's own
    workgroup routes the tokens, beyond that the router has its launch) gives, bit for bit, the picks of the
    stand-alone router and the output of fused_moe on those picks."""
    import cases
    from pyhip_amd import fused_moe, fused_moe_routed
    L = cases.make_layer("dsv3_s", T, seed=7)                          # E=64, top-8
    g = torch.Generator().manual_seed(70 + T)
    logits = torch.randn(T, L.E, generator=g).cuda()
    w1, w1s, w2, w2s = cases.device_weights(L)
    print(f"routed-layer case T={T} router={router} method={method}", flush=True)
    if router == "grouped":
        w, ids = routing.grouped_topk(logits, L.k, True, 8, 4)
        kw = dict(num_expert_group=8, topk_group=4)
    else:
        w, ids = routing.fused_topk(None, logits, L.k, True)
        kw = {}
    ref = fused_moe(L.hidden.cuda(), w1, w2, w, ids, w1_scale=w1s, w2_scale=w2s, method=method)
    out, tw, ti = fused_moe_routed(L.hidden.cuda(), w1, w2, logits, L.k, True, w1_scale=w1s, w2_scale=w2s, method=method,
                                   return_routing=True, **kw)
    torch.cuda.synchronize()
    assert torch.equal(ti, ids) and torch.equal(tw, w)
    assert torch.equal(out, ref) and torch.isfinite(out.float()).all()
