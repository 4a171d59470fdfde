"""The kernels launched from their code objects (pyhip_amd/co/*.co) through hipModuleLaunchKernel with a packed
argument struct, the way the reference's own loader launches kernels (src/core/hiptools.py:54-100), against the same
work done through libpyhip_moe.so: bit for bit."""
import ctypes

import pytest
import torch

from pyhip_amd import _lib, co_module as co
from pyhip_amd.moe_sorting import moe_sorting
import cases

pytestmark = pytest.mark.gpu
P = lambda t: ctypes.c_void_p(t.data_ptr())


def test_quantiser_and_reduction_from_code_objects():
    lib = _lib.load()
    g = torch.Generator().manual_seed(3)
    rows, K = 77, 1536
    x = torch.randn(rows, K, generator=g).to(torch.bfloat16).cuda()
    print("code-object case: act_quant rows=77 K=1536", flush=True)
    SK = lib.pyhip_moe_act_scale_stride(K)
    q0 = torch.empty(rows, K // 2, dtype=torch.uint8, device="cuda"); s0 = torch.zeros(rows, SK, dtype=torch.uint8, device="cuda")
    q1, s1 = torch.empty_like(q0), torch.zeros_like(s0)
    _lib.check(lib.pyhip_moe_act_quant_mxfp4(P(x), K, rows, K, P(q0), P(s0), None, _lib.current_stream()))
    qa = co.QuantArgs(x=x.data_ptr(), ldx=K, q=q1.data_ptr(), s=s1.data_ptr(), rows=rows, K=K, SK=SK, rows_limit=None)
    co.Module("moe_quant").kernel("moe_act_quant_mxfp4_kernel")([(rows * SK + 255) // 256], [256], qa)
    torch.cuda.synchronize()
    assert torch.equal(q0, q1) and torch.equal(s0, s1)

    T, k, H, E = 19, 4, 1024, 16
    print("code-object case: routed top-k reduce T=19 k=4 H=1024", flush=True)
    out3 = torch.randn(T, k, H, generator=g).to(torch.bfloat16).cuda()
    ids = torch.randint(-1, E + 1, (T, k), generator=g, dtype=torch.int32).cuda()
    o0 = torch.empty(T, H, dtype=torch.bfloat16, device="cuda"); o1 = torch.empty_like(o0)
    _lib.check(lib.pyhip_moe_topk_reduce_routed(P(out3), P(o0), T, k, H, 0, P(ids), E, None, None, _lib.current_stream()))
    rt = co.ReduceRouting(topk_ids=ids.data_ptr(), expert_mask=None, num_local_tok=None, experts=E)
    co.Module("moe_reduce").kernel(co.reduce_kernel_name(False, True))(
        [(T * (H // 8) + 255) // 256], [256], out3, o1, ctypes.c_longlong(T), k, H // 8, None, rt)
    torch.cuda.synchronize()
    assert torch.equal(o0, o1)


@pytest.mark.parametrize("name,T,bm", [("tiny", 300, 128), ("dsv3_s", 16, 16)])
def test_down_gemm_from_code_object(name, T, bm):
    """the stage-2 grouped GEMM: GemmArgs filled by hand, persistent grid sized by the caller"""
    lib = _lib.load()
    from pyhip_amd import fused_moe
    L = cases.make_layer(name, T, seed=23)
    w1, w1s, w2, w2s = cases.device_weights(L)
    tw, ti = torch.from_numpy(L.topk_w).cuda(), torch.from_numpy(L.topk_ids).cuda()
    print(f"code-object case: down GEMM {name} T={T} bm={bm}", flush=True)
    _, parts = fused_moe(L.hidden.cuda(), w1, w2, tw, ti, w1_scale=w1s, w2_scale=w2s, block_size_M=bm, method="a4w4",
                         return_parts=True)
    so, sw, se, nv, _, sched = moe_sorting(ti, tw, L.E, L.H, torch.bfloat16, bm, alloc_moe_out=False, return_schedule=True)
    assert torch.equal(so, parts["sorted_ids"])
    n_blk = se.numel()
    K, N = L.I, L.H
    out3 = torch.zeros(T, L.k, N, dtype=torch.bfloat16, device="cuda")
    args = co.GemmArgs(a_q=parts["a2_q"].data_ptr(), a_s=parts["a2_s"].data_ptr(), w=w2.data_ptr(), w_s=w2s.data_ptr(),
                       bias=None, sorted_ids=so.data_ptr(), sorted_w=sw.data_ptr(), sorted_e=se.data_ptr(),
                       num_valid=nv.data_ptr(), sched=sched.data_ptr() if K >= 1024 else None, out=out3.data_ptr(),
                       out_q=None, out_s=None, OSK=0, limit=0.0, T=T, topk=L.k, K=K, N=N, SK=(K + 511) // 512 * 16,
                       SC=(K // 32 + 7) // 8 * 8, n_blk=n_blk, n_tiles=N // 256, a_rows=n_blk * bm, E=L.E)
    tiles = n_blk * (N // 256)
    grid = tiles if K < 1024 else min((tiles + 7) // 8 * 8, 512)
    co.Module("moe_gemm_mxfp4").kernel(co.gemm_kernel_name(2, bm // 16))([grid], [256], args)
    torch.cuda.synchronize()
    written = parts["out3"].clone()
    # (token, slot) pairs the sort dropped are not written by either path: compare what was routed
    assert torch.equal(out3, written)
