"""The entry point that allocates nothing (pyhip_moe_forward_static: the library's own device array is the
workspace) against pyhip_moe_forward with a caller-provided workspace, through the C ABI: same kernels, same
order, so the outputs must agree bit for bit; two calls in a row, the second with a smaller input, so that what
the first call left in the shared array is seen not to matter.  Calls beyond the array's size are refused."""
import ctypes

import pytest
import torch

from pyhip_amd import _lib
import cases

pytestmark = pytest.mark.gpu



def _static_fn(lib):
    return lib.pyhip_moe_forward_static, lib.pyhip_moe_forward_static_capacity


def _both(lib, L, dev_w, w4a16, bm, nl=None):
    fn, _ = _static_fn(lib)
    w1, w1s, w2, w2s = dev_w
    hidden = L.hidden.cuda()
    tw, ti = torch.from_numpy(L.topk_w).cuda(), torch.from_numpy(L.topk_ids).cuda()
    T, H, I, E, k = L.T, L.H, L.I, L.E, L.k
    stream = _lib.current_stream()
    common = (_lib.dptr(hidden), H, _lib.dptr(w1), _lib.dptr(w1s), _lib.dptr(w2), _lib.dptr(w2s), None, None,
              _lib.dptr(ti), _lib.dptr(tw), None, _lib.dptr(nl))
    tail = (0, T, k, E, H, I, 0, 0, bm, w4a16, 0, 0, 0.0)
    out_a = torch.empty(T, H, dtype=torch.bfloat16, device="cuda")
    out_b = torch.full((T, H), float("nan"), dtype=torch.bfloat16, device="cuda")
    ws_bytes = lib.pyhip_moe_forward_workspace_bytes(T, k, E, H, I, bm, w4a16)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device="cuda")
    _lib.check(lib.pyhip_moe_forward(*common, _lib.dptr(out_a), *tail, _lib.dptr(ws), ws_bytes, stream), "moe_forward")
    _lib.check(fn(*common, _lib.dptr(out_b), *tail, stream), "moe_forward_static")
    torch.cuda.synchronize()
    return out_a, out_b


@pytest.mark.parametrize("w4a16", [0, 1])
def test_static_scratch_entry_point_matches_workspace_entry_point(w4a16):
    lib = _lib.load()
    big = cases.make_layer("dsv3_s", 96 if not w4a16 else 24, seed=31)
    small = cases.make_layer("dsv3_s", 5, seed=32)
    wb, wsm = cases.device_weights(big), cases.device_weights(small)
    for L, w in ((big, wb), (small, wsm)):          # second call: smaller input over the first call's leftovers
        print(f"static-scratch case dsv3_s T={L.T} w4a16={w4a16}", flush=True)
        a, b = _both(lib, L, w, w4a16, 16)
        assert torch.isfinite(a.float()).all()
        assert torch.equal(a, b)
    # a device-side token limit, as a captured decode step would use it
    nl = torch.tensor([3], dtype=torch.int32, device="cuda")
    a, b = _both(lib, small, wsm, w4a16, 16, nl)
    assert torch.equal(a, b) and (b[3:] == 0).all()


def test_static_scratch_entry_point_rejects_oversized_calls():
    lib = _lib.load()
    fn, cap = _static_fn(lib)
    assert cap() == 64 << 20
    one = ctypes.c_void_p(256)
    # DeepSeek-V3 shape, 8192 tokens: far more intermediates than the array holds; refused before anything is launched
    rc = fn(one, 7168, one, one, one, one, None, None, one, one, None, None, one, 0, 8192, 8, 256, 7168, 2048, 0, 0, 128, 0, 0, 0,
            0.0, None)
    assert rc == 1 and b"scratch array holds" in lib.pyhip_moe_last_error()


def _prepared_call(lib, L, dev_w, w4a16, bm):
    """everything the static entry point needs, allocated up front; returns (call, out)"""
    fn, cap = _static_fn(lib)
    cap()                                         # maps the library's array on this device, outside any capture
    w1, w1s, w2, w2s = dev_w
    hidden = L.hidden.cuda()
    tw, ti = torch.from_numpy(L.topk_w).cuda(), torch.from_numpy(L.topk_ids).cuda()
    out = torch.full((L.T, L.H), float("nan"), dtype=torch.bfloat16, device="cuda")
    keep = (hidden, tw, ti, w1, w1s, w2, w2s)
    args = (_lib.dptr(hidden), L.H, _lib.dptr(w1), _lib.dptr(w1s), _lib.dptr(w2), _lib.dptr(w2s), None, None,
            _lib.dptr(ti), _lib.dptr(tw), None, None, _lib.dptr(out), 0, L.T, L.k, L.E, L.H, L.I, 0, 0, bm, w4a16, 0, 0, 0.0)

    def call():
        _lib.check(fn(*args, _lib.current_stream()), "moe_forward_static")
    call.keep = keep
    return call, out


@pytest.mark.parametrize("w4a16", [0, 1])
def test_static_scratch_entry_point_allocates_nothing(w4a16):
    """device memory in use (the driver's count of free bytes and torch's own count) does not move across calls"""
    lib = _lib.load()
    L = cases.make_layer("dsv3_s", 24, seed=33)
    call, out = _prepared_call(lib, L, cases.device_weights(L), w4a16, 16)
    call()                                        # (first launch of these kernels in the process may load their code)
    torch.cuda.synchronize()
    free0, alloc0, reserved0 = torch.cuda.mem_get_info()[0], torch.cuda.memory_allocated(), torch.cuda.memory_reserved()
    for _ in range(3):
        call()
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free0
    assert torch.cuda.memory_allocated() == alloc0 and torch.cuda.memory_reserved() == reserved0
    assert torch.isfinite(out.float()).all()


@pytest.mark.parametrize("w4a16", [0, 1])
def test_static_scratch_entry_point_under_graph_capture(w4a16):
    """the call captured in a HIP graph and replayed, with eager work and synchronisations between the replays: every
    replay must reproduce the eager result bit for bit"""
    lib = _lib.load()
    L = cases.make_layer("dsv3_s", 24, seed=34)
    call, out = _prepared_call(lib, L, cases.device_weights(L), w4a16, 16)
    call()
    torch.cuda.synchronize()
    eager = out.clone()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        call()                                    # warm-up on the capture stream
        side.synchronize()
        with torch.cuda.graph(graph, stream=side):
            call()
    torch.cuda.current_stream().wait_stream(side)
    for i in range(3):
        out.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager), "replay %d differs" % i
        scribble = torch.randn(1 << 20, device="cuda").sum()     # the program's own eager work between replays
        torch.cuda.synchronize()
        assert torch.isfinite(scribble)
