#!/usr/bin/env python3
"""Benchmark of the MXFP4 fused-MoE operator on ONE MI355X.

A step is one ``fused_moe`` call (sort -> quantise -> gate_up GEMM -> quantise -> down GEMM -> top-k
reduce) on synthetic inputs that are resident in HBM.  Prints one JSON line.

  value        TFLOP/s of the whole layer at the headline workload (DeepSeek-V3 shape, 8192 tokens),
               FLOPs = 6*T*k*I*H, wall clock over exactly --steps calls of the one-call product path
  configs      every benchmark point (five shapes x their token counts): method and row block the operator
               picked, median and inter-quartile range of the time per call (HIP events around batches of
               back-to-back calls, product path only), TFLOP/s and GB/s on the algorithmic work and both
               roofline fractions.  Layers whose weights fit the 256 MB last-level cache rotate over
               several copies of the weights, as the reference's harness does (src/misc.py:180-273)
  decode       the headline shape at --decode-tokens (default 16), the HBM-bound end of the metric, with the
               same call captured in a HIP graph and replayed; decode_other_method: the kernel family "auto" did
               not pick, forced
  roofline     the dominant kernel (stage-1 gate_up GEMM) of the headline workload: average launch duration
               from HIP events recorded on the launch stream around that launch in a separate, untimed pass
               of the step-by-step path; traffic is read from the committed counter summary under profiles/
  cpu_baseline the CPU oracle (oracle/moe.py) on a bounded sample of the headline workload

Measurement modes.  ``--epilogue-comparison``, ``--tile256-comparison TOKENS`` and ``--calibrate-copy MIB`` are not part
of the default line: each adds one extra object to it (or, for the copy, only extra launches for a counter run) and
exists so that the command lines quoted in ``profiles/*.txt`` run from this file alone.  ``--frontier`` runs nothing of
the layer: it times the probe ``pyhip_moe_probe_mfma_stream`` (the 288-row GEMM's inner loop reduced to its MFMA / LDS /
memory pattern, pyhip_amd/csrc/probe_mfma_stream.hip) and prints one line with what the machine sustains for that
pattern: matrix-pipeline duty and TB/s per variant.
"""
import argparse
import json
import os
import re
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_MFMA_FP4_TFLOPS = 10100.0     # MI355X dense MXFP4/MXFP6
PEAK_HBM_GBPS = 8000.0
LAST_LEVEL_CACHE_BYTES = 256 << 20

# the benchmark points: shape -> token counts
POINTS = {
    "tiny": [64],
    "mixtral": [1, 32, 512, 4096],
    "gptoss": [16, 256, 4096],
    "qwen3": [64, 2048, 8192],
    "dsv3": [16, 128, 1024, 8192],
}
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "fused_moe_dsv3_hbm_traffic.txt")


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--shape", default="dsv3", help="shape of the headline workload")
    ap.add_argument("--tokens", type=int, default=8192)
    ap.add_argument("--decode-tokens", type=int, default=16)
    ap.add_argument("--points", default="all",
                    help="'all', 'none', or a comma separated list like dsv3:16,qwen3:8192 for the 'configs' array")
    ap.add_argument("--block-m", type=int, default=0)
    ap.add_argument("--method", default="auto")
    ap.add_argument("--cpu-seconds", type=float, default=20.0, help="target size of the CPU sample; 0 = skip")
    ap.add_argument("--epilogue-comparison", action="store_true",
                    help="also time the down GEMM with the atomic top-k epilogue against store + reduction")
    ap.add_argument("--tile256-comparison", type=int, default=0, metavar="TOKENS",
                    help="also time the GEMMs of the headline shape at TOKENS tokens on the 128-row tile, the four-wave "
                         "256-row tile and the eight-wave 256-row tile with both operands through LDS")
    ap.add_argument("--calibrate-copy", type=int, default=0, metavar="MIB",
                    help="also run 3 plain device copies of MIB mebibytes (a yardstick for HBM traffic counters)")
    ap.add_argument("--frontier", action="store_true",
                    help="only run the MFMA / HBM-stream probe (six variants of the 288-row GEMM's inner loop) and print "
                         "matrix-pipeline duty and TB/s of each")
    ap.add_argument("--print-kernel-sources-digest", action="store_true",
                    help="print the digest that profiles/fused_moe_dsv3_hbm_traffic.txt records next to its counters, and exit")
    return ap.parse_args()


def call_kwargs(W, block_m, method):
    return dict(w1_scale=W["w1_scale"], w2_scale=W["w2_scale"], bias1=W.get("bias1"), bias2=W.get("bias2"),
                block_size_M=block_m or None, hidden_pad=W["hidden_pad"], intermediate_pad=W["intermediate_pad"],
                method=method)


def weight_copies(torch, W, work):
    """the weights the timed calls rotate over: one set when a call's working set exceeds the last-level cache
    twice over, otherwise enough copies that consecutive calls cannot find their weights cached"""
    if work["bytes"] >= 2 * LAST_LEVEL_CACHE_BYTES:
        return [W]
    total = sum(W[k].numel() * W[k].element_size() for k in ("w1", "w2", "w1_scale", "w2_scale"))
    n = int(min(64, max(2, -(-(3 * LAST_LEVEL_CACHE_BYTES) // max(work["bytes"], 1)))))
    n = int(max(2, min(n, (4 << 30) // max(total, 1))))
    copies = [W]
    for _ in range(n - 1):
        C = dict(W)
        for k in ("w1", "w2", "w1_scale", "w2_scale"):
            C[k] = W[k].clone()
        C["w1"].is_shuffled = C["w2"].is_shuffled = True
        copies.append(C)
    return copies


def time_point(torch, fused_moe, W, shape, tokens, steps, warmup, block_m, method="auto"):
    """-> dict with wall-clock ms over exactly `steps` calls, and median / IQR over event-timed batches; only the
    one-call product path runs inside the timed regions"""
    from pyhip_amd import workloads
    from pyhip_amd.fused_moe import pick_block_m, pick_w4a16
    hidden, topk_w, topk_ids = workloads.make_inputs(shape, tokens)
    if W["hidden_pad"]:      # padded shapes (gpt-oss): activations at the padded width, as the reference passes them
        hidden = torch.nn.functional.pad(hidden, (0, W["hidden_pad"]))
    work = workloads.algorithmic_work(shape, tokens, topk_ids)
    sets = weight_copies(torch, W, work)
    kws = [call_kwargs(C, block_m, method) for C in sets]

    def call(i):
        C = sets[i % len(sets)]
        return fused_moe(hidden, C["w1"], C["w2"], topk_w, topk_ids, **kws[i % len(sets)])

    for i in range(max(warmup, len(sets))):
        out = call(i)
    torch.cuda.synchronize()
    # the first measurements after a pause run at lower clocks (measured: up to 10 % slower): keep the GPU busy for
    # a quarter of a second before timing
    t_busy = time.perf_counter()
    i = 0
    while time.perf_counter() - t_busy < 0.25:
        out = call(i)
        i += 1
        if i % 16 == 0:
            torch.cuda.synchronize()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        out = call(i)
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    assert torch.isfinite(out.float()).all()
    # event-timed batches: enough calls per batch that the events' own cost (microseconds) does not show
    reps = int(max(1, min(64, round(2.0 / max(wall_ms, 1e-3)))))
    batches = 15
    evs = [torch.cuda.Event(enable_timing=True) for _ in range(batches + 1)]
    evs[0].record()
    n = 0
    for b in range(batches):
        for _ in range(reps):
            call(n)
            n += 1
        evs[b + 1].record()
    torch.cuda.synchronize()
    per = sorted(evs[b].elapsed_time(evs[b + 1]) / reps for b in range(batches))
    q = lambda f: per[min(batches - 1, int(f * batches))]
    cfg = workloads.SHAPES[shape]
    Hp = cfg["H"] + W["hidden_pad"]
    w4a16 = method == "w4a16" or (method != "a4w4" and pick_w4a16(tokens, cfg["k"], cfg["E"], Hp))
    bm = block_m or pick_block_m(tokens, cfg["k"], cfg["E"], Hp, w4a16)
    return dict(wall_ms=wall_ms, median_ms=q(0.5), q1_ms=q(0.25), q3_ms=q(0.75), work=work, hidden=hidden,
                topk_w=topk_w, topk_ids=topk_ids, out=out, method="w4a16" if w4a16 else "a4w4",
                block_m=min(bm, 64) if w4a16 else bm, weight_copies=len(sets), calls_per_batch=reps)


def stage_pass(torch, fused_moe, W, res, block_m, method, passes=8):
    """average duration of each launch group of the step-by-step path, from events on the launch stream; untimed
    (not part of any ms_per_step)"""
    kw = call_kwargs(W, block_m, method)
    events = []
    for _ in range(2):
        fused_moe(res["hidden"], W["w1"], W["w2"], res["topk_w"], res["topk_ids"], stage_events=[], **kw)
    for _ in range(passes):
        fused_moe(res["hidden"], W["w1"], W["w2"], res["topk_w"], res["topk_ids"], stage_events=events, **kw)
    torch.cuda.synchronize()
    acc = {}
    for name, a, b in events:
        acc.setdefault(name, []).append(a.elapsed_time(b))
    return {k: sum(v) / len(v) for k, v in acc.items()}


def epilogue_comparison(torch, fused_moe, W, res, block_m, modes=("store", "atomic", "last_arriver")):
    """the tail of the layer three ways, from events in untimed passes of the step-by-step path: down GEMM storing
    out3[T, k, H] + top-k reduction (deterministic, the product path); output clear + down GEMM with packed bf16
    atomics into out[T, H] (the reference's atomic variant); counter set-up + down GEMM whose workgroups also sum a
    token's slots, whoever stores the last one (deterministic, bit-identical to the first)"""
    names = {"store": "down_gemm_store_plus_reduce_ms", "atomic": "clear_plus_down_gemm_atomic_ms",
             "last_arriver": "setup_plus_down_gemm_last_arriver_ms"}
    r = {"block_m": block_m}
    for mode in modes:
        kw = call_kwargs(W, block_m, "a4w4")
        events = []
        for i in range(10):
            fused_moe(res["hidden"], W["w1"], W["w2"], res["topk_w"], res["topk_ids"], topk_reduce=mode,
                      stage_events=events if i >= 2 else [], **kw)
        torch.cuda.synchronize()
        acc = {}
        for name, a, b in events:
            acc.setdefault(name, []).append(a.elapsed_time(b))
        acc = {k: sum(v) / len(v) for k, v in acc.items()}
        r[names[mode]] = round(acc["gemm2"] + acc.get("reduce", 0.0), 4)
    return r


FRONTIER_VARIANTS = ("mfma_only", "plus_lds_reads", "plus_weight_stream", "plus_lds_dma", "weight_stream_half_the_mfmas",
                     "weight_stream_no_mfmas", "all_with_weights_from_l2",
                     "rows128_mfma_plus_lds_reads", "rows128_all_with_weights_from_l2", "rows128_all_with_weight_stream")


def frontier(torch, iters=4000):
    """the probe's six variants, one workgroup per CU: ns per MFMA slot (288 slots per wave and iteration), the share of the
    MFMA-only rate that the matrix pipeline keeps, and the HBM rate of the weight stream (16 KB per wave and iteration)"""
    import ctypes
    from pyhip_amd import _lib
    lib = _lib.load()
    # random bytes: what the matrix pipeline draws depends on the operands, and real MXFP4 weights look like noise
    buf = torch.randint(0, 256, ((1 << 30) + (16 << 20),), dtype=torch.uint8, device="cuda",
                        generator=torch.Generator(device="cuda").manual_seed(0))
    sink = torch.zeros(4, dtype=torch.int32, device="cuda")
    wgs = ctypes.c_int(0)
    out, base = {}, None
    for v, name in enumerate(FRONTIER_VARIANTS):
        def go(n):
            _lib.check(lib.pyhip_moe_probe_mfma_stream(v, iters, _lib.dptr(buf), buf.numel(), _lib.dptr(sink), n,
                                                   ctypes.byref(wgs), _lib.current_stream()), "probe_mfma_stream")
        # the clock settles under sustained load only: half a second of the same launches first, then 16 timed ones
        t0 = time.perf_counter()
        while time.perf_counter() - t0 < 0.5:
            go(4)
            torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        go(16)
        e1.record()
        torch.cuda.synchronize()
        best = e0.elapsed_time(e1) / 16
        # MFMA slots per wave and iteration: 288 (288-row tile), 128 (128-row tile, two waves per SIMD)
        slots = 128.0 if v >= 7 else 288.0
        ns_slot = best * 1e6 / (iters * slots) / (2 if v >= 7 else 1)       # per SIMD
        base = base or ns_slot
        mfmas = {4: 0.5, 5: 0.0}.get(v, 1.0)
        row = {"ms": round(best, 3), "ns_per_mfma_slot": round(ns_slot, 3), "mfma_duty": round(mfmas * base / ns_slot, 4),
               "pflops": round(mfmas * wgs.value * 4 * slots * iters * 65536 / (best * 1e-3) / 1e15, 3)}
        if v in (2, 3, 4, 5, 9):
            row["stream_tbps"] = round(wgs.value * 4 * 16384 * iters / (best * 1e-3) / 1e12, 3)
        if v in (6, 8):
            row["l2_weight_tbps"] = round(wgs.value * 4 * 16384 * iters / (best * 1e-3) / 1e12, 3)
        out[name] = row
    return {"workgroups": wgs.value, "iterations": iters, "variants": out}


def tile256_comparison(torch, fused_moe, W, shape, tokens):
    """gate_up + down GEMM time of the same layer on three tiles (events around the launches of the step-by-step path,
    untimed passes): 128 rows (weights into registers, two workgroups per CU), 256 rows with four waves (weights into
    registers, one wave per SIMD), 256 rows with eight waves and both operands staged through LDS"""
    from pyhip_amd import workloads
    hidden, tw, ti = workloads.make_inputs(shape, tokens)
    if W["hidden_pad"]:
        hidden = torch.nn.functional.pad(hidden, (0, W["hidden_pad"]))
    out, ref = {}, None
    for name, kw in (("rows128_registers", dict(block_size_M=128)), ("rows256_registers_4waves", dict(block_size_M=256)),
                     ("rows256_lds_8waves", dict(operand_staging="lds"))):
        base = call_kwargs(W, 0, "a4w4")
        base.update(kw)
        events = []
        for i in range(10):
            o = fused_moe(hidden, W["w1"], W["w2"], tw, ti, stage_events=events if i >= 2 else [], **base)
        torch.cuda.synchronize()
        ref = o if ref is None else ref
        assert torch.equal(o, ref), "tiles disagree"
        acc = {}
        for nm, a, b in events:
            acc.setdefault(nm, []).append(a.elapsed_time(b))
        out[name] = {k: round(sum(v) / len(v), 4) for k, v in acc.items() if k in ("gemm1", "gemm2")}
    return out


def graph_replay_ms(torch, fused_moe, W, res, steps, block_m, method="auto"):
    """the same call captured once in a HIP graph and replayed: what a serving loop that captures its decode step
    pays per layer (no host work between the launches)"""
    kw = call_kwargs(W, block_m, method)
    args = (res["hidden"], W["w1"], W["w2"], res["topk_w"], res["topk_ids"])
    eager = fused_moe(*args, **kw)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = fused_moe(*args, **kw)
    for _ in range(5):
        graph.replay()
    torch.cuda.synchronize()
    assert torch.equal(out, eager), "graph replay differs from the eager result"
    t0 = time.perf_counter()
    for _ in range(steps):
        graph.replay()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) * 1e3 / steps


KERNEL_SOURCES = ("moe_gemm_mxfp4.hip", "gemm_device.h", "common.h", "quant_device.h")


def kernel_sources_digest():
    """sha256 over the sources the measured GEMM kernels are compiled from"""
    import hashlib
    h = hashlib.sha256()
    for name in KERNEL_SOURCES:
        with open(os.path.join(ROOT, "pyhip_amd", "csrc", name), "rb") as f:
            h.update(f.read())
    return h.hexdigest()


def measured_traffic(kernel_key):
    """HBM-side bytes per launch of a kernel from the committed counter summary (lines of the form
    `traffic_bytes_per_launch <key> <bytes>`, written when the counters were collected, next to a line
    `kernel_sources_sha256 <digest>` of the kernel sources they were collected with).  None when the summary has no
    such line, or when the kernel sources have changed since: a counter reading of other code is not reported."""
    try:
        text = open(TRAFFIC_FILE).read()
    except OSError:
        return None, None
    m = re.search(r"^traffic_bytes_per_launch\s+%s\s+([0-9.eE+]+)" % re.escape(kernel_key), text, re.M)
    c = re.search(r"^collected_at\s+(.+)$", text, re.M)
    d = re.search(r"^kernel_sources_sha256\s+([0-9a-f]{64})", text, re.M)
    if m is None or d is None or d.group(1) != kernel_sources_digest():
        return None, None
    return float(m.group(1)), (c.group(1).strip() if c else None)


class LazyExperts:
    """expert-indexed view that copies one expert's (de-shuffled) bytes from the device on demand"""

    def __init__(self, fetch, shape):
        self.fetch, self.shape = fetch, shape

    def __getitem__(self, e):
        return self.fetch(int(e))


def cpu_baseline(torch, W, shape, res, budget_s):
    """times oracle.moe.moe_ref on the host for as many hit experts as fit the budget"""
    import numpy as np
    from oracle import moe as omoe
    from pyhip_amd import mxfp4, workloads
    cfg = workloads.SHAPES[shape]
    E, H, I, k = cfg["E"], cfg["H"], cfg["I"], cfg["k"]
    flop_dims = I * H                                # FLOPs are counted at the true sizes
    H, I = H + W["hidden_pad"], I + W["intermediate_pad"]
    threads = min(os.cpu_count() or 1, 16)
    torch.set_num_threads(threads)
    w1q = LazyExperts(lambda e: mxfp4.deshuffle_weight(W["w1"][e]).cpu().numpy(), (E, 2 * I, H // 2))
    w2q = LazyExperts(lambda e: mxfp4.deshuffle_weight(W["w2"][e]).cpu().numpy(), (E, H, I // 2))
    w1s = LazyExperts(lambda e: W["w1_scale_plain"][e * 2 * I:(e + 1) * 2 * I].cpu().numpy(), (E,))
    w2s = LazyExperts(lambda e: W["w2_scale_plain"][e * H:(e + 1) * H].cpu().numpy(), (E,))
    ids = res["topk_ids"].cpu().numpy()
    hidden = res["hidden"].float().cpu().numpy()
    tw = res["topk_w"].cpu().numpy()
    b1 = None if "bias1" not in W else W["bias1"].float().cpu().numpy()
    b2 = None if "bias2" not in W else W["bias2"].float().cpu().numpy()
    hit = [int(e) for e in np.unique(ids)]
    done, pairs, t_total = [], 0, 0.0
    for e in hit:
        t0 = time.perf_counter()
        omoe.moe_ref(hidden, w1q, w1s, w2q, w2s, tw, ids, act="a4", bias1=b1, bias2=b2, experts=[e])
        t_total += time.perf_counter() - t0
        done.append(e)
        pairs += int((ids == e).sum())
        if t_total >= budget_s:
            break
    flops = 6.0 * pairs * flop_dims
    return dict(value=flops / t_total / 1e12, unit="TFLOP/s", cores=threads, kind="port",
                sample="%d of %d hit experts (%d of %d token-expert pairs) of the %s T=%d layer, %.1f s; "
                       "includes per-expert weight dequantisation and the quantisation of all activations"
                       % (len(done), len(hit), pairs, ids.size, shape, ids.shape[0], t_total))


def point_record(shape, tokens, r):
    w, ms = r["work"], r["median_ms"]
    tfl = w["flops"] / (ms * 1e-3) / 1e12
    gbs = w["bytes"] / (ms * 1e-3) / 1e9
    return {"shape": shape, "tokens": tokens, "method": r["method"], "block_m": r["block_m"], "experts_hit": w["e_hit"],
            "ms_median": round(ms, 4), "ms_iqr": [round(r["q1_ms"], 4), round(r["q3_ms"], 4)],
            "ms_wall_mean": round(r["wall_ms"], 4), "tflops": round(tfl, 1),
            "frac_of_mfma_peak": round(tfl / PEAK_MFMA_FP4_TFLOPS, 4), "hbm_gbps": round(gbs, 1),
            "frac_of_hbm_peak": round(gbs / PEAK_HBM_GBPS, 4), "weight_copies": r["weight_copies"]}


def main():
    a = parse()
    if a.print_kernel_sources_digest:
        print(kernel_sources_digest())
        return
    if a.frontier:
        import torch
        torch.cuda.set_device(0)
        print(json.dumps({"mfma_hbm_frontier": frontier(torch)}))
        return
    if a.gpus != 1:
        print("bench.py: this build runs on one GPU only (--gpus %d requested); expert-parallel sharding over "
              "several GPUs is not built." % a.gpus, file=sys.stderr)
        sys.exit(2)
    import torch
    from pyhip_amd import fused_moe, workloads
    torch.cuda.set_device(0)
    if a.points == "all":
        points = [(s, t) for s, ts in POINTS.items() for t in ts]
    elif a.points in ("none", ""):
        points = []
    else:
        points = [(p.split(":")[0], int(p.split(":")[1])) for p in a.points.split(",")]

    cfg = workloads.SHAPES[a.shape]
    configs = []
    main_res = dec = None
    shapes = list(dict.fromkeys([s for s, _ in points] + [a.shape]))
    shapes.sort(key=lambda s: s == a.shape)              # the headline shape last: its results feed the rest of the line
    for shape in shapes:
        W = workloads.make_weights(shape)
        torch.cuda.synchronize()
        for s, t in points:
            if s != shape:
                continue
            steps, warm = (a.steps, a.warmup) if t >= 1024 else (max(a.steps, 50), max(a.warmup, 10))
            r = time_point(torch, fused_moe, W, s, t, steps, warm, 0, "auto")
            rec = point_record(s, t, r)
            # where the time goes: launch groups of the step-by-step path, from events in a separate untimed pass
            if rec["method"] == "a4w4" and rec["block_m"] >= 64:
                # how evenly the persistent GEMMs' tiles spread over the 8 XCDs for this routing
                rec["gate_up_tiles_per_xcd"] = workloads.xcd_tile_counts(s, r["topk_ids"], rec["block_m"], W["intermediate_pad"])
            rec["stage_ms_untimed_pass"] = {k: round(v, 4) for k, v in stage_pass(torch, fused_moe, W, r, 0, "auto", 4).items()}
            configs.append(rec)
            del r
        if shape == a.shape:
            # headline: exactly --steps timed calls after --warmup untimed ones
            main_res = time_point(torch, fused_moe, W, a.shape, a.tokens, a.steps, a.warmup, a.block_m, a.method)
            main_stage = stage_pass(torch, fused_moe, W, main_res, a.block_m, a.method)
            dec = time_point(torch, fused_moe, W, a.shape, a.decode_tokens, max(a.steps, 50), max(a.warmup, 10), a.block_m)
            dec_stage = stage_pass(torch, fused_moe, W, dec, a.block_m, "auto")
            other = "a4w4" if dec["method"] == "w4a16" else "w4a16"
            dec4 = time_point(torch, fused_moe, W, a.shape, a.decode_tokens, max(a.steps, 50), max(a.warmup, 10), a.block_m, other)
            dec_graph_ms = graph_replay_ms(torch, fused_moe, W, dec, max(a.steps, 50), a.block_m)
            cpu = cpu_baseline(torch, W, a.shape, main_res, a.cpu_seconds) if a.cpu_seconds > 0 else None
            tile256 = tile256_comparison(torch, fused_moe, W, a.shape, a.tile256_comparison) if a.tile256_comparison else None
            epi = None
            if a.epilogue_comparison:
                epi = {"tokens_%d" % a.tokens: epilogue_comparison(torch, fused_moe, W, main_res, 128),
                       "tokens_%d_rows_288" % a.tokens: epilogue_comparison(torch, fused_moe, W, main_res, 288,
                                                                            ("store", "last_arriver")),
                       "tokens_%d" % a.decode_tokens: epilogue_comparison(torch, fused_moe, W, dec, 16)}
        del W
        torch.cuda.empty_cache()

    if a.calibrate_copy:
        src = torch.zeros(a.calibrate_copy << 20, dtype=torch.uint8, device="cuda")
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    w = main_res["work"]
    tflops = w["flops"] / (main_res["wall_ms"] * 1e-3) / 1e12
    g1_ms = main_stage["gemm1"]
    g1_tflops = w["flops_stage1"] / (g1_ms * 1e-3) / 1e12
    dw = dec["work"]
    dec_gbps = dw["bytes"] / (dec["median_ms"] * 1e-3) / 1e9
    dg1_ms = dec_stage["gemm1"]
    traffic, collected = measured_traffic("gate_up_%s_T%d" % (a.shape, a.tokens))
    dtraffic, _ = measured_traffic("gate_up_%s_T%d" % (a.shape, a.decode_tokens))
    out = {
        "metric": "MXFP4 fused-MoE TFLOP/s (DeepSeek-V3 routed-expert layer, %d tokens); decode-size HBM GB/s in 'decode'"
                  % a.tokens if a.shape == "dsv3" else "MXFP4 fused-MoE TFLOP/s (%s, %d tokens)" % (a.shape, a.tokens),
        "value": round(tflops, 2), "unit": "TFLOP/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": round(main_res["wall_ms"], 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "mxfp4 (e2m1 x e2m1, e8m0 1x32 scales, fp32 accumulate)", "data": "synthetic",
        "config": {"workload": "%s E=%d top%d H=%d I=%d T=%d" % (a.shape, cfg["E"], cfg["k"], cfg["H"], cfg["I"], a.tokens),
                   "experts_hit": w["e_hit"], "method": main_res["method"], "block_m": main_res["block_m"]},
        "ms_median": round(main_res["median_ms"], 4), "ms_iqr": [round(main_res["q1_ms"], 4), round(main_res["q3_ms"], 4)],
        "frac_of_mfma_peak": round(tflops / PEAK_MFMA_FP4_TFLOPS, 4),
        "hbm_gbps": round(w["bytes"] / (main_res["wall_ms"] * 1e-3) / 1e9, 1),
        "frac_of_hbm_peak": round(w["bytes"] / (main_res["wall_ms"] * 1e-3) / 1e9 / PEAK_HBM_GBPS, 4),
        "stage_ms_untimed_pass": {k: round(v, 4) for k, v in main_stage.items()},
        "roofline": {"kernel": "moe_gemm_mxfp4_kernel<1,*> (gate_up)", "bound": "mfma", "achieved": round(g1_tflops, 2),
                     "peak": PEAK_MFMA_FP4_TFLOPS, "unit": "TFLOP/s", "frac": round(g1_tflops / PEAK_MFMA_FP4_TFLOPS, 4),
                     "traffic": traffic, "traffic_source": None if traffic is None else
                     "profiles/%s (%s)" % (os.path.basename(TRAFFIC_FILE), collected or "commit not recorded"),
                     "avg_launch_ms": round(g1_ms, 4),
                     # the other roof of the same kernel (its algorithmic bytes against the HBM peak)
                     "hbm_achieved_gbps": round(w["bytes_stage1"] / (g1_ms * 1e-3) / 1e9, 1),
                     "hbm_frac": round(w["bytes_stage1"] / (g1_ms * 1e-3) / 1e9 / PEAK_HBM_GBPS, 4)},
        "decode": {"tokens": a.decode_tokens, "method": dec["method"], "block_m": dec["block_m"],
                   "ms_per_step": round(dec["median_ms"], 4), "ms_iqr": [round(dec["q1_ms"], 4), round(dec["q3_ms"], 4)],
                   "ms_wall_mean": round(dec["wall_ms"], 4), "experts_hit": dw["e_hit"],
                   "hbm_gbps": round(dec_gbps, 1), "frac_of_hbm_peak": round(dec_gbps / PEAK_HBM_GBPS, 4),
                   "tflops": round(dw["flops"] / (dec["median_ms"] * 1e-3) / 1e12, 2),
                   "stage_ms_untimed_pass": {k: round(v, 4) for k, v in dec_stage.items()},
                   "graph_replay_ms_per_step": round(dec_graph_ms, 4),
                   "roofline": {"kernel": "moe_gemm_w4a16_kernel<1,1> (gate_up, bf16 activations)" if dec["method"] == "w4a16"
                                else "moe_gemm_mxfp4_kernel<1,1,0,true> (gate_up, MXFP4 activations)", "bound": "hbm",
                                "achieved": round(dw["bytes_stage1"] / (dg1_ms * 1e-3) / 1e9, 1), "peak": PEAK_HBM_GBPS,
                                "unit": "GB/s",
                                "frac": round(dw["bytes_stage1"] / (dg1_ms * 1e-3) / 1e9 / PEAK_HBM_GBPS, 4),
                                "traffic": dtraffic, "avg_launch_ms": round(dg1_ms, 4)}},
        "decode_other_method": {"tokens": a.decode_tokens, "method": dec4["method"], "ms_per_step": round(dec4["median_ms"], 4),
                        "hbm_gbps": round(dw["bytes"] / (dec4["median_ms"] * 1e-3) / 1e9, 1),
                        "frac_of_hbm_peak": round(dw["bytes"] / (dec4["median_ms"] * 1e-3) / 1e9 / PEAK_HBM_GBPS, 4)},
        "configs": configs,
    }
    if epi is not None:
        out["down_epilogue_comparison"] = epi
    if tile256:
        out["tile256_comparison_ms"] = {"tokens": a.tile256_comparison, **tile256}
    if cpu is not None:
        out["cpu_baseline"] = cpu
    print(json.dumps(out))


if __name__ == "__main__":
    main()
