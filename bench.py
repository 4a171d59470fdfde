#!/usr/bin/env python3
"""Benchmark of the MXFP4 fused-MoE operator on ONE MI355X.

A step is one ``fused_moe`` call (sort -> quantise -> gate_up GEMM -> quantise -> down GEMM -> top-k
reduce) on synthetic inputs that are resident in HBM.  Prints one JSON line.

  value     TFLOP/s of the whole layer at --tokens (default 8192), FLOPs = 6*T*k*I*H
  decode    the same layer at --decode-tokens (default 16): ms, HBM GB/s on algorithmic bytes (method="auto":
            bf16 activations x MXFP4 weights at this size)
            bf16 activations x MXFP4 weights at this size); graph_replay_ms_per_step is the same call captured in
            a HIP graph and replayed
  decode_a4w4  the same with MXFP4 activations forced (method="a4w4")
  sweep     the same layer at --sweep-tokens (default 128, 1024, 4096): ms, TFLOP/s and GB/s on algorithmic work
  roofline  the dominant kernel (stage-1 gate_up GEMM) of the primary workload, timed with events
            recorded around it inside the timed steps (every fourth one)
  cpu_baseline  the CPU oracle (oracle/moe.py) on a bounded sample of the same workload
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_MFMA_FP4_TFLOPS = 10100.0     # MI355X dense MXFP4/MXFP6
PEAK_HBM_GBPS = 8000.0

# HBM-side bytes per launch of the gate_up GEMM, (shape, tokens) -> bytes, from the hardware counters
# FETCH_SIZE (x 2.0: a plain 1 GiB device copy reads 524 288) + WRITE_SIZE (x 1.0), KiB per dispatch,
# collected with `rocprofv3 --pmc` around this script; other workloads report null.
MEASURED_TRAFFIC = {
    ("dsv3", 8192): 3.252e6 * 2 * 1024 + 1.014e5 * 1024,
    ("dsv3", 16): 8.012e5 * 2 * 1024 + 6.765e3 * 1024,
}


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--shape", default="dsv3")
    ap.add_argument("--tokens", type=int, default=8192)
    ap.add_argument("--decode-tokens", type=int, default=16)
    ap.add_argument("--sweep-tokens", type=lambda v: [int(x) for x in v.split(",") if x], default=[128, 1024, 4096],
                    help="further token counts reported in 'sweep' (comma separated; empty = none)")
    ap.add_argument("--block-m", type=int, default=0)
    ap.add_argument("--cpu-seconds", type=float, default=20.0, help="target size of the CPU sample; 0 = skip")
    ap.add_argument("--calibrate-copy", type=int, default=0, metavar="MIB",
                    help="also run 3 plain device copies of MIB mebibytes (a yardstick for HBM traffic counters)")
    return ap.parse_args()


def run_config(torch, fused_moe, W, shape, tokens, steps, warmup, block_m, method="auto"):
    from pyhip_amd import workloads
    hidden, topk_w, topk_ids = workloads.make_inputs(shape, tokens)
    if W["hidden_pad"]:      # padded shapes (gpt-oss): activations at the padded width, as the reference passes them
        hidden = torch.nn.functional.pad(hidden, (0, W["hidden_pad"]))
    kw = dict(w1_scale=W["w1_scale"], w2_scale=W["w2_scale"], bias1=W.get("bias1"), bias2=W.get("bias2"),
              block_size_M=block_m or None, hidden_pad=W["hidden_pad"], intermediate_pad=W["intermediate_pad"],
              method=method)
    for _ in range(warmup):
        out = fused_moe(hidden, W["w1"], W["w2"], topk_w, topk_ids, **kw)
    torch.cuda.synchronize()
    events = []
    t0 = time.perf_counter()
    for i in range(steps):
        # stage events on every fourth timed step: recording one costs several microseconds of GPU time
        out = fused_moe(hidden, W["w1"], W["w2"], topk_w, topk_ids, stage_events=events if i % 4 == 0 else None, **kw)
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    assert torch.isfinite(out.float()).all()
    stage_ms = {}
    for name, a, b in events:
        stage_ms.setdefault(name, []).append(a.elapsed_time(b))
    stage_ms = {k: sum(v) / len(v) for k, v in stage_ms.items()}
    work = workloads.algorithmic_work(shape, tokens, topk_ids)
    return dict(ms=wall * 1e3 / steps, stage_ms=stage_ms, work=work, hidden=hidden, topk_w=topk_w, topk_ids=topk_ids,
                out=out)


def graph_replay_ms(torch, fused_moe, W, res, steps, block_m, method="auto"):
    """the same call captured once in a HIP graph and replayed: what a serving loop that captures its decode step
    pays per layer (no host work between the launches)"""
    kw = dict(w1_scale=W["w1_scale"], w2_scale=W["w2_scale"], bias1=W.get("bias1"), bias2=W.get("bias2"),
              block_size_M=block_m or None, hidden_pad=W["hidden_pad"], intermediate_pad=W["intermediate_pad"],
              method=method)
    args = (res["hidden"], W["w1"], W["w2"], res["topk_w"], res["topk_ids"])
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = fused_moe(*args, **kw)
    for _ in range(5):
        graph.replay()
    torch.cuda.synchronize()
    assert torch.equal(out, res["out"]), "graph replay differs from the eager result"
    t0 = time.perf_counter()
    for _ in range(steps):
        graph.replay()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) * 1e3 / steps


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


def main():
    a = parse()
    if a.gpus != 1:
        print("bench.py: this build runs on one GPU only (--gpus %d requested); expert-parallel sharding over "
              "several GPUs is not built." % a.gpus, file=sys.stderr)
        sys.exit(2)
    import torch
    from pyhip_amd import fused_moe, workloads
    torch.cuda.set_device(0)
    cfg = workloads.SHAPES[a.shape]
    W = workloads.make_weights(a.shape)
    torch.cuda.synchronize()
    main_res = run_config(torch, fused_moe, W, a.shape, a.tokens, a.steps, a.warmup, a.block_m)
    dec = run_config(torch, fused_moe, W, a.shape, a.decode_tokens, max(a.steps, 50), max(a.warmup, 10), a.block_m)
    dec4 = run_config(torch, fused_moe, W, a.shape, a.decode_tokens, max(a.steps, 50), max(a.warmup, 10), a.block_m, "a4w4")
    dec_graph_ms = graph_replay_ms(torch, fused_moe, W, dec, max(a.steps, 50), a.block_m)
    # the same layer at sizes between the two headline points (method and row block chosen by the operator)
    sweep = []
    for t in a.sweep_tokens:
        r = run_config(torch, fused_moe, W, a.shape, t, a.steps, a.warmup, a.block_m)
        sweep.append({"tokens": t, "ms_per_step": round(r["ms"], 4),
                      "tflops": round(r["work"]["flops"] / (r["ms"] * 1e-3) / 1e12, 1),
                      "frac_of_mfma_peak": round(r["work"]["flops"] / (r["ms"] * 1e-3) / 1e12 / PEAK_MFMA_FP4_TFLOPS, 4),
                      "hbm_gbps": round(r["work"]["bytes"] / (r["ms"] * 1e-3) / 1e9, 1),
                      "frac_of_hbm_peak": round(r["work"]["bytes"] / (r["ms"] * 1e-3) / 1e9 / PEAK_HBM_GBPS, 4)})
        del r

    if a.calibrate_copy:
        src = torch.zeros(a.calibrate_copy << 20, dtype=torch.uint8, device="cuda")
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    w = main_res["work"]
    tflops = w["flops"] / (main_res["ms"] * 1e-3) / 1e12
    g1_ms = main_res["stage_ms"]["gemm1"]
    g1_tflops = w["flops_stage1"] / (g1_ms * 1e-3) / 1e12
    dw = dec["work"]
    dec_gbps = dw["bytes"] / (dec["ms"] * 1e-3) / 1e9
    dg1_ms = dec["stage_ms"]["gemm1"]
    out = {
        "metric": "MXFP4 fused-MoE TFLOP/s (DeepSeek-V3 routed-expert layer, %d tokens); decode-size HBM GB/s in 'decode'"
                  % a.tokens if a.shape == "dsv3" else "MXFP4 fused-MoE TFLOP/s (%s, %d tokens)" % (a.shape, a.tokens),
        "value": round(tflops, 2), "unit": "TFLOP/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": round(main_res["ms"], 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "mxfp4 (e2m1 x e2m1, e8m0 1x32 scales, fp32 accumulate)", "data": "synthetic",
        "config": {"workload": "%s E=%d top%d H=%d I=%d T=%d" % (a.shape, cfg["E"], cfg["k"], cfg["H"], cfg["I"], a.tokens),
                   "experts_hit": w["e_hit"], "block_m": a.block_m or "auto"},
        "frac_of_mfma_peak": round(tflops / PEAK_MFMA_FP4_TFLOPS, 4),
        "hbm_gbps": round(w["bytes"] / (main_res["ms"] * 1e-3) / 1e9, 1),
        "stage_ms": {k: round(v, 4) for k, v in main_res["stage_ms"].items()},
        "roofline": {"kernel": "moe_gemm_mxfp4_kernel<1,*> (gate_up)", "bound": "mfma", "achieved": round(g1_tflops, 2),
                     "peak": PEAK_MFMA_FP4_TFLOPS, "unit": "TFLOP/s", "frac": round(g1_tflops / PEAK_MFMA_FP4_TFLOPS, 4),
                     "traffic": MEASURED_TRAFFIC.get((a.shape, a.tokens)), "avg_launch_ms": round(g1_ms, 4),
                     # the other roof of the same kernel (its algorithmic bytes against the HBM peak)
                     "hbm_achieved_gbps": round(w["bytes_stage1"] / (g1_ms * 1e-3) / 1e9, 1),
                     "hbm_frac": round(w["bytes_stage1"] / (g1_ms * 1e-3) / 1e9 / PEAK_HBM_GBPS, 4)},
        "decode": {"tokens": a.decode_tokens, "ms_per_step": round(dec["ms"], 4), "experts_hit": dw["e_hit"],
                   "hbm_gbps": round(dec_gbps, 1), "frac_of_hbm_peak": round(dec_gbps / PEAK_HBM_GBPS, 4),
                   "tflops": round(dw["flops"] / (dec["ms"] * 1e-3) / 1e12, 2),
                   "stage_ms": {k: round(v, 4) for k, v in dec["stage_ms"].items()},
                   "graph_replay_ms_per_step": round(dec_graph_ms, 4),
                   "roofline": {"kernel": "moe_gemm_w4a16_kernel<1,1> (gate_up, bf16 activations)", "bound": "hbm",
                                "achieved": round(dw["bytes_stage1"] / (dg1_ms * 1e-3) / 1e9, 1), "peak": PEAK_HBM_GBPS,
                                "unit": "GB/s",
                                "frac": round(dw["bytes_stage1"] / (dg1_ms * 1e-3) / 1e9 / PEAK_HBM_GBPS, 4),
                                "traffic": MEASURED_TRAFFIC.get((a.shape, a.decode_tokens)),
                                "avg_launch_ms": round(dg1_ms, 4)}},
    }
    out["decode_a4w4"] = {"tokens": a.decode_tokens, "ms_per_step": round(dec4["ms"], 4),
                          "hbm_gbps": round(dw["bytes"] / (dec4["ms"] * 1e-3) / 1e9, 1),
                          "frac_of_hbm_peak": round(dw["bytes"] / (dec4["ms"] * 1e-3) / 1e9 / PEAK_HBM_GBPS, 4),
                          "stage_ms": {k: round(v, 4) for k, v in dec4["stage_ms"].items()}}
    out["sweep"] = sweep
    if a.cpu_seconds > 0:
        out["cpu_baseline"] = cpu_baseline(torch, W, a.shape, main_res, a.cpu_seconds)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
