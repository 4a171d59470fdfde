"""Synthetic MoE layers of the benchmark shapes (weights generated on the device, inputs and routing on the CPU) and
the routers that produce ``topk_weight`` / ``topk_ids``.  Used by ``bench.py`` and the large-size GPU tests.

Shapes (experts, top-k, hidden, intermediate):
  tiny 8/2/1024/512, Mixtral-8x7B 8/2/4096/14336, gpt-oss-120b 128/4/2880/2880 (+biases),
  Qwen3-235B-A22B 128/8/4096/1536 (Zipf-skewed router), DeepSeek-V3 256/8/7168/2048 (sigmoid scores,
  8 groups, top-4 groups).  Weights ~N(0, 0.02) quantised to MXFP4; activations bf16 ~N(0, 1).
"""
import math

import torch

from . import mxfp4

SHAPES = {
    "tiny": dict(E=8, k=2, H=1024, I=512, router="softmax"),
    "mixtral": dict(E=8, k=2, H=4096, I=14336, router="softmax"),
    "gptoss": dict(E=128, k=4, H=2880, I=2880, router="softmax", bias=True),
    "qwen3": dict(E=128, k=8, H=4096, I=1536, router="zipf"),
    "dsv3": dict(E=256, k=8, H=7168, I=2048, router="grouped"),
}


def softmax_topk(logits, k):
    p = torch.softmax(logits.double(), dim=-1)
    w, ids = torch.topk(p, k, dim=-1)
    w = w / w.sum(-1, keepdim=True)
    return w.float().contiguous(), ids.to(torch.int32).contiguous()


def grouped_sigmoid_topk(logits, k, n_group=8, topk_group=4):
    """DeepSeek-V3 routing: sigmoid scores; groups ranked by the sum of their two best scores;
    top-k experts inside the best ``topk_group`` groups; weights renormalised."""
    T, E = logits.shape
    s = torch.sigmoid(logits.double())
    gs = s.view(T, n_group, E // n_group).topk(2, dim=-1).values.sum(-1)
    gsel = gs.topk(topk_group, dim=-1).indices
    gmask = torch.zeros(T, n_group, dtype=torch.bool, device=logits.device).scatter_(1, gsel, True)
    masked = s.masked_fill(~gmask.repeat_interleave(E // n_group, dim=1), float("-inf"))
    ids = masked.topk(k, dim=-1).indices
    w = s.gather(1, ids)
    w = w / w.sum(-1, keepdim=True)
    return w.float().contiguous(), ids.to(torch.int32).contiguous()


def route(shape, logits):
    cfg = SHAPES[shape] if isinstance(shape, str) else shape
    E, k = cfg["E"], cfg["k"]
    if cfg["router"] == "softmax":
        return softmax_topk(logits, k)
    if cfg["router"] == "zipf":
        zb = -1.1 * torch.log(torch.arange(1, E + 1, dtype=torch.float64, device=logits.device))
        return softmax_topk(logits.double() + (zb - zb.mean())[None, :], k)
    return grouped_sigmoid_topk(logits, k)


def make_weights(shape, device="cuda", seed=0, experts_per_chunk=8):
    """-> dict(w1, w1_scale, w2, w2_scale[, bias1, bias2]) in the layouts ``fused_moe`` takes.
    Weights are drawn and quantised chunk by chunk; fp32 copies of all experts never coexist."""
    cfg = SHAPES[shape] if isinstance(shape, str) else shape
    E, H, I = cfg["E"], cfg["H"], cfg["I"]
    Hp, Ip = mxfp4.pad_to(H), mxfp4.pad_to(I)      # the GEMMs tile K by 512: gpt-oss 2880 -> 3072
    g = torch.Generator(device=device).manual_seed(seed)
    w1 = torch.empty(E, 2 * Ip, Hp // 2, dtype=torch.uint8, device=device)
    w2 = torch.empty(E, Hp, Ip // 2, dtype=torch.uint8, device=device)
    s1 = torch.empty(E * 2 * Ip, Hp // 32, dtype=torch.uint8, device=device)
    s2 = torch.empty(E * Hp, Ip // 32, dtype=torch.uint8, device=device)
    for e0 in range(0, E, experts_per_chunk):
        e1 = min(E, e0 + experts_per_chunk)
        q1, sc1 = mxfp4.quantize_mxfp4(torch.randn(e1 - e0, 2 * I, H, generator=g, device=device) * 0.02)
        q2, sc2 = mxfp4.quantize_mxfp4(torch.randn(e1 - e0, H, I, generator=g, device=device) * 0.02)
        q1, sc1, q2, sc2 = mxfp4.pad_layer_weights(q1, sc1, q2, sc2)[:4]
        w1[e0:e1] = mxfp4.shuffle_weight(q1)
        s1[e0 * 2 * Ip:e1 * 2 * Ip] = sc1.reshape(-1, Hp // 32)
        w2[e0:e1] = mxfp4.shuffle_weight(q2)
        s2[e0 * Hp:e1 * Hp] = sc2.reshape(-1, Ip // 32)
        del q1, sc1, q2, sc2
    w1.is_shuffled = True
    w2.is_shuffled = True
    out = dict(w1=w1, w2=w2, w1_scale=mxfp4.e8m0_shuffle(s1), w2_scale=mxfp4.e8m0_shuffle(s2),
               w1_scale_plain=s1, w2_scale_plain=s2, hidden_pad=Hp - H, intermediate_pad=Ip - I)
    if cfg.get("bias"):
        b1 = (torch.randn(E, 2 * I, generator=g, device=device) * 0.01).to(torch.bfloat16)
        b2 = (torch.randn(E, H, generator=g, device=device) * 0.01).to(torch.bfloat16)
        out["bias1"] = torch.zeros(E, 2 * Ip, dtype=torch.bfloat16, device=device)
        out["bias1"][:, :I], out["bias1"][:, Ip:Ip + I] = b1[:, :I], b1[:, I:]
        out["bias2"] = torch.nn.functional.pad(b2, (0, Hp - H))
    return out


def make_inputs(shape, tokens, device="cuda", seed=1):
    """hidden states and routing of a call, drawn with a CPU generator and routed on the CPU, so that any machine
    reproduces them bit for bit (the weights, gigabytes of them, are drawn on the device: see make_weights)"""
    cfg = SHAPES[shape] if isinstance(shape, str) else shape
    g = torch.Generator().manual_seed(seed)
    hidden = torch.randn(tokens, cfg["H"], generator=g).to(torch.bfloat16)
    logits = torch.randn(tokens, cfg["E"], generator=g)
    topk_w, topk_ids = route(cfg, logits)
    return hidden.to(device), topk_w.to(device), topk_ids.to(device)


def algorithmic_work(shape, tokens, topk_ids):
    """FLOPs and HBM bytes a perfectly fused layer would need:
    FLOPs = 6*T*k*I*H; bytes = E_hit*3*I*H*(1/2+1/32) + 4*T*H + 8*T*k."""
    cfg = SHAPES[shape] if isinstance(shape, str) else shape
    k, H, I = cfg["k"], cfg["H"], cfg["I"]
    e_hit = int(torch.unique(topk_ids).numel())
    flops = 6.0 * tokens * k * I * H
    byts = e_hit * 3.0 * I * H * (0.5 + 1.0 / 32) + 4.0 * tokens * H + 8.0 * tokens * k
    return dict(flops=flops, bytes=byts, e_hit=e_hit,
                flops_stage1=4.0 * tokens * k * I * H, flops_stage2=2.0 * tokens * k * I * H,
                bytes_stage1=e_hit * 2.0 * I * H * (0.5 + 1.0 / 32) + tokens * H * (0.5 + 1.0 / 32),
                bytes_stage2=e_hit * 1.0 * I * H * (0.5 + 1.0 / 32) + tokens * k * I * (0.5 + 1.0 / 32))


def xcd_tile_counts(shape, topk_ids, block_m, pad=0):
    """gate_up tiles per XCD for a routing: under the grouped GEMMs' schedule (the list expert -> weight tile -> row
    block cut into 8 equal runs) and, for comparison, with whole experts dealt to the XCDs round-robin (e % 8)"""
    cfg = SHAPES[shape] if isinstance(shape, str) else shape
    cnt = torch.bincount(topk_ids.flatten().long().clamp(0, cfg["E"] - 1), minlength=cfg["E"]).cpu()
    nb = (cnt + block_m - 1) // block_m
    n_tiles = (cfg["I"] + pad + 127) // 128
    total = int(nb.sum()) * n_tiles
    chunk = (total + 7) // 8
    return dict(equal_runs=[min(chunk, max(0, total - x * chunk)) for x in range(8)],
                experts_round_robin=[int(nb[x::8].sum()) * n_tiles for x in range(8)],
                rows_per_expert_max=int(cnt.max()), rows_per_expert_median=int(cnt.median()))
