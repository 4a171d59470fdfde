"""Seeded synthetic MoE layers for the tests.  Inputs are drawn with a CPU generator so that the
build container and the GPU box see identical data; weights are quantised with the ORACLE's numpy
quantiser (the product's torch quantiser is checked against it separately)."""
import numpy as np
import torch

from oracle import layout, mxfp4, routing

CONFIGS = {
    # name: E, topk, H, I, router
    "tiny": dict(E=8, k=2, H=1024, I=512, router="softmax"),
    "mixtral_s": dict(E=8, k=2, H=1024, I=1024, router="softmax"),          # Mixtral-shaped, scaled down
    "qwen3_s": dict(E=32, k=8, H=1024, I=512, router="zipf"),
    "dsv3_s": dict(E=64, k=8, H=1024, I=512, router="grouped"),
    # gpt-oss-shaped, scaled down: hidden = inter = 2880/2, not multiples of the kernels' 512-wide K tiles
    "gptoss_s": dict(E=16, k=4, H=1440, I=1440, router="softmax"),
    "gptoss_s1": dict(E=16, k=4, H=1536, I=1536, router="softmax"),         # 12 K-steps: an odd share per wave under split K
    # an expert count that is not a multiple of the 8 XCDs the tile schedule deals experts to, an odd top-k,
    # three K-groups in the gate_up GEMM
    "odd": dict(E=12, k=3, H=1536, I=1024, router="softmax"),
    # long K in both GEMMs (16 and 20 K-steps of 128): the sixteen-wave split of the bf16-activation kernels, with one
    # K-step per wave in gate_up and an uneven share (one or two) in down
    "longk_s": dict(E=4, k=2, H=2048, I=2560, router="softmax"),
    # a down GEMM with 68 K-steps: the sixteen-wave split on 32-row tiles gives a wave four or five of them, more than the
    # three it keeps in flight, and with two experts and four 256-row tiles it is what the launcher picks by itself
    "verylongk_s": dict(E=2, k=2, H=1024, I=8704, router="softmax"),
}


class Layer:
    pass


def make_layer(name, T, seed=0, bias=False, E=None, k=None, H=None, I=None, router=None):
    cfg = dict(CONFIGS[name]) if name in CONFIGS else {}
    for key, v in dict(E=E, k=k, H=H, I=I, router=router).items():
        if v is not None:
            cfg[key] = v
    E, k, H, I = cfg["E"], cfg["k"], cfg["H"], cfg["I"]
    g = torch.Generator().manual_seed(seed)
    L = Layer()
    L.E, L.k, L.H, L.I, L.T = E, k, H, I, T
    L.hidden = torch.randn(T, H, generator=g).to(torch.bfloat16)
    w1 = (torch.randn(E, 2 * I, H, generator=g) * 0.02).numpy()
    w2 = (torch.randn(E, H, I, generator=g) * 0.02).numpy()
    L.w1q, L.w1s = mxfp4.quantize_mxfp4(w1)
    L.w2q, L.w2s = mxfp4.quantize_mxfp4(w2)
    logits = torch.randn(T, E, generator=g).numpy().astype(np.float64)
    if cfg["router"] == "softmax":
        L.topk_w, L.topk_ids = routing.softmax_topk(logits, k)
    elif cfg["router"] == "zipf":
        zb = np.log(1.0 / np.arange(1, E + 1) ** 1.1)
        L.topk_w, L.topk_ids = routing.softmax_topk(logits + zb[None, :] - zb.mean(), k)
    else:
        L.topk_w, L.topk_ids = routing.grouped_sigmoid_topk(logits, k, n_group=8, topk_group=4)
    L.bias1 = L.bias2 = None
    if bias:
        L.bias1 = (torch.randn(E, 2 * I, generator=g) * 0.01).to(torch.bfloat16)
        L.bias2 = (torch.randn(E, H, generator=g) * 0.01).to(torch.bfloat16)
    return L


def device_weights(L, dev="cuda"):
    """shuffled device tensors in the layout fused_moe takes"""
    w1 = torch.from_numpy(layout.shuffle_weight(L.w1q)).to(dev)
    w2 = torch.from_numpy(layout.shuffle_weight(L.w2q)).to(dev)
    w1s = torch.from_numpy(layout.e8m0_shuffle(L.w1s.reshape(L.E * 2 * L.I, L.H // 32))).to(dev)
    w2s = torch.from_numpy(layout.e8m0_shuffle(L.w2s.reshape(L.E * L.H, L.I // 32))).to(dev)
    w1.is_shuffled = w2.is_shuffled = True        # the mark the operator looks for (src/contrib/fused_moe.py:198-206)
    return w1, w1s, w2, w2s


def plain_device_weights(L, dev="cuda"):
    """the same weights in the plain [E, N, K/2] layout (no ``is_shuffled`` mark); scales shuffled as always"""
    w1, w1s, w2, w2s = device_weights(L, dev)
    return torch.from_numpy(L.w1q).to(dev), w1s, torch.from_numpy(L.w2q).to(dev), w2s


def padded_device_weights(L, dev="cuda"):
    """as device_weights, for shapes that need zero-padding to the kernels' tile multiples:
    -> (w1, w1s, w2, w2s, bias1, bias2, hidden_pad, intermediate_pad)"""
    from pyhip_amd import mxfp4 as pm
    t = lambda a: torch.from_numpy(a)
    w1q, w1s, w2q, w2s, b1, b2, hp, ip = pm.pad_layer_weights(t(L.w1q), t(L.w1s), t(L.w2q), t(L.w2s), L.bias1, L.bias2)
    E, Hp, Ip = L.E, L.H + hp, L.I + ip
    w1 = torch.from_numpy(layout.shuffle_weight(w1q.numpy())).to(dev)
    w2 = torch.from_numpy(layout.shuffle_weight(w2q.numpy())).to(dev)
    s1 = torch.from_numpy(layout.e8m0_shuffle(w1s.numpy().reshape(E * 2 * Ip, Hp // 32))).to(dev)
    s2 = torch.from_numpy(layout.e8m0_shuffle(w2s.numpy().reshape(E * Hp, Ip // 32))).to(dev)
    w1.is_shuffled = w2.is_shuffled = True
    return w1, s1, w2, s2, None if b1 is None else b1.to(dev), None if b2 is None else b2.to(dev), hp, ip


def untranspose_act_scales(s, K):
    """kernel activation-scale layout [rows, SK] -> plain [rows, K/32] (numpy)"""
    rows, SK = s.shape
    g = s.reshape(rows, SK // 16, 4, 4)            # [q][kb][i]  ->  block 16q + 4i + kb
    plain = g.transpose(0, 1, 3, 2).reshape(rows, SK)
    return plain[:, : K // 32]
