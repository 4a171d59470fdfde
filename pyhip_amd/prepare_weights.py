"""Offline weight preparation: bf16 / float expert weights -> the tensors ``fused_moe`` consumes, and a file
format for them.

What it replaces on the reference side is the weight-prep block of its MoE tests
(tests/contrib/moe/test_moe.py:161-189): ``aiter.get_torch_quant(per_1x32)`` -> ``pre_shuffle(x, 16)``
(src/misc.py:116-130) -> ``e8m0_shuffle`` (tests/contrib/moe/test_fused_moe.py:222-236), plus the zero padding
aiter applies to shapes that are not multiples of the kernels' tiles (hidden_pad / intermediate_pad,
tests/contrib/moe/test_fused_moe.py:92-105).

File: one ``.safetensors`` with

    w1        uint8 [E, 2*Ip, Hp/2]   e2m1 pairs, gate rows [0, I) and up rows [Ip, Ip+I), pre-shuffled
    w1_scale  uint8 [pad256(E*2*Ip), pad8(Hp/32)]   e8m0, shuffled
    w2        uint8 [E, Hp, Ip/2]     pre-shuffled
    w2_scale  uint8 [pad256(E*Hp), pad8(Ip/32)]
    bias1     bf16  [E, 2*Ip]         (optional)
    bias2     bf16  [E, Hp]           (optional)

and the metadata ``format = pyhip_amd.mxfp4.v1``, ``experts``, ``hidden``, ``inter`` (true sizes), ``hidden_pad``,
``intermediate_pad`` (Hp = hidden + hidden_pad, Ip = inter + intermediate_pad; both multiples of 512).

Command line (expert by expert, so the float weights of one expert are all that is ever held):

    python -m pyhip_amd.prepare_weights IN.safetensors OUT.safetensors \\
        [--w1 NAME --w2 NAME --bias1 NAME --bias2 NAME]

where IN holds ``w1 [E, 2*I, H]`` (gate rows then up rows) and ``w2 [E, H, I]`` in bf16 / fp16 / fp32.
"""
import argparse
import json

import torch

from . import mxfp4

FORMAT = "pyhip_amd.mxfp4.v1"


def convert(w1, w2, bias1=None, bias2=None, multiple=512):
    """float [E, 2I, H], float [E, H, I] (+ biases [E, 2I], [E, H]) -> (dict of tensors, dict of metadata)."""
    E, N1, H = w1.shape
    I = N1 // 2
    assert w2.shape == (E, H, I), (w1.shape, w2.shape)
    assert H % mxfp4.BLOCK == 0 and I % mxfp4.BLOCK == 0, "hidden and inter must be multiples of 32"
    q1, s1, q2, s2 = [], [], [], []
    for e in range(E):                                     # one expert at a time in float
        a, b = mxfp4.quantize_mxfp4(w1[e].float())
        c, d = mxfp4.quantize_mxfp4(w2[e].float())
        q1.append(a), s1.append(b), q2.append(c), s2.append(d)
    q1, s1, q2, s2 = torch.stack(q1), torch.stack(s1), torch.stack(q2), torch.stack(s2)
    b1 = None if bias1 is None else bias1.to(torch.bfloat16)
    b2 = None if bias2 is None else bias2.to(torch.bfloat16)
    q1, s1, q2, s2, b1, b2, hp, ip = mxfp4.pad_layer_weights(q1, s1, q2, s2, b1, b2, multiple)
    Hp, Ip = H + hp, I + ip
    tensors = {
        "w1": mxfp4.shuffle_weight(q1).contiguous(),
        "w1_scale": mxfp4.e8m0_shuffle(s1.reshape(E * 2 * Ip, Hp // mxfp4.BLOCK)).contiguous(),
        "w2": mxfp4.shuffle_weight(q2).contiguous(),
        "w2_scale": mxfp4.e8m0_shuffle(s2.reshape(E * Hp, Ip // mxfp4.BLOCK)).contiguous(),
    }
    if b1 is not None:
        tensors["bias1"] = b1.contiguous()
    if b2 is not None:
        tensors["bias2"] = b2.contiguous()
    meta = {"format": FORMAT, "experts": E, "hidden": H, "inter": I, "hidden_pad": hp, "intermediate_pad": ip}
    return tensors, meta


def save(path, tensors, meta):
    from safetensors.torch import save_file
    save_file({k: v.cpu() for k, v in tensors.items()}, path, metadata={k: str(v) for k, v in meta.items()})


def load(path, device="cpu"):
    """-> (tensors, meta); ``fused_moe_kwargs(tensors, meta)`` turns them into the operator's arguments."""
    from safetensors import safe_open
    with safe_open(path, framework="pt", device=str(device)) as f:
        meta = dict(f.metadata() or {})
        if meta.get("format") != FORMAT:
            raise ValueError("%s: not a %s file (format = %r)" % (path, FORMAT, meta.get("format")))
        tensors = {k: f.get_tensor(k) for k in f.keys()}
    meta = {k: (v if k == "format" else int(v)) for k, v in meta.items()}
    E, Hp, Ip = meta["experts"], meta["hidden"] + meta["hidden_pad"], meta["inter"] + meta["intermediate_pad"]
    if tuple(tensors["w1"].shape) != (E, 2 * Ip, Hp // 2) or tuple(tensors["w2"].shape) != (E, Hp, Ip // 2):
        raise ValueError("%s: tensor shapes do not match the metadata" % path)
    tensors["w1"].is_shuffled = True                       # what the reference looks for (src/contrib/fused_moe.py:198-206)
    tensors["w2"].is_shuffled = True
    return tensors, meta


def fused_moe_kwargs(tensors, meta):
    """positional (w1, w2) and the keyword arguments of ``pyhip_amd.fused_moe`` that come from the file"""
    kw = dict(w1_scale=tensors["w1_scale"], w2_scale=tensors["w2_scale"], bias1=tensors.get("bias1"),
              bias2=tensors.get("bias2"), hidden_pad=meta["hidden_pad"], intermediate_pad=meta["intermediate_pad"])
    return (tensors["w1"], tensors["w2"]), kw


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("src")
    ap.add_argument("dst")
    ap.add_argument("--w1", default="w1")
    ap.add_argument("--w2", default="w2")
    ap.add_argument("--bias1", default=None)
    ap.add_argument("--bias2", default=None)
    a = ap.parse_args(argv)
    from safetensors import safe_open
    with safe_open(a.src, framework="pt", device="cpu") as f:
        get = lambda name: None if name is None else f.get_tensor(name)
        tensors, meta = convert(get(a.w1), get(a.w2), get(a.bias1), get(a.bias2))
    save(a.dst, tensors, meta)
    print(json.dumps(dict(meta, file=a.dst, bytes=sum(t.numel() * t.element_size() for t in tensors.values()))))


if __name__ == "__main__":
    main()
