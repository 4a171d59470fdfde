"""Weight-prep tool and its file format (CPU): what is written is what the direct helpers produce, the file loads
back bit for bit, and the stored weights dequantise to the originals within the MXFP4 rounding bound."""
import numpy as np
import pytest
import torch

from oracle import layout, mxfp4 as om
from pyhip_amd import mxfp4 as pm, prepare_weights as pw


def _layer(E, H, I, seed=0, bias=False):
    g = torch.Generator().manual_seed(seed)
    w1 = (torch.randn(E, 2 * I, H, generator=g) * 0.05).to(torch.bfloat16)
    w2 = (torch.randn(E, H, I, generator=g) * 0.05).to(torch.bfloat16)
    b1 = (torch.randn(E, 2 * I, generator=g) * 0.01).to(torch.bfloat16) if bias else None
    b2 = (torch.randn(E, H, generator=g) * 0.01).to(torch.bfloat16) if bias else None
    return w1, w2, b1, b2


def test_round_trip_through_the_file(tmp_path):
    from safetensors.torch import save_file
    E, H, I = 3, 512, 512
    w1, w2, _, _ = _layer(E, H, I)
    src, dst = tmp_path / "in.safetensors", tmp_path / "out.safetensors"
    save_file({"w1": w1, "w2": w2}, str(src))
    pw.main([str(src), str(dst)])
    tensors, meta = pw.load(str(dst))
    assert meta == {"format": pw.FORMAT, "experts": E, "hidden": H, "inter": I, "hidden_pad": 0, "intermediate_pad": 0}
    q1, s1 = pm.prepare_expert_weights(w1.float())
    q2, s2 = pm.prepare_expert_weights(w2.float())
    assert torch.equal(tensors["w1"], q1) and torch.equal(tensors["w1_scale"], s1)
    assert torch.equal(tensors["w2"], q2) and torch.equal(tensors["w2_scale"], s2)
    assert getattr(tensors["w1"], "is_shuffled", False)
    (a, b), kw = pw.fused_moe_kwargs(tensors, meta)
    assert a is tensors["w1"] and kw["hidden_pad"] == 0 and kw["bias1"] is None
    # the stored bytes, taken apart with the oracle's own layout code, give back the weights: within half of the
    # largest e2m1 spacing (2 units) where the value fits, within 2 units where the block maximum saturates at 6
    plain = layout.deshuffle_weight(tensors["w1"].numpy())
    scales = layout.e8m0_deshuffle(tensors["w1_scale"].numpy(), E * 2 * I, H // 32).reshape(E, 2 * I, H // 32)
    deq = om.dequantize_mxfp4(plain, scales)
    step = np.repeat(np.exp2(scales.astype(np.float64) - 127), 32, axis=-1)          # one e2m1 unit of the block
    err = np.abs(deq - w1.float().numpy())
    fits = np.abs(w1.float().numpy()) <= 6 * step
    assert (err <= step * 2.0 + 1e-12).all() and (err[fits] <= step[fits] + 1e-12).all()


def test_padded_shape_and_biases(tmp_path):
    E, H, I = 2, 1440, 1440                                 # gpt-oss / 2: padded to 1536
    w1, w2, b1, b2 = _layer(E, H, I, seed=1, bias=True)
    tensors, meta = pw.convert(w1, w2, b1, b2)
    assert (meta["hidden_pad"], meta["intermediate_pad"]) == (96, 96)
    Hp = Ip = 1536
    assert tuple(tensors["w1"].shape) == (E, 2 * Ip, Hp // 2) and tuple(tensors["w2"].shape) == (E, Hp, Ip // 2)
    assert tuple(tensors["bias1"].shape) == (E, 2 * Ip) and tuple(tensors["bias2"].shape) == (E, Hp)
    plain = layout.deshuffle_weight(tensors["w1"].numpy())
    assert (plain[:, I:Ip] == 0).all() and (plain[:, Ip + I:] == 0).all() and (plain[:, :, H // 2:] == 0).all()
    q, _ = pm.quantize_mxfp4(w1.float())
    assert (plain[:, :I, :H // 2] == q[:, :I].numpy()).all() and (plain[:, Ip:Ip + I, :H // 2] == q[:, I:].numpy()).all()
    assert torch.equal(tensors["bias1"][:, Ip:Ip + I], b1[:, I:]) and (tensors["bias1"][:, I:Ip] == 0).all()
    path = tmp_path / "padded.safetensors"
    pw.save(str(path), tensors, meta)
    back, meta2 = pw.load(str(path))
    assert meta2 == meta and all(torch.equal(back[k], tensors[k]) for k in tensors)


def test_foreign_file_is_rejected(tmp_path):
    from safetensors.torch import save_file
    path = tmp_path / "x.safetensors"
    save_file({"w1": torch.zeros(1, dtype=torch.uint8)}, str(path))
    with pytest.raises(ValueError, match="not a pyhip_amd.mxfp4.v1 file"):
        pw.load(str(path))
