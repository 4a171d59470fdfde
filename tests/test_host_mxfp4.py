"""The product's torch weight preparation against the oracle's numpy restatement (CPU)."""
import numpy as np
import torch

from oracle import layout as ol, mxfp4 as om
from pyhip_amd import mxfp4


def test_quantize_matches_oracle_bitwise():
    g = torch.Generator().manual_seed(0)
    x = torch.randn(3, 48, 256, generator=g) * torch.exp(torch.randn(3, 48, 1, generator=g) * 2)
    x[0, 0, :32] = 0
    x[0, 1, :8] = torch.tensor([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0, 4.0])      # ties at scale 1
    q, s = mxfp4.quantize_mxfp4(x)
    oq, os_ = om.quantize_mxfp4(x.numpy())
    assert (q.numpy() == oq).all() and (s.numpy() == os_).all()
    d = mxfp4.dequantize_mxfp4(q, s)
    assert (d.numpy() == om.dequantize_mxfp4(oq, os_)).all()
    qb, sb = mxfp4.quantize_mxfp4(x.to(torch.bfloat16))
    oqb, osb = om.quantize_mxfp4(x.to(torch.bfloat16).float().numpy())
    assert (qb.numpy() == oqb).all() and (sb.numpy() == osb).all()


def test_shuffles_match_oracle():
    rng = np.random.default_rng(0)
    w = rng.integers(0, 256, (2, 64, 128), dtype=np.uint8)
    tw = torch.from_numpy(w)
    assert (mxfp4.shuffle_weight(tw).numpy() == ol.shuffle_weight(w)).all()
    assert (mxfp4.deshuffle_weight(mxfp4.shuffle_weight(tw)) == tw).all()
    s = rng.integers(0, 255, (300, 13), dtype=np.uint8)
    ts = torch.from_numpy(s)
    assert (mxfp4.e8m0_shuffle(ts).numpy() == ol.e8m0_shuffle(s)).all()
    assert (mxfp4.e8m0_deshuffle(mxfp4.e8m0_shuffle(ts), 300, 13) == ts).all()


def test_prepare_expert_weights():
    g = torch.Generator().manual_seed(1)
    w = torch.randn(4, 64, 128, generator=g) * 0.02
    q, s = mxfp4.prepare_expert_weights(w)
    assert q.shape == (4, 64, 64) and q.is_shuffled and s.shape == (256, 8)
    oq, os_ = om.quantize_mxfp4(w.numpy())
    assert (q.numpy() == ol.shuffle_weight(oq)).all()
    assert (s.numpy() == ol.e8m0_shuffle(os_.reshape(256, 4))).all()
