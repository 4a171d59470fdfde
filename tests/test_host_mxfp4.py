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


def test_pad_layer_weights_is_exact():
    """zero-padding quantised weights changes nothing: dequantised padded weights are the originals
    surrounded by zeros, gate/up halves land where the padded layout expects them"""
    from oracle import mxfp4 as om
    rng = np.random.default_rng(5)
    E, H, I = 3, 96, 160
    w1 = (rng.standard_normal((E, 2 * I, H)) * 0.02).astype(np.float32)
    w2 = (rng.standard_normal((E, H, I)) * 0.02).astype(np.float32)
    w1q, w1s = om.quantize_mxfp4(w1)
    w2q, w2s = om.quantize_mxfp4(w2)
    b1 = torch.arange(E * 2 * I, dtype=torch.float32).reshape(E, 2 * I).to(torch.bfloat16)
    b2 = torch.arange(E * H, dtype=torch.float32).reshape(E, H).to(torch.bfloat16)
    t = torch.from_numpy
    pm = mxfp4
    p1q, p1s, p2q, p2s, pb1, pb2, hp, ip = pm.pad_layer_weights(t(w1q), t(w1s), t(w2q), t(w2s), b1, b2, multiple=128)
    Hp, Ip = 128, 256
    assert (hp, ip) == (Hp - H, Ip - I)
    d1 = om.dequantize_mxfp4(p1q.numpy(), p1s.numpy())
    d2 = om.dequantize_mxfp4(p2q.numpy(), p2s.numpy())
    o1, o2 = om.dequantize_mxfp4(w1q, w1s), om.dequantize_mxfp4(w2q, w2s)
    assert d1.shape == (E, 2 * Ip, Hp) and d2.shape == (E, Hp, Ip)
    assert (d1[:, :I, :H] == o1[:, :I]).all() and (d1[:, Ip:Ip + I, :H] == o1[:, I:]).all()
    assert d1.sum() == o1.sum() and np.abs(d1).sum() == np.abs(o1).sum()          # everything else is zero
    assert (d2[:, :H, :I] == o2).all() and np.abs(d2).sum() == np.abs(o2).sum()
    assert (pb1[:, :I] == b1[:, :I]).all() and (pb1[:, Ip:Ip + I] == b1[:, I:]).all() and pb1.float().abs().sum() == b1.float().abs().sum()
    assert (pb2[:, :H] == b2).all() and (pb2[:, H:] == 0).all()
    # already aligned: returned unchanged
    same = pm.pad_layer_weights(t(w1q), t(w1s), t(w2q), t(w2s), multiple=32)
    assert same[0].data_ptr() == t(w1q).data_ptr() and same[6:] == (0, 0)


def test_row_block_heuristic():
    """16 rows below 4 expected rows per expert, 32 below 12, 64 up to 32, 128 above"""
    from pyhip_amd.fused_moe import pick_block_m
    assert pick_block_m(16, 8, 256) == 16            # 0.5 rows per expert
    assert pick_block_m(96, 8, 256) == 16            # 3
    assert pick_block_m(128, 8, 256) == 32           # 4
    assert pick_block_m(256, 8, 256) == 32           # 8
    assert pick_block_m(384, 8, 256) == 64           # 12
    assert pick_block_m(512, 8, 256) == 64           # 16
    assert pick_block_m(1024, 8, 256) == 64          # 32
    assert pick_block_m(1056, 8, 256) == 128         # 33
    assert pick_block_m(2048, 8, 256) == 128         # 64
    assert pick_block_m(8192, 8, 256) == 128         # 256 rows per expert, short K loop: 128-row tiles
    # the bf16-activation kernels: twice the mean, at most 64 rows
    assert pick_block_m(128, 8, 256, 7168, True) == 16 and pick_block_m(256, 8, 256, 7168, True) == 16
    assert pick_block_m(512, 8, 256, 7168, True) == 32 and pick_block_m(8192, 8, 256, 7168, True) == 64
    # few experts: the smallest tile that holds twice the mean
    assert pick_block_m(1, 2, 8) == 16 and pick_block_m(32, 2, 8) == 16 and pick_block_m(64, 2, 8) == 32
    assert pick_block_m(128, 2, 8) == 64 and pick_block_m(4096, 2, 8) == 128
    # long K loop: one row block per expert where a tile of 160 / 192 / 256 / 288 rows holds it
    assert pick_block_m(3072, 8, 256, 7168) == 128 and pick_block_m(3200, 8, 256, 7168) == 160
    assert pick_block_m(4096, 8, 256, 7168) == 160 and pick_block_m(4352, 8, 256, 7168) == 192
    assert pick_block_m(5440, 8, 256, 7168) == 192 and pick_block_m(5632, 8, 256, 7168) == 256
    assert pick_block_m(6144, 8, 256, 7168) == 256 and pick_block_m(7424, 8, 256, 7168) == 256
    assert pick_block_m(7680, 8, 256, 7168) == 288 and pick_block_m(8192, 8, 256, 7168) == 288
    assert pick_block_m(8832, 8, 256, 7168) == 288 and pick_block_m(8864, 8, 256, 7168) == 128
    assert pick_block_m(8192, 8, 256, 7168, True) == 64
    # short K loop: 160 rows where one such block holds an expert that would need a second, nearly empty 128-row block
    # (100 to 132 expected rows per expert), 128 rows otherwise
    assert pick_block_m(4096, 4, 128, 3072) == 160 and pick_block_m(2048, 8, 128, 4096) == 160
    assert pick_block_m(512, 2, 8, 4096) == 160 and pick_block_m(4096, 2, 8, 4096) == 128
    assert pick_block_m(1584, 8, 128, 4096) == 128 and pick_block_m(1600, 8, 128, 4096) == 160     # 99 / 100
    assert pick_block_m(2112, 8, 128, 4096) == 160 and pick_block_m(2128, 8, 128, 4096) == 128     # 132 / 133
    assert pick_block_m(8192, 8, 128, 4096) == 128


def test_auto_method_rule():
    """bf16 activations while at most one expert in eight gets a row, or while few experts leave the down GEMM short of
    tiles"""
    from pyhip_amd.fused_moe import pick_w4a16
    assert pick_w4a16(1, 8, 256, 7168) and pick_w4a16(4, 8, 256, 7168)            # DS-V3: 8 and 32 pairs over 256 experts
    assert not pick_w4a16(8, 8, 256, 7168) and not pick_w4a16(16, 8, 256, 7168) and not pick_w4a16(8192, 8, 256, 7168)
    assert pick_w4a16(2, 8, 128, 4096) and not pick_w4a16(4, 8, 128, 4096)        # Qwen3
    assert pick_w4a16(4, 4, 128, 3072) and not pick_w4a16(16, 4, 128, 3072)       # gpt-oss, padded width
    assert pick_w4a16(1, 2, 8, 4096) and pick_w4a16(32, 2, 8, 4096)               # Mixtral: 8 experts x 16 tiles
    assert not pick_w4a16(48, 2, 8, 4096) and not pick_w4a16(4096, 2, 8, 4096)
    assert not pick_w4a16(64, 2, 8, 1024)                                         # the tiny shape at 16 rows per expert


def test_library_makes_the_same_choices():
    """the host functions are thin calls of pyhip_moe_pick_block_m / pyhip_moe_pick_w4a16 (one source of truth)"""
    from pyhip_amd import _lib
    from pyhip_amd.fused_moe import pick_block_m, pick_w4a16
    lib = _lib.load()
    for E, k, H in ((8, 2, 1024), (8, 2, 4096), (128, 4, 3072), (128, 8, 4096), (256, 8, 7168), (12, 3, 1536)):
        for T in list(range(1, 70)) + [96, 128, 200, 256, 500, 512, 1000, 1024, 2048, 3072, 3840, 4096, 5000, 6144, 6145, 8192, 32768]:
            for w4 in (0, 1):
                assert lib.pyhip_moe_pick_block_m(T, k, E, H, w4) == pick_block_m(T, k, E, H, bool(w4)), (T, k, E, H, w4)
            assert bool(lib.pyhip_moe_pick_w4a16(T, k, E, H)) == pick_w4a16(T, k, E, H), (T, k, E, H)


def test_plain_layout_cache_follows_the_source_storage():
    """The operator re-tiles plain-layout weights once and remembers the copy.  The copy must die with the source:
    a second tensor of the same shape that reuses the freed address (and starts at version 0 like the first) has to
    be re-tiled from its own bytes."""
    import gc
    import importlib
    fm = importlib.import_module("pyhip_amd.fused_moe")      # (the package re-exports the function under the module's name)
    fm._shuffle_cache.clear()
    g = torch.Generator().manual_seed(5)
    a = torch.randint(0, 256, (2, 64, 128), dtype=torch.uint8, generator=g)
    ptr = a.data_ptr()
    sa = fm._shuffled_u8(a)
    assert (sa == mxfp4.shuffle_weight(a)).all() and len(fm._shuffle_cache) == 1
    assert fm._shuffled_u8(a) is sa                                  # hit
    assert fm._shuffled_u8(a.view(torch.int8)) is sa                 # another view of the same storage: hit
    a[0, 0, 0] ^= 0xFF                                               # in-place change: version moves, copy is redone
    sa2 = fm._shuffled_u8(a)
    assert sa2 is not sa and (sa2 == mxfp4.shuffle_weight(a)).all()
    del a, sa, sa2
    gc.collect()
    assert len(fm._shuffle_cache) == 0                               # freed with its source
    same_address = False
    for _ in range(8):                                               # the allocator normally hands the block out again
        b = torch.randint(0, 256, (2, 64, 128), dtype=torch.uint8, generator=g)
        same_address = same_address or b.data_ptr() == ptr
        assert (fm._shuffled_u8(b) == mxfp4.shuffle_weight(b)).all()
        del b
        gc.collect()
        assert len(fm._shuffle_cache) == 0
    # (whether or not the address came back, every result above was made from the tensor's own bytes)
    # the number of storages remembered at once is bounded
    keep = [torch.randint(0, 256, (1, 16, 64), dtype=torch.uint8, generator=g) for _ in range(fm._SHUFFLE_CACHE_STORAGES + 3)]
    for t in keep:
        fm._shuffled_u8(t)
    assert len(fm._shuffle_cache) == fm._SHUFFLE_CACHE_STORAGES
    fm._shuffle_cache.clear()
