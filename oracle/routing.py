"""Routers that produce (topk_weight, topk_ids) for the harness.  Test infrastructure only.

The reference has no router on this path: its tests draw ids with ``torch.topk(randn)``
(tests/contrib/moe/test_moe_sorting.py:81-84), tile a ``randperm``
(tests/contrib/moe/test_moe.py:264-272) or call ``aiter.fused_topk``
(tests/contrib/moe/test_fused_moe.py:38,87).  These follow the benchmark definitions instead
(softmax -> top-k -> renormalise; DeepSeek-V3: sigmoid scores, 8 groups, top-4 groups by the
sum of each group's two best scores, top-8 experts inside them, renormalise).

Pins: invariants (k distinct experts per token, weights sum to 1, at most ``topk_group``
groups per token) and brute force on tiny inputs (tests/test_oracle_moe.py).
"""
import numpy as np


def softmax_topk(logits, k, renormalize=True):
    x = np.asarray(logits, dtype=np.float64)
    p = np.exp(x - x.max(axis=-1, keepdims=True))
    p /= p.sum(axis=-1, keepdims=True)
    ids = np.argsort(-p, axis=-1, kind="stable")[:, :k]
    w = np.take_along_axis(p, ids, axis=-1)
    if renormalize:
        w = w / w.sum(axis=-1, keepdims=True)
    return w.astype(np.float32), ids.astype(np.int32)


def grouped_sigmoid_topk(logits, k, n_group, topk_group, renormalize=True):
    x = np.asarray(logits, dtype=np.float64)
    T, E = x.shape
    s = 1.0 / (1.0 + np.exp(-x))
    g = s.reshape(T, n_group, E // n_group)
    gs = np.sort(g, axis=-1)[..., -2:].sum(-1)                       # [T, n_group]
    gsel = np.argsort(-gs, axis=-1, kind="stable")[:, :topk_group]
    gmask = np.zeros((T, n_group), dtype=bool)
    np.put_along_axis(gmask, gsel, True, axis=-1)
    masked = np.where(np.repeat(gmask, E // n_group, axis=1), s, -np.inf)
    ids = np.argsort(-masked, axis=-1, kind="stable")[:, :k]
    w = np.take_along_axis(s, ids, axis=-1)
    if renormalize:
        w = w / w.sum(axis=-1, keepdims=True)
    return w.astype(np.float32), ids.astype(np.int32)
