"""Routers on the device: gating scores -> (topk_weight f32 [T, k], topk_ids i32 [T, k]).

``fused_topk`` has the argument list of ``aiter.fused_topk`` as the reference calls it
(tests/contrib/moe/test_fused_moe.py:38,87): softmax over the experts, top-k, optional renormalisation.
``grouped_topk`` is DeepSeek-V3's routing (sigmoid scores, ``num_expert_group`` groups of consecutive experts,
the ``topk_group`` groups with the largest sum of their two best scores stay, top-k inside them).
"""
import torch

from . import _lib

__all__ = ["fused_topk", "grouped_topk"]


def _scores(gating_output, pad_ok):
    assert gating_output.is_cuda and gating_output.dim() == 2
    g = gating_output.float().contiguous()
    E = g.shape[1]
    Ep = 64
    while Ep < E:                # the kernel handles 64 * 2^n experts: -inf columns are never picked
        Ep *= 2
    if Ep != E and pad_ok:
        g = torch.nn.functional.pad(g, (0, Ep - E), value=float("-inf"))
    return g


def fused_topk(hidden_states, gating_output, topk, renormalize=True):
    """-> (topk_weights f32 [T, topk], topk_ids i32 [T, topk]); ``hidden_states`` only supplies the token count."""
    lib = _lib.load()
    T, E = gating_output.shape
    assert hidden_states is None or hidden_states.shape[0] == T
    assert topk <= E
    g = _scores(gating_output, True)
    w = torch.empty(T, topk, dtype=torch.float32, device=g.device)
    ids = torch.empty(T, topk, dtype=torch.int32, device=g.device)
    _lib.check(lib.pyhip_moe_topk_softmax(_lib.dptr(g), T, g.shape[1], topk, 1 if renormalize else 0, _lib.dptr(w),
                                          _lib.dptr(ids), _lib.current_stream()), "topk_softmax")
    return w, ids


def grouped_topk(gating_output, topk, renormalize=True, num_expert_group=8, topk_group=4):
    """-> (topk_weights f32 [T, topk], topk_ids i32 [T, topk]) with sigmoid scoring and grouped selection."""
    lib = _lib.load()
    T, E = gating_output.shape
    g = _scores(gating_output, False)
    w = torch.empty(T, topk, dtype=torch.float32, device=g.device)
    ids = torch.empty(T, topk, dtype=torch.int32, device=g.device)
    _lib.check(lib.pyhip_moe_topk_grouped_sigmoid(_lib.dptr(g), T, E, topk, num_expert_group, topk_group,
                                                  1 if renormalize else 0, _lib.dptr(w), _lib.dptr(ids),
                                                  _lib.current_stream()), "topk_grouped_sigmoid")
    return w, ids
