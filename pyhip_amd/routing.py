"""Routers on the device: gating scores -> (topk_weight f32 [T, k], topk_ids i32 [T, k]).

``fused_topk`` has the argument list of ``aiter.fused_topk`` as the reference calls it
(tests/contrib/moe/test_fused_moe.py:38,87): softmax over the experts, top-k, optional renormalisation.
``grouped_topk`` is DeepSeek-V3's routing (sigmoid scores, ``num_expert_group`` groups of consecutive experts,
the ``topk_group`` groups with the largest sum of their two best scores stay, top-k inside them).
``append_shared_experts`` turns experts that every token visits (DeepSeek-V3 has one) into extra routing slots, so
that the grouped GEMMs compute them in the same launches as the routed experts.
"""
import torch

from . import _lib

__all__ = ["fused_topk", "grouped_topk", "append_shared_experts"]


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


def append_shared_experts(topk_weights, topk_ids, num_routed_experts, num_shared_experts=1, shared_weight=1.0):
    """Routing for a layer whose weight tensors hold ``num_shared_experts`` shared experts behind the
    ``num_routed_experts`` routed ones (``w1`` [E + S, 2I, H/2], ``w2`` [E + S, H, I/2]): every token gets S more
    slots, slot ``k + s`` naming expert ``E + s`` with weight ``shared_weight``.  The layer then computes
    ``sum_k w_k * expert_k(x) + shared_weight * sum_s shared_s(x)`` in one pass: to the sort and the GEMMs a shared
    expert is an expert that happens to receive every token (T rows, T / block_size row blocks), and the top-k
    reduction adds its slot last, in fp32, before the one rounding of the output.
    -> (topk_weights f32 [T, k + S], topk_ids i32 [T, k + S]) on the inputs' device."""
    assert topk_ids.dim() == 2 and topk_weights.shape == topk_ids.shape and num_shared_experts >= 1
    T = topk_ids.shape[0]
    ids = torch.arange(num_routed_experts, num_routed_experts + num_shared_experts, dtype=torch.int32,
                       device=topk_ids.device).expand(T, num_shared_experts)
    w = torch.full((T, num_shared_experts), float(shared_weight), dtype=torch.float32, device=topk_weights.device)
    return (torch.cat([topk_weights.float(), w], dim=1).contiguous(),
            torch.cat([topk_ids.to(torch.int32), ids], dim=1).contiguous())
