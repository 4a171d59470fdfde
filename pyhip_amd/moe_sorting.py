"""``moe_sorting``: the routing contract of the fused-MoE layer.

Drop-in for ``aiter.fused_moe.moe_sorting`` as the reference calls it
(src/contrib/fused_moe.py:283,301-305; CPU statement of the result: src/contrib/fused_moe.py:56-100).
"""
import torch

from . import _lib


def max_blocks(num_pairs, num_experts, block_size):
    return (num_pairs + num_experts * (block_size - 1) + block_size - 1) // block_size


def moe_sorting(topk_ids, topk_weights, num_experts, model_dim, moebuf_dtype, block_size=32,
                expert_mask=None, num_local_tokens=None, dispatch_policy=0, *, alloc_moe_out=True,
                return_schedule=False, quant_input=None):
    """-> (sorted_ids u32 [n_blk*Bm] viewed as int32, sorted_weights f32, sorted_expert_ids int32 [n_blk],
    num_valid_ids int32 [2], moe_out [T, model_dim] zero-filled)

    ``sorted_ids = (slot << 24) | token``; padding entries hold ``(topk << 24) | T`` with weight 0;
    ``num_valid_ids = [padded total, number of (local) tokens]``; entries of ``sorted_expert_ids`` past
    the last valid block hold -1.  ``num_local_tokens`` is a device int32 scalar tensor (or None).

    ``quant_input`` (bf16 [rows, K], unit column stride; needs ``alloc_moe_out=False``): its MXFP4 quantisation
    rides in the sort's launches and ``(q, scales)`` is appended to the result, as ``act_quant_mxfp4`` returns them.
    """
    lib = _lib.load()
    assert topk_ids.is_cuda and topk_ids.dtype == torch.int32 and topk_ids.is_contiguous()
    assert topk_weights.dtype == torch.float32 and topk_weights.is_contiguous()
    assert topk_weights.shape == topk_ids.shape
    T, k = topk_ids.shape
    dev = topk_ids.device
    n_blk = max_blocks(T * k, num_experts, block_size)
    sorted_ids = torch.empty(n_blk * block_size, dtype=torch.int32, device=dev)
    sorted_w = torch.empty(n_blk * block_size, dtype=torch.float32, device=dev)
    sorted_e = torch.empty(n_blk, dtype=torch.int32, device=dev)
    num_valid = torch.empty(2, dtype=torch.int32, device=dev)
    moe_out = torch.empty(T, model_dim, dtype=moebuf_dtype, device=dev) if alloc_moe_out else None
    sched = torch.empty(lib.pyhip_moe_schedule_words(num_experts), dtype=torch.int32, device=dev) \
        if return_schedule else None
    ws_bytes = lib.pyhip_moe_sorting_workspace_bytes(T, k, num_experts)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    if expert_mask is not None:
        expert_mask = expert_mask.to(device=dev, dtype=torch.int32).contiguous()
        assert expert_mask.numel() == num_experts
    if num_local_tokens is not None:
        assert num_local_tokens.is_cuda and num_local_tokens.dtype == torch.int32
    extra = ()
    if quant_input is not None:
        x = quant_input
        assert moe_out is None and x.is_cuda and x.dtype == torch.bfloat16 and x.dim() == 2 and x.stride(1) == 1
        rows, K = x.shape
        q = torch.empty(rows, K // 2, dtype=torch.uint8, device=dev)
        s = torch.empty(rows, lib.pyhip_moe_act_scale_stride(K), dtype=torch.uint8, device=dev)
        rc = lib.pyhip_moe_sorting_quant(
            _lib.dptr(topk_ids), _lib.dptr(topk_weights), T, k, num_experts, block_size,
            _lib.dptr(expert_mask), _lib.dptr(num_local_tokens),
            _lib.dptr(sorted_ids), _lib.dptr(sorted_w), _lib.dptr(sorted_e), _lib.dptr(num_valid), _lib.dptr(sched),
            _lib.dptr(ws), ws_bytes, _lib.dptr(x), x.stride(0), rows, K, _lib.dptr(q), _lib.dptr(s),
            _lib.current_stream())
        _lib.check(rc, "moe_sorting_quant")
        extra = ((q, s),)
    else:
        rc = lib.pyhip_moe_sorting(
            _lib.dptr(topk_ids), _lib.dptr(topk_weights), T, k, num_experts, block_size,
            _lib.dptr(expert_mask), _lib.dptr(num_local_tokens),
            _lib.dptr(sorted_ids), _lib.dptr(sorted_w), _lib.dptr(sorted_e), _lib.dptr(num_valid), _lib.dptr(sched),
            _lib.dptr(moe_out), 0 if moe_out is None else moe_out.numel() * moe_out.element_size(),
            _lib.dptr(ws), ws_bytes, _lib.current_stream())
        _lib.check(rc, "moe_sorting")
    if return_schedule:
        return (sorted_ids, sorted_w, sorted_e, num_valid, moe_out, sched) + extra
    return (sorted_ids, sorted_w, sorted_e, num_valid, moe_out) + extra
