"""MoE routing sort: group (token, slot) pairs by expert, pad every expert to the block size.

Test infrastructure only (see ``oracle/__init__.py``).  Integer exact.

Restates
  * src/contrib/fused_moe.py:56-100 (``moe_sorting_ref``; same as
    tests/contrib/moe/test_moe_sorting.py:10-50): experts ascending, then tokens ascending,
    then slots ascending; id = (slot << 24) | token; padding id = (topk << 24) | num_tokens with
    weight 0; first id of a block fixes ``sorted_expert_ids``; experts without tokens get no
    block; ``num_valid_ids[0]`` = padded total.
    That function pads to multiples of 256 whatever ``block_size`` is (:91-96); the in-tree CK
    host reference pads to ``unit_size`` (= block size), which is what the GPU sorter it models
    does, so this restatement pads to ``block_size``.
  * archive/ck_tile/ck_tile/host/reference/reference_moe_sorting.hpp:13-117 for
    ``expert_mask`` (masked experts are dropped and expert ids become local indices) and the
    sentinel ``MOCK_ID(num_token, topk)`` (:11-12,34-37).
  * buffer sizes: src/contrib/fused_moe.py:73-79.
  * ``num_valid_ids[1]`` = number of (local) tokens: src/contrib/moe.py:1445.

Pins: ``moe_sorting_brute`` (the triple loop, literally) on small inputs; the compiled CK
host reference (oracle/_ref) on random inputs incl. masks; the worked example of
archive/ck_tile/ck_tile/ops/fused_moe/kernel/moe_sorting_kernel.hpp:30-97 re-derived through
that compiled reference; invariants of tests/contrib/moe/test_moe_sorting.py:109-125.
Content of entries at and beyond ``num_valid_ids[0]`` in aiter's own sorter: **parity unpinned**
(aiter absent); here they hold the padding id, weight 0 and expert id 0xFFFFFFFF.
"""
import numpy as np

#: value of ``sorted_expert_ids`` entries past the last valid block
EXPERT_ID_FILL = 0xFFFFFFFF


def max_blocks(num_pairs, num_experts, block_size):
    """src/contrib/fused_moe.py:73"""
    return (num_pairs + num_experts * (block_size - 1) + block_size - 1) // block_size


def moe_sorting_ref(topk_ids, topk_weights, num_experts, block_size,
                    expert_mask=None, num_local_tokens=None):
    """-> sorted_ids u32[n_blk*Bm], sorted_weights f32[n_blk*Bm], sorted_expert_ids u32[n_blk],
    num_valid_ids u32[2]."""
    topk_ids = np.asarray(topk_ids)
    T_all, k = topk_ids.shape
    T = T_all if num_local_tokens is None else int(num_local_tokens)
    n_blk = max_blocks(T_all * k, num_experts, block_size)
    pad_id = np.uint32((k << 24) | (T & 0xFFFFFF))
    sorted_ids = np.full(n_blk * block_size, pad_id, dtype=np.uint32)
    sorted_w = np.zeros(n_blk * block_size, dtype=np.float32)
    sorted_e = np.full(n_blk, EXPERT_ID_FILL, dtype=np.uint32)

    ids = topk_ids[:T].reshape(-1).astype(np.int64)
    w = np.asarray(topk_weights, dtype=np.float32)[:T].reshape(-1)
    order = np.argsort(ids, kind="stable")           # keeps (token, slot) order inside an expert
    counts = np.bincount(ids, minlength=num_experts)[:num_experts]
    if expert_mask is not None:
        mask = np.asarray(expert_mask).astype(bool)
        local_id = np.cumsum(mask) - 1
    else:
        mask = np.ones(num_experts, dtype=bool)
        local_id = np.arange(num_experts)
    start_in_sorted = np.concatenate([[0], np.cumsum(counts)])
    pos = 0
    for e in range(num_experts):
        c = int(counts[e])
        if not mask[e] or c == 0:
            continue
        sel = order[start_in_sorted[e]:start_in_sorted[e] + c]
        tok, slot = sel // k, sel % k
        sorted_ids[pos:pos + c] = (slot.astype(np.uint32) << 24) | tok.astype(np.uint32)
        sorted_w[pos:pos + c] = w[sel]
        nb = (c + block_size - 1) // block_size
        sorted_e[pos // block_size: pos // block_size + nb] = local_id[e]
        pos += nb * block_size
    num_valid = np.array([pos, T], dtype=np.uint32)
    return sorted_ids, sorted_w, sorted_e, num_valid


def moe_sorting_brute(topk_ids, topk_weights, num_experts, block_size):
    """The triple loop of src/contrib/fused_moe.py:81-98 with the pad unit set to ``block_size``.
    Pure Python; small inputs only.  -> (ids, weights, expert id per block, padded total)."""
    T, k = len(topk_ids), len(topk_ids[0])
    ids, ws, es = [], [], []
    for e in range(num_experts):
        for i in range(T):
            for t in range(k):
                if topk_ids[i][t] == e:
                    if len(ids) % block_size == 0:
                        es.append(e)
                    ids.append((t << 24) | i)
                    ws.append(float(topk_weights[i][t]))
        while len(ids) % block_size:
            ids.append((k << 24) | T)
            ws.append(0.0)
    return ids, ws, es, len(ids)
