/* C ABI of libpyhip_moe.so: MXFP4 fused-MoE for MI355X (gfx950).
 *
 * Plain pointers and sizes only; every pointer named "device" is HIP device memory of the
 * current device; `stream` is a hipStream_t (NULL = default stream).  All calls only enqueue
 * work; none synchronises.  Return value: 0 = ok, 1 = invalid argument, 2 = HIP error; the
 * message of the last failure on the calling thread is returned by pyhip_moe_last_error().
 *
 * Each entry point names the reference interface (tingqli/pyhip, file:line) whose job it does.
 */
#ifndef PYHIP_MOE_H
#define PYHIP_MOE_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void* pyhip_stream_t; /* hipStream_t */

/* ABI revision of this header. */
int pyhip_moe_abi_version(void);

/* Message of the last failed call on this thread (replaces the Python exception text of
 * hip_check_error, src/core/hiptools.py:37-39). */
const char* pyhip_moe_last_error(void);

/* ------------------------------------------------------------------------------------------
 * Routers: gating scores f32 [tokens, experts] -> topk_weight f32 [tokens, topk], topk_ids i32 [tokens, topk],
 * the inputs of the routing sort.  Picks are in descending score order; ties go to the lower expert index.
 * experts must be 64 * 2^n, at most 2048 (pad the scores with -inf columns otherwise); topk <= 64.
 *   pyhip_moe_topk_softmax          softmax over the experts, top-k, weights renormalised to sum 1 when
 *                                   renormalize != 0: replaces aiter.fused_topk(hidden, score, topk, True) as
 *                                   called at tests/contrib/moe/test_fused_moe.py:38,87.
 *   pyhip_moe_topk_grouped_sigmoid  DeepSeek-V3 routing: sigmoid scores, the experts form n_group equal groups
 *                                   of consecutive experts, the topk_group groups with the largest sum of their
 *                                   two best scores stay, top-k inside them.  Not in the reference (its tests
 *                                   draw ids with torch.topk(randn), tests/contrib/moe/test_moe_sorting.py:81-84);
 *                                   n_group must be a power of two <= 64. */
int pyhip_moe_topk_softmax(const float* gating, int tokens, int experts, int topk, int renormalize,
                           float* topk_weight, int32_t* topk_ids, pyhip_stream_t stream);
int pyhip_moe_topk_grouped_sigmoid(const float* gating, int tokens, int experts, int topk, int n_group, int topk_group,
                                   int renormalize, float* topk_weight, int32_t* topk_ids, pyhip_stream_t stream);

/* ------------------------------------------------------------------------------------------
 * Routing sort.  Replaces aiter.fused_moe.moe_sorting as called at src/contrib/fused_moe.py:283,
 * 301-305,368-372 (CPU statement of the result: src/contrib/fused_moe.py:56-100; in-tree C++
 * statement: archive/ck_tile/ck_tile/host/reference/reference_moe_sorting.hpp:13-117) and the
 * JIT sorter src/contrib/moe_sorting.py:7-212.
 *
 *   n_blk             = pyhip_moe_sorting_max_blocks(tokens, topk, experts, block_size)
 *   sorted_ids        u32 [n_blk * block_size]  (slot << 24) | token ; padding (topk << 24) | tokens
 *   sorted_weights    f32 [n_blk * block_size]  routing weight ; padding 0
 *   sorted_expert_ids u32 [n_blk]               (local) expert of each block ; 0xFFFFFFFF past the end
 *   num_valid_ids     u32 [2]                   { padded total, number of (local) tokens }
 * Order: experts ascending, then tokens, then slots (deterministic).  expert_mask (device int32
 * [experts], may be NULL) drops the pairs of masked experts and makes expert ids local;
 * num_local_tokens (device int32 scalar, may be NULL) limits the tokens that are read.
 * moe_out (may be NULL) is zero-filled over moe_out_bytes, as the reference's sorter does for the
 * layer output.  workspace: pyhip_moe_sorting_workspace_bytes() bytes of device memory.
 * schedule (may be NULL; pyhip_moe_schedule_words(experts) = 2 * experts + 1 u32 words) receives the table the
 * grouped GEMMs below walk as a persistent grid: schedule[e], e = 0..experts, is the number of row blocks of
 * the experts before e, schedule[experts + 1 + e] the local id of expert e.  A GEMM orders its tiles expert ->
 * weight tile -> row block and gives each of the 8 XCDs an equal run of that list, so skewed expert loads still
 * fill every XCD.  It has no counterpart in the reference, which launches one workgroup per (tile, worst-case
 * block) (src/contrib/moe_gemm_mxfp4.py:1000-1011). */
int64_t pyhip_moe_sorting_max_blocks(int64_t tokens, int topk, int experts, int block_size);
int64_t pyhip_moe_sorting_workspace_bytes(int64_t tokens, int topk, int experts);
int64_t pyhip_moe_schedule_words(int experts);
int pyhip_moe_sorting(const int32_t* topk_ids, const float* topk_weights, int tokens, int topk, int experts,
                      int block_size, const int32_t* expert_mask, const int32_t* num_local_tokens,
                      uint32_t* sorted_ids, float* sorted_weights, uint32_t* sorted_expert_ids,
                      uint32_t* num_valid_ids, uint32_t* schedule, void* moe_out, int64_t moe_out_bytes,
                      void* workspace, int64_t workspace_bytes, pyhip_stream_t stream);

/* The same sort with the dynamic MXFP4 quantisation of the layer input (pyhip_moe_act_quant_mxfp4 below: x, row
 * stride, rows, K -> q, scales) carried in the sort's own launches: the two are independent, and the sort has
 * a single-workgroup phase during which the quantisation runs on the rest of the GPU.  One dispatch less than
 * calling both; the results are those of the separate calls.  In the reference the two are separate steps as well
 * (src/contrib/fused_moe.py:283 and tests/contrib/moe/test_moe.py:664-679). */
int pyhip_moe_sorting_quant(const int32_t* topk_ids, const float* topk_weights, int tokens, int topk, int experts,
                            int block_size, const int32_t* expert_mask, const int32_t* num_local_tokens,
                            uint32_t* sorted_ids, float* sorted_weights, uint32_t* sorted_expert_ids,
                            uint32_t* num_valid_ids, uint32_t* schedule, void* workspace, int64_t workspace_bytes,
                            const void* x_bf16, int64_t row_stride_elems, int64_t rows, int K, uint8_t* q,
                            uint8_t* scales, pyhip_stream_t stream);

/* Router + sort in one call, the two steps before the GEMMs (aiter.fused_topk followed by
 * aiter.fused_moe.moe_sorting in the reference: tests/contrib/moe/test_fused_moe.py:38,87 and
 * src/contrib/fused_moe.py:283).  gating f32 [tokens, experts]; n_group = 0 selects pyhip_moe_topk_softmax's
 * router, n_group > 0 pyhip_moe_topk_grouped_sigmoid's; the picks are written to topk_weight / topk_ids (both
 * required: the top-k reduction and the caller read them) and sorted as pyhip_moe_sorting does.  x_bf16 (may be
 * NULL) .. scales: the input quantisation of pyhip_moe_sorting_quant.  Up to 64 tokens (and 512 experts, a power of
 * two times 64) all of it is ONE launch: the sort's single workgroup routes the tokens itself; larger inputs take
 * the router's own launch first.  Same results either way.  experts must be a multiple of 64. */
int pyhip_moe_route_sorting(const float* gating, int tokens, int topk, int experts, int n_group, int topk_group,
                            int renormalize, int block_size, const int32_t* expert_mask,
                            const int32_t* num_local_tokens, float* topk_weight, int32_t* topk_ids,
                            uint32_t* sorted_ids, float* sorted_weights, uint32_t* sorted_expert_ids,
                            uint32_t* num_valid_ids, uint32_t* schedule, void* workspace, int64_t workspace_bytes,
                            const void* x_bf16, int64_t row_stride_elems, int64_t rows, int K, uint8_t* q,
                            uint8_t* scales, pyhip_stream_t stream);

/* ------------------------------------------------------------------------------------------
 * Dynamic MXFP4 quantisation of bf16 activations (1x32 blocks, e8m0 scale
 * 2^(floor(log2 amax) - 2), e2m1 round-to-nearest-even).  Replaces
 * aiter.get_hip_quant(QuantType.per_1x32) + fp4_utils.moe_mxfp4_sort as used at
 * tests/contrib/moe/test_moe.py:664-679,732-744.
 *   x       bf16 [rows, K], row stride row_stride_elems
 *   q       u8   [rows, K/2]   low nibble = even element
 *   scales  u8   [rows, pyhip_moe_act_scale_stride(K)]  every 16-byte group stored 4x4-transposed:
 *           byte kb*4 + i = scale of block 4*i + kb (the grouped GEMM's operand order)
 *   rows_limit  device u32 scalar (may be NULL): only rows < *rows_limit are processed. */
int64_t pyhip_moe_act_scale_stride(int K);
int pyhip_moe_act_quant_mxfp4(const void* x_bf16, int64_t row_stride_elems, int64_t rows, int K, uint8_t* q,
                              uint8_t* scales, const uint32_t* rows_limit, pyhip_stream_t stream);

/* ------------------------------------------------------------------------------------------
 * Stage 1: gate_up grouped GEMM with the fused gated activation.  Replaces moe_gemm_mxfp4(gate_up=True),
 * src/contrib/moe_gemm_mxfp4.py:972-1290 (launch: tests/contrib/moe/test_moe.py:720-730).
 *   activation   0: SiLU(gate) * up;  1: gpt-oss's clamped SwiGLU, min(gate, L) * sigmoid(1.702 * min(gate, L)) *
 *                (clamp(up, -L, L) + 1) with L = swiglu_limit > 0 (tests/contrib/moe/test_moe.py:73-82)
 *   a_q/a_scale  quantised hidden states [tokens, hidden/2] / scales (token order, see above)
 *   w1           u8 [experts, 2*inter, hidden/2], gate rows then up rows, pre-shuffled as
 *                src/misc.py:116-130 (pre_shuffle(x, 16))
 *   w1_scale     e8m0, shuffled as tests/contrib/moe/test_fused_moe.py:222-236 over [experts*2*inter, hidden/32]
 *   bias1        bf16 [experts, 2*inter] or NULL
 *   a2           bf16 [n_blk*block_m, inter], row = sorted position (padding rows are zero); may be NULL
 *   a2_q/a2_scale  (both or neither; may be NULL) the MXFP4 quantisation of a2 in the layout of
 *                pyhip_moe_act_quant_mxfp4, written by the same kernel: bit-identical to quantising a2
 *                afterwards, and it replaces the second aiter.get_hip_quant + moe_mxfp4_sort call of
 *                tests/contrib/moe/test_moe.py:732-744.  Needs inter % 512 == 0.  At least one of a2 and
 *                a2_q must be given.
 *   hidden_pad, inter_pad   how many of the last columns of `hidden` / of the last rows of each half of `inter` are
 *                zero padding (the reference operator's hidden_pad / intermediate_pad, src/contrib/fused_moe.py:149-150:
 *                shapes such as gpt-oss's 2880 arrive padded to the tiles' multiples).  0 <= pad < size.  The padding of
 *                the weights must be zeros; the kernels do not fetch groups of 32 (stage 2: 64) weight rows that are all
 *                padding, nor (16- and 32-row blocks) groups of 32 columns that are; results are the same as with 0, 0.
 * block_m must equal the block_size the sort ran with and `experts` the expert count it ran with;
 * block_m is 16, 32, 64, 128, 160, 192, 256 or 288; hidden % 512 == 0, inter % 128 == 0.  schedule: as written by pyhip_moe_sorting, or NULL (then one
 * workgroup per tile and worst-case block is launched, as the reference does). */
int pyhip_moe_gemm1_mxfp4(const uint8_t* a_q, const uint8_t* a_scale, const uint8_t* w1, const uint8_t* w1_scale,
                          const void* bias1_bf16, const uint32_t* sorted_ids, const uint32_t* sorted_expert_ids,
                          const uint32_t* num_valid_ids, const uint32_t* schedule, void* a2_bf16, uint8_t* a2_q,
                          uint8_t* a2_scale, int tokens, int topk, int experts, int hidden, int inter, int hidden_pad,
                          int inter_pad, int block_m, int64_t n_blk, int activation, float swiglu_limit,
                          pyhip_stream_t stream);

/* Stage 2: down grouped GEMM, times the routing weight.  Replaces moe_gemm_mxfp4(gate_up=False),
 * src/contrib/moe_gemm_mxfp4.py:1291-1333 (launch: tests/contrib/moe/test_moe.py:751-763).
 *   a2_q/a2_scale  quantised stage-1 output [n_blk*block_m, inter/2] / scales (sorted-row order)
 *   w2, w2_scale   u8 [experts, hidden, inter/2] pre-shuffled; e8m0 shuffled over [experts*hidden, inter/32]
 *   bias2          bf16 [experts, hidden] or NULL (added before the routing weight)
 *   out3           bf16 [tokens, topk, hidden]; only (token, slot) pairs that were sorted are written: the slots of
 *                  pairs the sort dropped (expert id outside [0, experts), masked expert, token past the local
 *                  count) keep whatever the buffer held.  Reduce with pyhip_moe_topk_reduce_routed, which leaves
 *                  those slots out by the same rule, or clear out3 first when the plain pyhip_moe_topk_reduce is
 *                  used with a routing that drops pairs.
 *   hidden_pad, inter_pad   as for stage 1: here the last hidden_pad rows of w2 and its last inter_pad columns
 * inter % 512 == 0, hidden % 256 == 0. */
int pyhip_moe_gemm2_mxfp4(const uint8_t* a2_q, const uint8_t* a2_scale, const uint8_t* w2, const uint8_t* w2_scale,
                          const void* bias2_bf16, const uint32_t* sorted_ids, const float* sorted_weights,
                          const uint32_t* sorted_expert_ids, const uint32_t* num_valid_ids,
                          const uint32_t* schedule, void* out3_bf16, int tokens, int topk, int experts, int hidden,
                          int inter, int hidden_pad, int inter_pad, int block_m, int64_t n_blk, pyhip_stream_t stream);

/* The same two GEMMs on the eight-wave tile of 256 rows x 256 weight rows whose operands BOTH go through LDS (LDS-DMA
 * into a ring of five weight stages and three activation stages, two wave rows half a K-step apart), the tile shape of
 * the reference's prefill kernel (src/contrib/moe_gemm_mxfp4.py:318-637).  Arguments as pyhip_moe_gemm1_mxfp4 /
 * pyhip_moe_gemm2_mxfp4 with block_m = 256: the sort must have been run with block_size 256 and must have written the
 * schedule (required here); hidden / inter (the K of the GEMM) >= 1024; at most 512 experts.  Results are bit-identical
 * to the other tiles'.  Measured slower than the four-wave 256-row tile (DeepSeek-V3 shape, 6144 tokens: layer 1.86
 * against 1.70 ms), so no other entry point selects it. */
int pyhip_moe_gemm1_mxfp4_lds(const uint8_t* a_q, const uint8_t* a_scale, const uint8_t* w1, const uint8_t* w1_scale,
                              const void* bias1_bf16, const uint32_t* sorted_ids, const uint32_t* sorted_expert_ids,
                              const uint32_t* num_valid_ids, const uint32_t* schedule, void* a2_bf16, uint8_t* a2_q,
                              uint8_t* a2_scale, int tokens, int topk, int experts, int hidden, int inter,
                              int64_t n_blk, int activation, float swiglu_limit, pyhip_stream_t stream);
int pyhip_moe_gemm2_mxfp4_lds(const uint8_t* a2_q, const uint8_t* a2_scale, const uint8_t* w2, const uint8_t* w2_scale,
                              const void* bias2_bf16, const uint32_t* sorted_ids, const float* sorted_weights,
                              const uint32_t* sorted_expert_ids, const uint32_t* num_valid_ids,
                              const uint32_t* schedule, void* out3_bf16, int tokens, int topk, int experts,
                              int hidden, int inter, int64_t n_blk, pyhip_stream_t stream);

/* Stage 2 with the top-k reduction in its epilogue: bf16(acc * routing weight) is added into out[tokens, hidden]
 * (bf16, cleared by the caller) with packed bf16 atomics; no out3, no pyhip_moe_topk_reduce.  Replaces the atomic
 * variant of the reference, src/contrib/moe_gemm_mxfp4.py:1334-1398 (and src/contrib/moe.py:703-787).  The result
 * depends on the arrival order of a token's slots (each addition rounds to bf16); block_m is 16 or 128.  The
 * deterministic out3 + reduce pair above is what pyhip_moe_forward uses. */
int pyhip_moe_gemm2_mxfp4_atomic(const uint8_t* a2_q, const uint8_t* a2_scale, const uint8_t* w2,
                                 const uint8_t* w2_scale, const void* bias2_bf16, const uint32_t* sorted_ids,
                                 const float* sorted_weights, const uint32_t* sorted_expert_ids,
                                 const uint32_t* num_valid_ids, const uint32_t* schedule, void* out_bf16, int tokens,
                                 int topk, int experts, int hidden, int inter, int block_m, int64_t n_blk,
                                 pyhip_stream_t stream);

/* Stage 2 with the top-k reduction done inside it, deterministically: out3 is written as by pyhip_moe_gemm2_mxfp4, and the
 * workgroup that stores the last of a token's slots for a 256-channel weight tile sums that token's slots in fp32 in
 * slot order and writes out[tokens, hidden] (bf16, or fp32 when out_is_f32 != 0): the arithmetic of
 * pyhip_moe_topk_reduce_routed, so the same bits whatever the arrival order, with no reduction launch and no waiting
 * between workgroups.  The deterministic counterpart of the reference's atomic epilogue
 * (src/contrib/moe_gemm_mxfp4.py:1334-1398); pyhip_moe_forward keeps the two-kernel path, which measures faster at
 * prefill sizes.
 *   topk_ids, expert_mask, num_local_tokens   the routing as given to the sort (for the drop rule)
 *   arrive        int32 [tokens * hidden / 256], scratch (initialised by this call)
 * block_m 16, 128 or 288. */
int pyhip_moe_gemm2_mxfp4_reduce(const uint8_t* a2_q, const uint8_t* a2_scale, const uint8_t* w2, const uint8_t* w2_scale,
                                 const void* bias2_bf16, const uint32_t* sorted_ids, const float* sorted_weights,
                                 const uint32_t* sorted_expert_ids, const uint32_t* num_valid_ids,
                                 const uint32_t* schedule, void* out3_bf16, const int32_t* topk_ids,
                                 const int32_t* expert_mask, const int32_t* num_local_tokens, int32_t* arrive, void* out,
                                 int out_is_f32, int tokens, int topk, int experts, int hidden, int inter, int block_m,
                                 int64_t n_blk, pyhip_stream_t stream);

/* ------------------------------------------------------------------------------------------
 * The same two GEMMs with bf16 activations ("w4a16"): weights are expanded from MXFP4 to bf16 in registers
 * and multiplied with the bf16 MFMA; nothing is quantised at run time.  Replaces moe_2stage_splitk with fp4
 * weights, src/contrib/moe.py:362-787 (gate_up: with_silu=True; down: :471-500,703-787; launches:
 * tests/contrib/moe/test_moe.py:347-374), the variant the reference uses when few tokens are routed.
 * Buffers as above, except hidden / a2 are bf16 ([tokens, hidden] in token order; [n_blk*block_m, inter] in
 * sorted-row order) and the down GEMM writes out3[tokens, topk, hidden] for pyhip_moe_topk_reduce instead of
 * adding into the layer output with atomics.  block_m is 16, 32 or 64; hidden % 512 == 0, inter % 512 == 0.
 * split_k: 4 = the four waves of a workgroup share a 64-row weight tile and split K between them (partial sums
 * meet in LDS; four times as many workgroups), 16 = the same with sixteen waves per workgroup (block_m = 16,
 * K >= 2048), 32 = sixteen waves share a 32-row weight tile and keep three K-steps in flight (down GEMM; block_m = 16,
 * K >= 2048; the gate_up GEMM takes 16 instead), 1 = every wave owns 64 rows over the whole K, 0 = split when the launch would otherwise have fewer
 * than 2048 workgroups with work, sixteen-fold (the down GEMM: split 32) when even then fewer workgroups than CUs would start and K >= 8192.  activation / swiglu_limit: as for
 * pyhip_moe_gemm1_mxfp4. */
int pyhip_moe_gemm1_w4a16(const void* hidden_bf16, const uint8_t* w1, const uint8_t* w1_scale, const void* bias1_bf16,
                          const uint32_t* sorted_ids, const uint32_t* sorted_expert_ids, const uint32_t* num_valid_ids,
                          void* a2_bf16, int tokens, int topk, int experts, int hidden, int inter, int block_m,
                          int64_t n_blk, int split_k, int activation, float swiglu_limit, pyhip_stream_t stream);
int pyhip_moe_gemm2_w4a16(const void* a2_bf16, const uint8_t* w2, const uint8_t* w2_scale, const void* bias2_bf16,
                          const uint32_t* sorted_ids, const float* sorted_weights, const uint32_t* sorted_expert_ids,
                          const uint32_t* num_valid_ids, void* out3_bf16, int tokens, int topk, int experts,
                          int hidden, int inter, int block_m, int64_t n_blk, int split_k, pyhip_stream_t stream);

/* The same two GEMMs for a single token, without the routing sort in front of them: the kernels read the token's
 * topk_ids [topk] / topk_weights [topk] themselves, one 16-row block per slot, and apply the sort's drop rule
 * (expert id outside [0, experts), masked expert, *num_local_tokens < 1) and the local expert numbering under an
 * expert mask.  The reference's decode path runs its sort for every token count (src/contrib/fused_moe.py:283-305);
 * at one token the sort is a launch of 6 us on the critical path of a layer of 40-50 us.
 *   a2    bf16 [topk * 16, inter]: slot s is row 16 * s (what a sort with block_size 16 gives when every slot has an
 *         expert of its own)
 *   out3  bf16 [1, topk, hidden]; dropped slots are left unwritten, as by pyhip_moe_gemm2_w4a16
 * Results equal those of pyhip_moe_sorting + pyhip_moe_gemm{1,2}_w4a16 bit for bit.  pyhip_moe_forward takes this
 * path by itself for tokens == 1 with bf16 activations. */
int pyhip_moe_gemm1_w4a16_token(const void* hidden_bf16, const uint8_t* w1, const uint8_t* w1_scale,
                                const void* bias1_bf16, const int32_t* topk_ids, const int32_t* expert_mask,
                                const int32_t* num_local_tokens, void* a2_bf16, int topk, int experts, int hidden,
                                int inter, int split_k, int activation, float swiglu_limit, pyhip_stream_t stream);
int pyhip_moe_gemm2_w4a16_token(const void* a2_bf16, const uint8_t* w2, const uint8_t* w2_scale, const void* bias2_bf16,
                                const int32_t* topk_ids, const float* topk_weights, const int32_t* expert_mask,
                                const int32_t* num_local_tokens, void* out3_bf16, int topk, int experts, int hidden,
                                int inter, int split_k, pyhip_stream_t stream);

/* ------------------------------------------------------------------------------------------
 * Top-k reduction out[t, :] = sum_slot in[t, slot, :] (fp32, slots in index order), one rounding.
 * Replaces moe_gemm_final_reduce_bf16, src/contrib/moe_gemm_mxfp4.py:199-282
 * (launch: tests/contrib/moe/test_moe.py:764-771).  out is bf16 or (out_is_f32 != 0) fp32.
 * num_valid_ids (may be NULL): when given, only tokens < num_valid_ids[1] are reduced.
 * Every slot of in[] is read: after a sort that dropped pairs (expert_mask, ids out of range) the down GEMMs have
 * left those slots unwritten, so either in[] was cleared before the GEMM or pyhip_moe_topk_reduce_routed is used. */
int pyhip_moe_topk_reduce(const void* in_bf16, void* out, int64_t tokens, int topk, int hidden, int out_is_f32,
                          const uint32_t* num_valid_ids, pyhip_stream_t stream);

/* The same reduction with the routing in view: a slot is left out (neither read nor added) when the sort dropped
 * its pair, i.e. when topk_ids[t, slot] is outside [0, experts), names an expert that expert_mask (device int32
 * [experts], may be NULL) masks, or t >= *num_local_tokens (device int32 scalar, may be NULL); rows of tokens past
 * the local count are written as zeros.  The down GEMMs write only the pairs that were sorted, so with this
 * reduction out3 needs no clearing (the reference clears its output buffer inside the sorter instead,
 * src/contrib/fused_moe.py:301-306) and under expert parallelism only the owned slots are read. */
int pyhip_moe_topk_reduce_routed(const void* in_bf16, void* out, int64_t tokens, int topk, int hidden, int out_is_f32,
                                 const int32_t* topk_ids, int experts, const int32_t* expert_mask,
                                 const int32_t* num_local_tokens, pyhip_stream_t stream);

/* ------------------------------------------------------------------------------------------
 * Zero fill of device memory with a kernel (safe inside a captured graph, where memset nodes are not).  The
 * reference zeroes its buffers with torch (src/contrib/fused_moe.py:306, moe_sorting's moe_buf). */
int pyhip_moe_zero_fill(void* p, int64_t bytes, pyhip_stream_t stream);

/* ------------------------------------------------------------------------------------------
 * Measurement probe (no counterpart in the reference; used by bench.py --frontier only): the inner loop of the 288-row
 * MXFP4 GEMM reduced to its instruction and memory pattern, one workgroup of four waves per CU, `iters` K-groups of 288
 * scaled FP4 MFMAs per wave.  variant 0: MFMAs only; 1: + LDS operand reads; 2: + the weight stream (16 KB per wave and
 * K-group from `buf`, prefetched one K-group ahead); 3: + 29 LDS-DMA operations per K-group; 4: as 2 with every second
 * MFMA replaced by VALU moves; 5: as 2 with none; 6: as 3 with the weight tiles from an L2-resident region; 7, 8, 9: the
 * 128-row tile's pattern (two workgroups per CU, 128 MFMAs per wave and K-group): MFMAs + operand reads; everything with
 * weights from the L2; everything with weights streamed.  Enqueues `launches` launches on `stream`; the caller times them.
 *   buf        device buffer of at least 2^30 + 2^24 bytes, read only (fill it with noise: what the matrix pipeline
 *              draws, and with it the clock, depends on the operands)
 *   sink       device int32[4], never written in practice
 *   workgroups receives the workgroups per launch (the CU count, or twice that) */
int pyhip_moe_probe_mfma_stream(int variant, int iters, const void* buf, int64_t buf_bytes, int32_t* sink, int launches,
                                int* workgroups, pyhip_stream_t stream);

/* ------------------------------------------------------------------------------------------
 * The whole layer in one call: sort (+ input quantisation) -> gate_up GEMM -> down GEMM -> top-k reduce, i.e. the
 * body of the reference's fused_moe (src/contrib/fused_moe.py:128-576) for the MXFP4 path, with every
 * intermediate buffer carved out of `workspace` (pyhip_moe_forward_workspace_bytes() bytes, 256-byte aligned)
 * instead of being allocated per call.  Enqueues on `stream`, never synchronises, allocates nothing.
 *   hidden        bf16 [tokens, hidden], row stride hidden_row_stride elements (== hidden when w4a16 != 0)
 *   w1, w2, scales, biases, expert_mask, num_local_tokens: as for the step-by-step entry points above
 *   out           bf16 (or fp32 when out_is_f32 != 0) [tokens, hidden]
 *   experts       the expert count the router saw (the length of expert_mask when one is given)
 *   hidden, inter the sizes the weights have, padding included; hidden_pad, inter_pad: how much of them is zero padding
 *                 (as for pyhip_moe_gemm1_mxfp4; the bf16-activation kernels take no notice)
 *   block_m       the row block: 16/32/64, with MXFP4 activations also 128/160/192/256/288
 *   w4a16         0 = MXFP4 activations (pyhip_moe_gemm*_mxfp4), 1 = bf16 activations (pyhip_moe_gemm*_w4a16)
 * pyhip_moe_pick_block_m / pyhip_moe_pick_w4a16 give the choices the reference's operator makes inside fused_moe
 * (block_size_M=None, method="auto": src/contrib/fused_moe.py:128-155) as this library makes them (the row block for
 * the kernel family given by w4a16; with bf16 activations it is at most 64). */
int pyhip_moe_pick_block_m(int64_t tokens, int topk, int experts, int hidden, int w4a16);
int pyhip_moe_pick_w4a16(int64_t tokens, int topk, int experts, int hidden);
int64_t pyhip_moe_forward_workspace_bytes(int64_t tokens, int topk, int experts, int hidden, int inter, int block_m,
                                          int w4a16);
int pyhip_moe_forward(const void* hidden_bf16, int64_t hidden_row_stride, const uint8_t* w1, const uint8_t* w1_scale,
                      const uint8_t* w2, const uint8_t* w2_scale, const void* bias1_bf16, const void* bias2_bf16,
                      const int32_t* topk_ids, const float* topk_weights, const int32_t* expert_mask,
                      const int32_t* num_local_tokens, void* out, int out_is_f32, int tokens, int topk, int experts,
                      int hidden, int inter, int hidden_pad, int inter_pad, int block_m, int w4a16, int split_k,
                      int activation, float swiglu_limit, void* workspace, int64_t workspace_bytes, pyhip_stream_t stream);

/* pyhip_moe_forward with the router inside the call: gating f32 [tokens, experts] in (n_group / topk_group /
 * renormalize as for pyhip_moe_route_sorting), the picks out in topk_ids / topk_weights next to the layer output.
 * The reference's callers run aiter.fused_topk and then fused_moe (tests/contrib/moe/test_fused_moe.py:38-60). */
int pyhip_moe_forward_routed(const void* hidden_bf16, int64_t hidden_row_stride, const uint8_t* w1,
                             const uint8_t* w1_scale, const uint8_t* w2, const uint8_t* w2_scale,
                             const void* bias1_bf16, const void* bias2_bf16, const float* gating, int n_group,
                             int topk_group, int renormalize, int32_t* topk_ids, float* topk_weights,
                             const int32_t* expert_mask, const int32_t* num_local_tokens, void* out, int out_is_f32,
                             int tokens, int topk, int experts, int hidden, int inter, int hidden_pad, int inter_pad,
                             int block_m, int w4a16, int split_k, int activation, float swiglu_limit, void* workspace,
                             int64_t workspace_bytes, pyhip_stream_t stream);

/* pyhip_moe_forward without the workspace argument: the intermediates live in a device array that belongs to the
 * library (64 MiB, pyhip_moe_forward_static_capacity(); one copy per GPU, held until the process ends).  It has no
 * counterpart in the reference.  It is for callers that cannot allocate device memory: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  The call allocates nothing (no hipMalloc, no
 * hipFree, no allocating library routine); calls whose intermediates exceed the capacity are refused with error 1
 * before anything is launched (decode-sized calls fit: DeepSeek-V3 shape, 128 tokens, bf16 activations: 35 MiB).
 * Same arguments, kernels and results as pyhip_moe_forward.  All calls on one GPU share the array: calls that
 * overlap on one GPU (two streams, two threads) race; nothing in the array needs clearing between calls.
 * pyhip_moe_forward_static_capacity() returns the array's size and makes the runtime map the array on the current
 * device: callers that capture the layer call in a graph run it once per device beforehand, so that the first call
 * inside the capture has nothing left to set up. */
int64_t pyhip_moe_forward_static_capacity(void);
int pyhip_moe_forward_static(const void* hidden_bf16, int64_t hidden_row_stride, const uint8_t* w1,
                             const uint8_t* w1_scale, const uint8_t* w2, const uint8_t* w2_scale,
                             const void* bias1_bf16, const void* bias2_bf16, const int32_t* topk_ids,
                             const float* topk_weights, const int32_t* expert_mask, const int32_t* num_local_tokens,
                             void* out, int out_is_f32, int tokens, int topk, int experts, int hidden, int inter,
                             int hidden_pad, int inter_pad, int block_m, int w4a16, int split_k, int activation,
                             float swiglu_limit, pyhip_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* PYHIP_MOE_H */
