// The whole layer behind one call: sort (+ input quantisation) -> gate_up GEMM -> down GEMM -> top-k reduce, with
// every intermediate buffer carved out of a workspace the caller provides.  It is what pyhip_amd/fused_moe.py does
// step by step (the reference's operator, src/contrib/fused_moe.py:128-576, allocates its intermediates with torch
// and launches its kernels one by one from Python); the choice of kernel family and row block stays with the caller.
#include "common.h"

extern "C" {
int64_t pyhip_moe_sorting_max_blocks(int64_t tokens, int topk, int experts, int block_size);
int64_t pyhip_moe_sorting_workspace_bytes(int64_t tokens, int topk, int experts);
int64_t pyhip_moe_schedule_words(int experts);
int64_t pyhip_moe_act_scale_stride(int K);
int pyhip_moe_sorting(const int32_t*, const float*, int, int, int, int, const int32_t*, const int32_t*, uint32_t*, float*,
                      uint32_t*, uint32_t*, uint32_t*, void*, int64_t, void*, int64_t, hipStream_t);
int pyhip_moe_sorting_quant(const int32_t*, const float*, int, int, int, int, const int32_t*, const int32_t*, uint32_t*,
                            float*, uint32_t*, uint32_t*, uint32_t*, void*, int64_t, const void*, int64_t, int64_t, int,
                            uint8_t*, uint8_t*, hipStream_t);
int pyhip_moe_gemm1_mxfp4(const uint8_t*, const uint8_t*, const uint8_t*, const uint8_t*, const void*, const uint32_t*,
                          const uint32_t*, const uint32_t*, const uint32_t*, void*, uint8_t*, uint8_t*, int, int, int, int,
                          int, int, int, int, int64_t, int, float, hipStream_t);
int pyhip_moe_gemm2_mxfp4(const uint8_t*, const uint8_t*, const uint8_t*, const uint8_t*, const void*, const uint32_t*,
                          const float*, const uint32_t*, const uint32_t*, const uint32_t*, void*, int, int, int, int, int,
                          int, int, int, int64_t, hipStream_t);
int pyhip_moe_gemm1_w4a16(const void*, const uint8_t*, const uint8_t*, const void*, const uint32_t*, const uint32_t*,
                          const uint32_t*, void*, int, int, int, int, int, int, int64_t, int, int, float, hipStream_t);
int pyhip_moe_gemm2_w4a16(const void*, const uint8_t*, const uint8_t*, const void*, const uint32_t*, const float*,
                          const uint32_t*, const uint32_t*, void*, int, int, int, int, int, int, int64_t, int, hipStream_t);
int pyhip_moe_gemm1_w4a16_token(const void*, const uint8_t*, const uint8_t*, const void*, const int32_t*, const int32_t*,
                                const int32_t*, void*, int, int, int, int, int, int, float, hipStream_t);
int pyhip_moe_gemm2_w4a16_token(const void*, const uint8_t*, const uint8_t*, const void*, const int32_t*, const float*,
                                const int32_t*, const int32_t*, void*, int, int, int, int, int, hipStream_t);
int pyhip_moe_route_sorting(const float*, int, int, int, int, int, int, int, const int32_t*, const int32_t*, float*, int32_t*,
                            uint32_t*, float*, uint32_t*, uint32_t*, uint32_t*, void*, int64_t, const void*, int64_t, int64_t,
                            int, uint8_t*, uint8_t*, hipStream_t);
int pyhip_moe_topk_reduce_routed(const void*, void*, int64_t, int, int, int, const int32_t*, int, const int32_t*,
                                 const int32_t*, hipStream_t);
}

namespace {
struct Carve
{
    int64_t off = 0;
    int64_t take(int64_t bytes)
    {
        int64_t o = off;
        off += (bytes + 255) / 256 * 256;
        return o;
    }
};
struct Layout
{
    int64_t n_blk, rows2;
    int64_t sorted_ids, sorted_w, sorted_e, num_valid, sched, sort_ws, sort_ws_bytes, a1_q, a1_s, a2, a2_q, a2_s, out3;
    int64_t total;
};
Layout make_layout(int64_t T, int k, int E, int H, int I, int bm, int w4a16)
{
    Layout l;
    Carve c;
    l.n_blk         = pyhip_moe_sorting_max_blocks(T, k, E, bm);
    l.rows2         = l.n_blk * bm;
    l.sorted_ids    = c.take(l.rows2 * 4);
    l.sorted_w      = c.take(l.rows2 * 4);
    l.sorted_e      = c.take(l.n_blk * 4);
    l.num_valid     = c.take(8);
    l.sched         = c.take(pyhip_moe_schedule_words(E) * 4);
    l.sort_ws_bytes = pyhip_moe_sorting_workspace_bytes(T, k, E);
    l.sort_ws       = c.take(l.sort_ws_bytes);
    l.a1_q = l.a1_s = l.a2 = l.a2_q = l.a2_s = 0;
    if(w4a16)
        l.a2 = c.take(l.rows2 * (int64_t)I * 2);
    else
    {
        l.a1_q = c.take(T * (int64_t)(H / 2));
        l.a1_s = c.take(T * pyhip_moe_act_scale_stride(H));
        l.a2_q = c.take(l.rows2 * (int64_t)(I / 2));
        l.a2_s = c.take(l.rows2 * pyhip_moe_act_scale_stride(I));
    }
    l.out3  = c.take(T * (int64_t)k * H * 2);
    l.total = c.off;
    return l;
}
}   // namespace

// The choices pyhip_amd/fused_moe.py makes for method="auto" and block_size_M=None (pick_block_m, pick_w4a16; the
// measurements behind them are quoted there), for callers that bind the library without the Python layer.
extern "C" int pyhip_moe_pick_block_m(int64_t tokens, int topk, int experts, int hidden, int w4a16)
{
    const double est = (double)tokens * topk / (experts > 0 ? experts : 1);      // routed rows per expert, on average
    // The tile is chosen from the AVERAGE load, which is all that is known before the sort has run, with room for routers
    // that load their experts unevenly: every extra row block of a busy expert streams that expert's weights again, while
    // a tile that is larger than a quiet expert needs only costs the occupancy of its kernel.  One step up the ladder
    // from "twice the mean" costs 1-2 % under an even router and saves 11-17 % under a Zipf(1.1) one (whole layer, ms,
    // tiles of 16 / 32 / 64 rows; DeepSeek-V3 shape, 128 tokens = 4 rows per expert: 0.904 / 0.917 / 0.942, gpt-oss shape, 256
    // tokens = 8: 0.301 / 0.305 / 0.320; Qwen3 shape with the Zipf router, 64 tokens = 4: 0.123 / 0.103 / 0.108, 128 = 8:
    // 0.169 / 0.140 / 0.137, 256 = 16: 0.218 / 0.191 / 0.169).
    // With a handful of experts (Mixtral: 8) every expert gets many rows, the loads are even in relative terms, and the
    // number of tiles is what such layers are short of: "twice the mean" stays (Mixtral shape, 32 tokens: 0.134 ms with
    // 16-row blocks, 0.158 with 32).
    // The same holds for the bf16-activation kernels, whose 32-row tile already halves the waves per SIMD (DeepSeek-V3
    // shape, 128 tokens, forced: gate_up 623 us with 16-row blocks, 761 with 32); their row block is at most 64.
    if(experts < 32 || w4a16)
    {
        for(int bm = 16; bm <= 64; bm *= 2)
            if(2 * est <= bm)
                return bm;
    }
    else
    {
        if(est < 4)
            return 16;
        if(est < 12)
            return 32;
        if(est <= 32)
            return 64;
    }
    if(w4a16)
        return 64;
    // Prefill sizes: 128 rows, except where a taller tile lets nearly every expert fit ONE row block, so that each weight
    // tile is read once instead of two or three times.  The tiles above 128 rows run one wave per SIMD and have a long
    // epilogue, which pays most with a long K loop (hidden >= 6144).  DeepSeek-V3 shape, whole layer, ms, tiles of 128 / 160 /
    // 192 / 256 / 288 rows by expected rows per expert (between machines the order of close neighbours can flip):
    //    96: 1.28 / 1.33 / 1.36 / 1.50 /  -       160: 2.26 / 1.93 / 1.49 / 1.60 / 1.73      232: 1.97 /  -   /  -   / 1.86 / 1.92
    //   104: 1.36 / 1.35 / 1.38 / 1.52 / 1.66     168: 2.08 / 2.22 / 1.55 / 1.62 / 1.75      240: 2.09 /  -   /  -   / 1.96 / 1.94
    //   120: 1.50 / 1.37 / 1.40 / 1.51 / 1.63     176: 2.04 / 2.63 / 1.65 / 1.64 / 1.77      256: 2.26 /  -   /  -   / 2.64 / 2.02
    //   128: 1.72 / 1.39 / 1.42 / 1.53 / 1.65     192: 1.92 / 2.67 / 2.20 / 1.68 / 1.81      272: 2.46 /  -   /  -   / 3.29 / 2.36
    //   136: 1.92 / 1.43 / 1.43 / 1.54 / 1.67     208: 1.91 /  -   /  -   / 1.72 / 1.85      288: 2.57 /  -   /  -   / 3.53 / 2.97
    // With the shorter K loop of hidden 3072 / 4096 only the first step pays, and only under an even router: 100-132
    // expected rows per expert, where the 128-row tile needs a second, nearly empty block for half of the experts (whole
    // layer, ms, 128 / 160 / 192 / 256 rows: Mixtral shape, 512 tokens: 0.210 / 0.191 / 0.198 / 0.216; gpt-oss shape, 4096
    // tokens: 0.564 / 0.499 / 0.513 / 0.556; the Qwen3 shape's Zipf router at 2048 tokens, the same mean: 0.399 / 0.420 /
    // 0.425 / 0.452: most of its experts are far below the mean and pay for the taller tile's empty row groups).  Further
    // up, the taller tiles win by 3-11 % under the even routers at exactly the sizes where an expert fills one block
    // (192 rows at 160 per expert, 288 at 256) and lose up to 20 % under the uneven one and between those sizes: left at
    // 128 rows.
    if(hidden < 6144 && est >= 100 && est <= 132)
        return 160;
    if(hidden >= 6144)
    {
        if(est >= 100 && est <= 132)
            return 160;
        if(est > 132 && est <= 172)
            return 192;
        if(est > 172 && est <= 236)
            return 256;
        if(est > 236 && est <= 276)
            return 288;
    }
    return 128;
}

extern "C" int pyhip_moe_pick_w4a16(int64_t tokens, int topk, int experts, int hidden)
{
    // bf16 activations win (a) when at most one expert in eight gets a row at all (DeepSeek-V3 shape: 1 token 0.046
    // against 0.051 ms, 4 tokens 0.128 against 0.127 ms, 16 tokens 0.393 against 0.377 ms; gpt-oss shape: 4 tokens 0.053
    // against 0.055 ms, 16 tokens 0.141 against 0.134 ms), and (b) in layers with so few experts that the down GEMM of
    // the MXFP4-activation path has fewer than 512 tiles, which the bf16 kernel splits K-wise over four times as many
    // workgroups (Mixtral shape: 1 token 0.054 against 0.071 ms, 16 tokens 0.132 against 0.137 ms, 64 tokens 0.181
    // against 0.140 ms)
    const int64_t pairs  = tokens * topk;
    const bool sparse    = 8 * pairs <= (int64_t)experts;
    const bool few_tiles = (pairs < experts ? pairs : experts) * (hidden / 256) < 512 && pairs <= 8 * (int64_t)experts;
    return sparse || few_tiles;
}

extern "C" int64_t pyhip_moe_forward_workspace_bytes(int64_t tokens, int topk, int experts, int hidden, int inter,
                                                     int block_m, int w4a16)
{
    if(tokens <= 0 || topk <= 0 || experts <= 0 || hidden <= 0 || inter <= 0 || block_m <= 0)
        return 0;
    return make_layout(tokens, topk, experts, hidden, inter, block_m, w4a16).total;
}

namespace {
struct Router
{
    const float* gating = nullptr;      // [tokens, experts] or null: topk_ids / topk_weights are inputs
    int n_group = 0, topk_group = 0, renormalize = 1;
};
}   // namespace

static int forward_impl(const void* hidden_bf16, int64_t hidden_row_stride, const uint8_t* w1, const uint8_t* w1_scale,
                        const uint8_t* w2, const uint8_t* w2_scale, const void* bias1_bf16, const void* bias2_bf16,
                        const Router& router, int32_t* topk_ids, float* topk_weights, const int32_t* expert_mask,
                        const int32_t* num_local_tokens, void* out, int out_is_f32, int tokens, int topk, int experts,
                        int hidden, int inter, int hidden_pad, int inter_pad, int block_m, int w4a16, int split_k,
                        int activation, float swiglu_limit, void* workspace, int64_t workspace_bytes, hipStream_t stream)
{
    PYHIP_REQUIRE(hidden_bf16 && w1 && w1_scale && w2 && w2_scale && topk_ids && topk_weights && out,
                  "moe_forward: null pointer");
    PYHIP_REQUIRE(tokens > 0 && topk > 0 && experts > 0 && hidden > 0 && inter > 0, "moe_forward: bad sizes");
    PYHIP_REQUIRE(block_m == 16 || block_m == 32 || block_m == 64 ||
                      ((block_m == 128 || block_m == 160 || block_m == 192 || block_m == 256 || block_m == 288) && !w4a16),
                  "moe_forward: block_m=%d (16/32/64, and 128/160/192/256/288 with MXFP4 activations)", block_m);
    PYHIP_REQUIRE(!w4a16 || hidden_row_stride == hidden, "moe_forward: the bf16-activation kernels need contiguous rows");
    const Layout l = make_layout(tokens, topk, experts, hidden, inter, block_m, w4a16);
    PYHIP_REQUIRE(workspace && workspace_bytes >= l.total && ((uintptr_t)workspace % 256) == 0,
                  "moe_forward: workspace of %lld bytes (256-byte aligned) needed, %lld given", (long long)l.total,
                  (long long)workspace_bytes);
    uint8_t* ws       = (uint8_t*)workspace;
    uint32_t* s_ids   = (uint32_t*)(ws + l.sorted_ids);
    float* s_w        = (float*)(ws + l.sorted_w);
    uint32_t* s_e     = (uint32_t*)(ws + l.sorted_e);
    uint32_t* n_valid = (uint32_t*)(ws + l.num_valid);
    uint32_t* sched   = (uint32_t*)(ws + l.sched);
    void* out3        = ws + l.out3;
    int rc;
    if(w4a16 && tokens == 1 && !router.gating)
    {
        // a single token with bf16 activations: no sort; the GEMMs read the routing themselves, one block per slot
        rc = pyhip_moe_gemm1_w4a16_token(hidden_bf16, w1, w1_scale, bias1_bf16, topk_ids, expert_mask, num_local_tokens,
                                         ws + l.a2, topk, experts, hidden, inter, split_k, activation, swiglu_limit, stream);
        if(rc)
            return rc;
        rc = pyhip_moe_gemm2_w4a16_token(ws + l.a2, w2, w2_scale, bias2_bf16, topk_ids, topk_weights, expert_mask,
                                         num_local_tokens, out3, topk, experts, hidden, inter, split_k, stream);
        if(rc)
            return rc;
        return pyhip_moe_topk_reduce_routed(out3, out, tokens, topk, hidden, out_is_f32, topk_ids, experts, expert_mask,
                                            num_local_tokens, stream);
    }
    if(router.gating)
        // the routing is part of the call: the sort's own workgroup routes the tokens when there are few of them
        rc = pyhip_moe_route_sorting(router.gating, tokens, topk, experts, router.n_group, router.topk_group,
                                     router.renormalize, block_m, expert_mask, num_local_tokens, topk_weights, topk_ids,
                                     s_ids, s_w, s_e, n_valid, sched, ws + l.sort_ws, l.sort_ws_bytes,
                                     w4a16 ? nullptr : hidden_bf16, hidden_row_stride, tokens, hidden,
                                     w4a16 ? nullptr : ws + l.a1_q, w4a16 ? nullptr : ws + l.a1_s, stream);
    else if(w4a16)
        rc = pyhip_moe_sorting(topk_ids, topk_weights, tokens, topk, experts, block_m, expert_mask, num_local_tokens,
                               s_ids, s_w, s_e, n_valid, sched, nullptr, 0, ws + l.sort_ws, l.sort_ws_bytes, stream);
    else
        rc = pyhip_moe_sorting_quant(topk_ids, topk_weights, tokens, topk, experts, block_m, expert_mask,
                                     num_local_tokens, s_ids, s_w, s_e, n_valid, sched, ws + l.sort_ws, l.sort_ws_bytes,
                                     hidden_bf16, hidden_row_stride, tokens, hidden, ws + l.a1_q, ws + l.a1_s, stream);
    if(rc)
        return rc;
    if(w4a16)
    {
        rc = pyhip_moe_gemm1_w4a16(hidden_bf16, w1, w1_scale, bias1_bf16, s_ids, s_e, n_valid, ws + l.a2, tokens, topk,
                                   experts, hidden, inter, block_m, l.n_blk, split_k, activation, swiglu_limit, stream);
        if(rc)
            return rc;
        rc = pyhip_moe_gemm2_w4a16(ws + l.a2, w2, w2_scale, bias2_bf16, s_ids, s_w, s_e, n_valid, out3, tokens, topk,
                                   experts, hidden, inter, block_m, l.n_blk, split_k, stream);
    }
    else
    {
        rc = pyhip_moe_gemm1_mxfp4(ws + l.a1_q, ws + l.a1_s, w1, w1_scale, bias1_bf16, s_ids, s_e, n_valid, sched, nullptr,
                                   ws + l.a2_q, ws + l.a2_s, tokens, topk, experts, hidden, inter, hidden_pad, inter_pad,
                                   block_m, l.n_blk, activation, swiglu_limit, stream);
        if(rc)
            return rc;
        rc = pyhip_moe_gemm2_mxfp4(ws + l.a2_q, ws + l.a2_s, w2, w2_scale, bias2_bf16, s_ids, s_w, s_e, n_valid, sched,
                                   out3, tokens, topk, experts, hidden, inter, hidden_pad, inter_pad, block_m, l.n_blk, stream);
    }
    if(rc)
        return rc;
    // Slots the sort dropped (ids outside [0, experts), experts this rank does not hold, tokens past the local count)
    // were never written by the down GEMM: the reduction reads the routing and leaves them out, so out3 needs no
    // clearing and the traffic under expert parallelism is that of the owned slots.
    return pyhip_moe_topk_reduce_routed(out3, out, tokens, topk, hidden, out_is_f32, topk_ids, experts, expert_mask,
                                        num_local_tokens, stream);
}

extern "C" int pyhip_moe_forward(const void* hidden_bf16, int64_t hidden_row_stride, const uint8_t* w1,
                                 const uint8_t* w1_scale, const uint8_t* w2, const uint8_t* w2_scale,
                                 const void* bias1_bf16, const void* bias2_bf16, const int32_t* topk_ids,
                                 const float* topk_weights, const int32_t* expert_mask,
                                 const int32_t* num_local_tokens, void* out, int out_is_f32, int tokens, int topk,
                                 int experts, int hidden, int inter, int hidden_pad, int inter_pad, int block_m,
                                 int w4a16, int split_k, int activation, float swiglu_limit, void* workspace,
                                 int64_t workspace_bytes, hipStream_t stream)
{
    return forward_impl(hidden_bf16, hidden_row_stride, w1, w1_scale, w2, w2_scale, bias1_bf16, bias2_bf16, Router{},
                        const_cast<int32_t*>(topk_ids), const_cast<float*>(topk_weights), expert_mask, num_local_tokens,
                        out, out_is_f32, tokens, topk, experts, hidden, inter, hidden_pad, inter_pad, block_m, w4a16,
                        split_k, activation, swiglu_limit, workspace, workspace_bytes, stream);
}

// The layer with its router: gating scores in, and the picks (topk_ids, topk_weights) out next to the layer output.
// n_group = 0: softmax over the experts, top-k; n_group > 0: sigmoid scores with grouped selection (DeepSeek-V3).
extern "C" int pyhip_moe_forward_routed(const void* hidden_bf16, int64_t hidden_row_stride, const uint8_t* w1,
                                        const uint8_t* w1_scale, const uint8_t* w2, const uint8_t* w2_scale,
                                        const void* bias1_bf16, const void* bias2_bf16, const float* gating, int n_group,
                                        int topk_group, int renormalize, int32_t* topk_ids, float* topk_weights,
                                        const int32_t* expert_mask, const int32_t* num_local_tokens, void* out,
                                        int out_is_f32, int tokens, int topk, int experts, int hidden, int inter,
                                        int hidden_pad, int inter_pad, int block_m, int w4a16, int split_k,
                                        int activation, float swiglu_limit, void* workspace, int64_t workspace_bytes,
                                        hipStream_t stream)
{
    PYHIP_REQUIRE(gating, "moe_forward_routed: null gating scores");
    Router r;
    r.gating = gating; r.n_group = n_group; r.topk_group = topk_group; r.renormalize = renormalize;
    return forward_impl(hidden_bf16, hidden_row_stride, w1, w1_scale, w2, w2_scale, bias1_bf16, bias2_bf16, r, topk_ids,
                        topk_weights, expert_mask, num_local_tokens, out, out_is_f32, tokens, topk, experts, hidden, inter,
                        hidden_pad, inter_pad, block_m, w4a16, split_k, activation, swiglu_limit, workspace, workspace_bytes,
                        stream);
}
