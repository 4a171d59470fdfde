// Routers: gating scores -> (topk_weight f32 [T, k], topk_ids i32 [T, k]), the inputs of the routing sort.
//   softmax -> top-k -> renormalise           (aiter.fused_topk as called at tests/contrib/moe/test_fused_moe.py:38,87)
//   sigmoid -> groups ranked by the sum of their two best scores -> top-k inside the best groups -> renormalise
//                                             (DeepSeek-V3 routing; not in the reference, part of the benchmark definition)
// Ties go to the lower expert (group) index, as a stable descending sort does.
//
// One wave per token.  Lane l holds the NE = E/64 consecutive experts l*NE .. l*NE+NE-1 in registers, so an expert
// group (E / n_group consecutive experts) is a run of consecutive lanes.  Selection is k rounds of
// (per-lane best, wave arg-max); with k <= 32 and NE <= 32 that is a few hundred instructions per token.
#include "common.h"
#include <math.h>

#define ROUTER_THREADS 256

// wave arg-max of (v, idx): larger v wins, equal v -> smaller idx.  Result in every lane.
__device__ __forceinline__ void wave_argmax(float& v, int& idx)
{
#pragma unroll
    for(int d = 1; d < WAVE; d <<= 1)
    {
        const float ov = __shfl_xor(v, d);
        const int oi   = __shfl_xor(idx, d);
        if(ov > v || (ov == v && oi < idx))
        {
            v   = ov;
            idx = oi;
        }
    }
}
__device__ __forceinline__ float wave_sum(float v)
{
#pragma unroll
    for(int d = 1; d < WAVE; d <<= 1)
        v += __shfl_xor(v, d);
    return v;
}
__device__ __forceinline__ float wave_max(float v)
{
#pragma unroll
    for(int d = 1; d < WAVE; d <<= 1)
        v = fmaxf(v, __shfl_xor(v, d));
    return v;
}

// k rounds of arg-max over s[] (entries taken are set to -inf); lane j (< k) keeps the j-th pick
template <int NE>
__device__ __forceinline__ void select_topk(float (&s)[NE], int lane, int k, float& my_w, int& my_id)
{
    for(int j = 0; j < k; j++)
    {
        float bv = -INFINITY;
        int bi   = 0x7FFFFFFF;
#pragma unroll
        for(int i = 0; i < NE; i++)
            if(s[i] > bv)          // strict: the first (lowest index) of equal values stays
            {
                bv = s[i];
                bi = lane * NE + i;
            }
        wave_argmax(bv, bi);
        if(lane == j)
        {
            my_w  = bv;
            my_id = bi;
        }
        if(bi / NE == lane)
        {
#pragma unroll
            for(int i = 0; i < NE; i++)
                if(i == bi - lane * NE)
                    s[i] = -INFINITY;
        }
    }
}

template <int NE, bool GROUPED>
__global__ void __launch_bounds__(ROUTER_THREADS)
    moe_router_kernel(const float* __restrict__ logits, int T, int E, int k, int n_group, int topk_group, int renorm,
                      float* __restrict__ out_w, int* __restrict__ out_ids)
{
    const int lane = lane_id();
    const int t    = blockIdx.x * (ROUTER_THREADS / WAVE) + threadIdx.x / WAVE;
    if(t >= T)
        return;
    float s[NE];
#pragma unroll
    for(int i = 0; i < NE; i++)
        s[i] = logits[(size_t)t * E + lane * NE + i];
    if(!GROUPED)
    {
        float m = s[0];
#pragma unroll
        for(int i = 1; i < NE; i++)
            m = fmaxf(m, s[i]);
        m         = wave_max(m);
        float sum = 0.f;
#pragma unroll
        for(int i = 0; i < NE; i++)
        {
            s[i] = expf(s[i] - m);
            sum += s[i];
        }
        sum = wave_sum(sum);
        const float inv = 1.0f / sum;
#pragma unroll
        for(int i = 0; i < NE; i++)
            s[i] *= inv;
    }
    else
    {
#pragma unroll
        for(int i = 0; i < NE; i++)
            s[i] = 1.0f / (1.0f + expf(-s[i]));
        // best two scores of this lane, then of its group (a run of lanes_per_group consecutive lanes)
        float a1 = -INFINITY, a2 = -INFINITY;
#pragma unroll
        for(int i = 0; i < NE; i++)
        {
            if(s[i] > a1)
            {
                a2 = a1;
                a1 = s[i];
            }
            else if(s[i] > a2)
                a2 = s[i];
        }
        const int lanes_per_group = WAVE / n_group;
        for(int d = 1; d < lanes_per_group; d <<= 1)
        {
            const float b1 = __shfl_xor(a1, d), b2 = __shfl_xor(a2, d);
            const float hi = fmaxf(a1, b1);
            a2             = fmaxf(fminf(a1, b1), fmaxf(a2, b2));
            a1             = hi;
        }
        const float gscore = a1 + a2;
        const int group    = lane / lanes_per_group;
        // choose topk_group groups: rounds of arg-max over (group score, group index)
        bool chosen = false;
        float gs    = gscore;
        for(int j = 0; j < topk_group; j++)
        {
            float bv = gs;
            int bi   = group;
            wave_argmax(bv, bi);
            if(bi == group)
            {
                chosen = true;
                gs     = -INFINITY;
            }
        }
        if(!chosen)
        {
#pragma unroll
            for(int i = 0; i < NE; i++)
                s[i] = -INFINITY;
        }
    }
    // keep the unmasked scores of this lane for the weights (selection overwrites s)
    float my_w = 0.f;
    int my_id  = 0;
    select_topk<NE>(s, lane, k, my_w, my_id);
    float wsum = wave_sum(lane < k ? my_w : 0.f);
    if(lane < k)
    {
        out_w[(size_t)t * k + lane]   = renorm ? my_w / wsum : my_w;
        out_ids[(size_t)t * k + lane] = my_id;
    }
}

template <bool GROUPED>
static int launch_router(int ne, dim3 grid, hipStream_t stream, const float* logits, int T, int E, int k, int n_group,
                         int topk_group, int renorm, float* w, int* ids)
{
#define ROUTER_CASE(N)                                                                                             \
    case N:                                                                                                        \
        hipLaunchKernelGGL((moe_router_kernel<N, GROUPED>), grid, dim3(ROUTER_THREADS), 0, stream, logits, T, E, k, \
                           n_group, topk_group, renorm, w, ids);                                                   \
        break;
    switch(ne)
    {
        ROUTER_CASE(1) ROUTER_CASE(2) ROUTER_CASE(4) ROUTER_CASE(8) ROUTER_CASE(16) ROUTER_CASE(32)
    default: pyhip_set_error("moe_router: experts/64 = %d not in {1,2,4,8,16,32}", ne); return PYHIP_ERR_INVALID;
    }
#undef ROUTER_CASE
    PYHIP_CHECK_LAUNCH("moe_router_kernel");
    return PYHIP_OK;
}

static int check_router(const char* name, const void* logits, const void* w, const void* ids, int tokens, int experts,
                        int topk)
{
    PYHIP_REQUIRE(logits && w && ids, "%s: null pointer", name);
    PYHIP_REQUIRE(tokens >= 0, "%s: tokens=%d", name, tokens);
    PYHIP_REQUIRE(experts >= 64 && experts <= 2048 && experts % 64 == 0,
                  "%s: experts=%d must be a multiple of 64 in [64, 2048]", name, experts);
    PYHIP_REQUIRE(topk >= 1 && topk <= 64 && topk <= experts, "%s: topk=%d outside [1, min(64, experts)]", name, topk);
    return PYHIP_OK;
}

extern "C" int pyhip_moe_topk_softmax(const float* gating, int tokens, int experts, int topk, int renormalize,
                                      float* topk_weight, int32_t* topk_ids, hipStream_t stream)
{
    int rc = check_router("topk_softmax", gating, topk_weight, topk_ids, tokens, experts, topk);
    if(rc || tokens == 0)
        return rc;
    dim3 grid((unsigned)((tokens + ROUTER_THREADS / WAVE - 1) / (ROUTER_THREADS / WAVE)));
    return launch_router<false>(experts / 64, grid, stream, gating, tokens, experts, topk, 1, 1, renormalize, topk_weight,
                                topk_ids);
}

extern "C" int pyhip_moe_topk_grouped_sigmoid(const float* gating, int tokens, int experts, int topk, int n_group,
                                              int topk_group, int renormalize, float* topk_weight, int32_t* topk_ids,
                                              hipStream_t stream)
{
    int rc = check_router("topk_grouped_sigmoid", gating, topk_weight, topk_ids, tokens, experts, topk);
    if(rc)
        return rc;
    PYHIP_REQUIRE(n_group >= 1 && n_group <= 64 && (n_group & (n_group - 1)) == 0 && experts % n_group == 0,
                  "topk_grouped_sigmoid: n_group=%d must be a power of two <= 64 dividing experts", n_group);
    PYHIP_REQUIRE(topk_group >= 1 && topk_group <= n_group, "topk_grouped_sigmoid: topk_group=%d", topk_group);
    PYHIP_REQUIRE(topk <= topk_group * (experts / n_group), "topk_grouped_sigmoid: topk=%d exceeds the chosen groups",
                  topk);
    if(tokens == 0)
        return PYHIP_OK;
    dim3 grid((unsigned)((tokens + ROUTER_THREADS / WAVE - 1) / (ROUTER_THREADS / WAVE)));
    return launch_router<true>(experts / 64, grid, stream, gating, tokens, experts, topk, n_group, topk_group,
                               renormalize, topk_weight, topk_ids);
}
