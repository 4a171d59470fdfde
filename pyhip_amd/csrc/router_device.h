// Device part of the routers, shared by the stand-alone router kernels (moe_router.hip) and by the routing sort
// that routes its tokens itself (moe_sort.hip).
//   softmax -> top-k -> renormalise           (aiter.fused_topk as called at tests/contrib/moe/test_fused_moe.py:38,87)
//   sigmoid -> groups ranked by the sum of their two best scores -> top-k inside the best groups -> renormalise
//                                             (DeepSeek-V3 routing; not in the reference, part of the benchmark definition)
// Ties go to the lower expert (group) index, as a stable descending sort does.
//
// One wave per token.  Lane l holds the NE = E/64 consecutive experts l*NE .. l*NE+NE-1 in registers, so an expert
// group (E / n_group consecutive experts) is a run of consecutive lanes.  Selection is k rounds of
// (per-lane best, wave arg-max); with k <= 32 and NE <= 32 that is a few hundred instructions per token.
#pragma once
#include "common.h"
#include <math.h>


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


// Routes one token with one wave: row = its E = 64*NE gating scores.  Lane j (< k) returns the j-th pick (descending
// score) in (w, id), the weight renormalised over the k picks when renorm != 0.
template <int NE, bool GROUPED>
__device__ __forceinline__ void route_token(const float* __restrict__ row, int lane, int k, int n_group, int topk_group,
                                            int renorm, float& w, int& id)
{
    float s[NE];
#pragma unroll
    for(int i = 0; i < NE; i++)
        s[i] = row[lane * NE + i];
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
    const float wsum = wave_sum(lane < k ? my_w : 0.f);
    w  = renorm ? my_w / wsum : my_w;
    id = my_id;
}
