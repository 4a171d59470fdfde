// Top-k reduction of the down-projection output: out[t, :] = sum over slots of in[t, slot, :],
// slots added in index order in fp32, one rounding to the output type at the end
// (what the reference's moe_gemm_final_reduce_bf16 computes, src/contrib/moe_gemm_mxfp4.py:199-282).
//
// ROUTED: the kernel also sees the routing (top-k ids, expert count, expert mask, local token count) and leaves
// out every slot that the sort dropped (id outside [0, experts), masked expert): the down GEMM never wrote those
// slots, so they are neither read nor need to be cleared beforehand.  Rows of tokens past the local count are
// written as zeros.
#include "common.h"

struct ReduceRouting
{
    const int* topk_ids;       // [T, k]
    const int* expert_mask;    // [experts] or null
    const int* num_local_tok;  // device scalar or null
    int experts;
};

template <bool OUT_F32, bool ROUTED>
__global__ void __launch_bounds__(256)
    moe_topk_reduce_kernel(const uint4* __restrict__ in, void* __restrict__ out, long long T, int k, int H8,
                           const u32* __restrict__ tokens_limit, ReduceRouting rt)
{
    if(tokens_limit)
    {
        long long lim = (long long)tokens_limit[1];
        T             = T < lim ? T : lim;
    }
    long long T_local = T;
    if(ROUTED && rt.num_local_tok)
    {
        const long long lim = (long long)*rt.num_local_tok;
        T_local             = lim < 0 ? 0 : (lim < T ? lim : T);
    }
    const long long total = T * H8;
    for(long long id = (long long)blockIdx.x * 256 + threadIdx.x; id < total; id += (long long)gridDim.x * 256)
    {
        const long long t = id / H8;
        const int c       = (int)(id - t * H8);
        float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
        const uint4* p = in + (t * k) * H8 + c;
        for(int s0 = 0; s0 < k; s0 += 8)         // up to 8 independent loads in flight, added in slot order
        {
            v4i v[8];
            bool on[8];
#pragma unroll
            for(int j = 0; j < 8; j++)
            {
                on[j] = s0 + j < k;
                if(ROUTED && on[j])
                {
                    const int e = t < T_local ? rt.topk_ids[t * k + s0 + j] : -1;
                    on[j]       = moe_pair_is_kept(e, rt.experts, rt.expert_mask);
                }
            }
#pragma unroll
            for(int j = 0; j < 8; j++)
                v[j] = on[j] ? __builtin_nontemporal_load((const v4i*)(p + (long long)(s0 + j) * H8)) : (v4i){0, 0, 0, 0};
#pragma unroll
            for(int j = 0; j < 8; j++)
            {
                // (a slot that is left out adds +0.0, which leaves every value, including -0.0 sums, unchanged)
                acc[0] += bf16_bits_to_f32((u32)v[j][0] & 0xFFFFu); acc[1] += bf16_bits_to_f32((u32)v[j][0] >> 16);
                acc[2] += bf16_bits_to_f32((u32)v[j][1] & 0xFFFFu); acc[3] += bf16_bits_to_f32((u32)v[j][1] >> 16);
                acc[4] += bf16_bits_to_f32((u32)v[j][2] & 0xFFFFu); acc[5] += bf16_bits_to_f32((u32)v[j][2] >> 16);
                acc[6] += bf16_bits_to_f32((u32)v[j][3] & 0xFFFFu); acc[7] += bf16_bits_to_f32((u32)v[j][3] >> 16);
            }
        }
        if(OUT_F32)
        {
            float4* o = (float4*)out + id * 2;
            o[0]      = make_float4(acc[0], acc[1], acc[2], acc[3]);
            o[1]      = make_float4(acc[4], acc[5], acc[6], acc[7]);
        }
        else
        {
            uint4 o;
            o.x = pack_bf16x2(acc[0], acc[1]);
            o.y = pack_bf16x2(acc[2], acc[3]);
            o.z = pack_bf16x2(acc[4], acc[5]);
            o.w = pack_bf16x2(acc[6], acc[7]);
            ((uint4*)out)[id] = o;
        }
    }
}

static int launch_reduce(const char* name, const void* in_bf16, void* out, int64_t tokens, int topk, int hidden,
                         int out_is_f32, const uint32_t* num_valid_ids, const ReduceRouting* rt, hipStream_t stream)
{
    PYHIP_REQUIRE(in_bf16 && out, "%s: null pointer", name);
    PYHIP_REQUIRE(hidden > 0 && hidden % 8 == 0, "%s: hidden=%d must be a multiple of 8", name, hidden);
    PYHIP_REQUIRE(topk >= 1, "%s: topk=%d", name, topk);
    PYHIP_REQUIRE(((uintptr_t)in_bf16 % 16) == 0 && ((uintptr_t)out % 16) == 0, "%s: unaligned pointer", name);
    if(tokens <= 0)
        return PYHIP_OK;
    long long total = (long long)tokens * (hidden / 8);
    long long grid  = (total + 255) / 256;
    grid            = grid > 8192 ? 8192 : grid;
    const ReduceRouting none = {nullptr, nullptr, nullptr, 0};
#define REDUCE_LAUNCH(F32, ROUTED)                                                                                  \
    hipLaunchKernelGGL((moe_topk_reduce_kernel<F32, ROUTED>), dim3((unsigned)grid), dim3(256), 0, stream,           \
                       (const uint4*)in_bf16, out, (long long)tokens, topk, hidden / 8, num_valid_ids, rt ? *rt : none)
    if(rt)
    {
        if(out_is_f32)
            REDUCE_LAUNCH(true, true);
        else
            REDUCE_LAUNCH(false, true);
    }
    else
    {
        if(out_is_f32)
            REDUCE_LAUNCH(true, false);
        else
            REDUCE_LAUNCH(false, false);
    }
#undef REDUCE_LAUNCH
    PYHIP_CHECK_LAUNCH("moe_topk_reduce_kernel");
    return PYHIP_OK;
}

extern "C" int pyhip_moe_topk_reduce(const void* in_bf16, void* out, int64_t tokens, int topk, int hidden,
                                     int out_is_f32, const uint32_t* num_valid_ids, hipStream_t stream)
{
    return launch_reduce("topk_reduce", in_bf16, out, tokens, topk, hidden, out_is_f32, num_valid_ids, nullptr, stream);
}

extern "C" int pyhip_moe_topk_reduce_routed(const void* in_bf16, void* out, int64_t tokens, int topk, int hidden,
                                            int out_is_f32, const int32_t* topk_ids, int experts,
                                            const int32_t* expert_mask, const int32_t* num_local_tokens,
                                            hipStream_t stream)
{
    PYHIP_REQUIRE(topk_ids && experts > 0, "topk_reduce_routed: topk_ids and the expert count are needed");
    const ReduceRouting rt = {topk_ids, expert_mask, num_local_tokens, experts};
    return launch_reduce("topk_reduce_routed", in_bf16, out, tokens, topk, hidden, out_is_f32, nullptr, &rt, stream);
}
