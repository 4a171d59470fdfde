// Routers: gating scores -> (topk_weight f32 [T, k], topk_ids i32 [T, k]), the inputs of the routing sort.
// The arithmetic is in router_device.h; these kernels give every token a wave of its own.
#include "router_device.h"

#define ROUTER_THREADS 256

template <int NE, bool GROUPED>
__global__ void __launch_bounds__(ROUTER_THREADS)
    moe_router_kernel(const float* __restrict__ logits, int T, int E, int k, int n_group, int topk_group, int renorm,
                      float* __restrict__ out_w, int* __restrict__ out_ids)
{
    const int lane = lane_id();
    const int t    = blockIdx.x * (ROUTER_THREADS / WAVE) + threadIdx.x / WAVE;
    if(t >= T)
        return;
    float w;
    int id;
    route_token<NE, GROUPED>(logits + (size_t)t * E, lane, k, n_group, topk_group, renorm, w, id);
    if(lane < k)
    {
        out_w[(size_t)t * k + lane]   = w;
        out_ids[(size_t)t * k + lane] = id;
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

int pyhip_check_router(const char* name, const void* logits, const void* w, const void* ids, int tokens, int experts,
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
    int rc = pyhip_check_router("topk_softmax", gating, topk_weight, topk_ids, tokens, experts, topk);
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
    int rc = pyhip_check_router("topk_grouped_sigmoid", gating, topk_weight, topk_ids, tokens, experts, topk);
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
