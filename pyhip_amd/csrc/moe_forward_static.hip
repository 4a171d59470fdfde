// The whole layer in one call that allocates nothing: pyhip_moe_forward with its workspace in a device array that
// belongs to the library.
#include "common.h"
#include <mutex>

extern "C" {
int64_t pyhip_moe_forward_workspace_bytes(int64_t tokens, int topk, int experts, int hidden, int inter, int block_m,
                                          int w4a16);
int pyhip_moe_forward(const void*, int64_t, const uint8_t*, const uint8_t*, const uint8_t*, const uint8_t*, const void*,
                      const void*, const int32_t*, const float*, const int32_t*, const int32_t*, void*, int, int, int, int,
                      int, int, int, int, int, int, int, int, float, void*, int64_t, hipStream_t);
}

// The same layer for callers that cannot allocate device memory (code under HIP graph capture, tight serving
// loops, harnesses that forbid hipMalloc): the workspace is a file-scope device array, one copy per GPU, held until
// the process ends.  64 MiB cover the decode-sized calls such callers make (DeepSeek-V3 shape up to 128 tokens
// with bf16 activations needs 35 MiB); larger calls are rejected.  Calls that overlap on one GPU share the array
// and race; every buffer inside it is fully written before it is read, so nothing has to be cleared between calls.
#define PYHIP_STATIC_SCRATCH_BYTES (64ll << 20)
static __device__ __align__(256) unsigned char scratch[PYHIP_STATIC_SCRATCH_BYTES];

// `scratch` names a host-side stand-in; the array's device address is asked for once per device, with that device
// current, and only that address is ever handed to kernels.  Asking is what makes the runtime map the array on that
// device, so it must not happen for the first time inside a stream capture: pyhip_moe_forward_static_capacity() asks
// for the current device's address too, and is what a caller runs once per device while setting up.
static void* scratch_device_ptr(int* rc_out)
{
    static void* ptrs[64] = {nullptr};
    static std::mutex mu;
    *rc_out = PYHIP_OK;
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if(e != hipSuccess || dev < 0 || dev >= 64)
    {
        pyhip_set_error("moe_forward_static: hipGetDevice: %s (device %d)", hipGetErrorString(e), dev);
        *rc_out = PYHIP_ERR_HIP;
        return nullptr;
    }
    std::lock_guard<std::mutex> lock(mu);
    if(!ptrs[dev])
    {
        void* p = nullptr;
        e       = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if(e != hipSuccess || !p)
        {
            pyhip_set_error("moe_forward_static: hipGetSymbolAddress: %s", hipGetErrorString(e));
            *rc_out = PYHIP_ERR_HIP;
            return nullptr;
        }
        ptrs[dev] = p;
    }
    return ptrs[dev];
}

extern "C" int64_t pyhip_moe_forward_static_capacity(void)
{
    int rc;
    scratch_device_ptr(&rc);        // set-up for the current device; a failure is reported by the first real call
    return PYHIP_STATIC_SCRATCH_BYTES;
}

extern "C" int pyhip_moe_forward_static(const void* hidden_bf16, int64_t hidden_row_stride, const uint8_t* w1,
                                        const uint8_t* w1_scale, const uint8_t* w2, const uint8_t* w2_scale,
                                        const void* bias1_bf16, const void* bias2_bf16, const int32_t* topk_ids,
                                        const float* topk_weights, const int32_t* expert_mask,
                                        const int32_t* num_local_tokens, void* out, int out_is_f32, int tokens,
                                        int topk, int experts, int hidden, int inter, int hidden_pad, int inter_pad,
                                        int block_m, int w4a16, int split_k, int activation, float swiglu_limit,
                                        hipStream_t stream)
{
    PYHIP_REQUIRE(tokens > 0 && topk > 0 && experts > 0 && hidden > 0 && inter > 0 && block_m > 0,
                  "moe_forward_static: bad sizes");
    const int64_t need = pyhip_moe_forward_workspace_bytes(tokens, topk, experts, hidden, inter, block_m, w4a16);
    PYHIP_REQUIRE(need <= PYHIP_STATIC_SCRATCH_BYTES,
                  "moe_forward_static: this call needs %lld bytes of intermediates, the built-in scratch array holds "
                  "%lld; use pyhip_moe_forward with a workspace of your own",
                  (long long)need, (long long)PYHIP_STATIC_SCRATCH_BYTES);
    int rc;
    void* ws = scratch_device_ptr(&rc);
    if(rc)
        return rc;
    return pyhip_moe_forward(hidden_bf16, hidden_row_stride, w1, w1_scale, w2, w2_scale, bias1_bf16, bias2_bf16, topk_ids,
                             topk_weights, expert_mask, num_local_tokens, out, out_is_f32, tokens, topk, experts, hidden,
                             inter, hidden_pad, inter_pad, block_m, w4a16, split_k, activation, swiglu_limit, ws,
                             PYHIP_STATIC_SCRATCH_BYTES, stream);
}
