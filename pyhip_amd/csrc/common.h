// Shared device/host helpers for the MXFP4 fused-MoE kernels (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <utility>
#include <type_traits>

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v2f __attribute__((ext_vector_type(2)));
typedef __bf16 v2bf __attribute__((ext_vector_type(2)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef unsigned int u32;
typedef unsigned long long u64;

#define PYHIP_OK 0
#define PYHIP_ERR_INVALID 1   // argument check failed (message in pyhip_moe_last_error)
#define PYHIP_ERR_HIP 2       // a HIP runtime call failed (message in pyhip_moe_last_error)

#define WAVE 64

// error plumbing shared by every translation unit of the library (defined in capi.hip)
extern "C" void pyhip_set_error(const char* fmt, ...);

#define PYHIP_REQUIRE(cond, ...)                 \
    do {                                         \
        if(!(cond)) {                            \
            pyhip_set_error(__VA_ARGS__);        \
            return PYHIP_ERR_INVALID;            \
        }                                        \
    } while(0)

#define PYHIP_CHECK_LAUNCH(name)                                                  \
    do {                                                                          \
        hipError_t e_ = hipGetLastError();                                        \
        if(e_ != hipSuccess) {                                                    \
            pyhip_set_error("%s: launch failed: %s", name, hipGetErrorString(e_)); \
            return PYHIP_ERR_HIP;                                                 \
        }                                                                         \
    } while(0)

// Which (token, slot) pairs take part in the layer: the expert id names an expert (0 <= e < experts) that the
// expert mask, when there is one, does not switch off.  The routing sort drops every other pair, the down GEMMs
// then never write that pair's slot of out3, and the routing-aware top-k reduction leaves the slot out: all three
// by this one rule.  (Tokens past num_local_tokens are dropped as whole rows by the callers' token limits.)
__device__ __forceinline__ bool moe_pair_is_kept(int e, int experts, const int* expert_mask)
{
    return e >= 0 && e < experts && (!expert_mask || expert_mask[e] != 0);
}

__device__ __forceinline__ u32 pack_bf16x2(float a, float b)
{
    v2f v = {a, b};
    v2bf r = __builtin_convertvector(v, v2bf);   // v_cvt_pk_bf16_f32: round to nearest even
    return __builtin_bit_cast(u32, r);
}

__device__ __forceinline__ float bf16_bits_to_f32(u32 hi16) { return __builtin_bit_cast(float, hi16 << 16); }

// silu(x) = x / (1 + 2^(-x*log2 e)) with the hardware exp2 / rcp approximations
__device__ __forceinline__ float silu_f32(float x)
{
    float e = __builtin_amdgcn_exp2f(-1.4426950408889634f * x);
    return x * __builtin_amdgcn_rcpf(1.0f + e);
}

// gpt-oss's gated activation (tests/contrib/moe/test_moe.py:76-81): the gate is clamped from above, the up
// projection from both sides, out = gate * sigmoid(1.702 * gate) * (up + 1); same hardware approximations
__device__ __forceinline__ float swiglu_f32(float gate, float up, float limit)
{
    gate    = fminf(gate, limit);
    up      = fminf(fmaxf(up, -limit), limit);
    float e = __builtin_amdgcn_exp2f(-1.702f * 1.4426950408889634f * gate);
    return gate * __builtin_amdgcn_rcpf(1.0f + e) * (up + 1.0f);
}

// The gated activation of the gate_up GEMMs in one branch-free form,
//     g' * sigmoid(alpha * g') * (u' + beta),   g' = min(gate, limit),  u' = clamp(up, -limit, limit):
// SiLU(gate) * up is alpha = 1, beta = 0, limit = +inf (the clamps then change nothing); gpt-oss's clamped SwiGLU
// (tests/contrib/moe/test_moe.py:76-81) is alpha = 1.702, beta = 1 and its limit.  Same hardware approximations
// as silu_f32.  Used by the bf16-activation GEMM; the MXFP4 GEMM is instantiated per activation instead (the extra
// four instructions per element showed in its time, and a branch between two forms in its epilogue costs registers
// the 128-row tile does not have).
struct GatedAct
{
    float neg_alpha_log2e, beta, limit;
};
__device__ __host__ __forceinline__ GatedAct make_gated_act(int activation, float swiglu_limit)
{
    GatedAct a;
    a.neg_alpha_log2e = -1.4426950408889634f * (activation ? 1.702f : 1.0f);
    a.beta            = activation ? 1.0f : 0.0f;
    a.limit           = activation ? swiglu_limit : __builtin_inff();
    return a;
}
__device__ __forceinline__ float gated_act_f32(const GatedAct& a, float gate, float up)
{
    gate    = fminf(gate, a.limit);
    up      = fminf(fmaxf(up, -a.limit), a.limit);
    float e = __builtin_amdgcn_exp2f(a.neg_alpha_log2e * gate);
    return gate * __builtin_amdgcn_rcpf(1.0f + e) * (up + a.beta);
}

// ---- MXFP4 quantisation of bf16 values (shared by the quantisation kernel and the stage-1 GEMM epilogue)
// running maximum of the magnitudes (15-bit patterns) of the two bf16 halves of w
__device__ __forceinline__ u32 amax15(u32 acc, u32 w)
{
    u32 lo = w & 0x7FFFu, hi = (w >> 16) & 0x7FFFu;
    acc    = acc > lo ? acc : lo;
    return acc > hi ? acc : hi;
}

// the same on packed halves: per 16-bit half, the larger magnitude pattern of a and b; amax15_fold joins the halves
__device__ __forceinline__ u32 amax15x2(u32 a, u32 b)
{
    typedef unsigned short v2us __attribute__((ext_vector_type(2)));
    const v2us x = __builtin_bit_cast(v2us, a & 0x7FFF7FFFu), y = __builtin_bit_cast(v2us, b & 0x7FFF7FFFu);
    return __builtin_bit_cast(u32, __builtin_elementwise_max(x, y));      // v_pk_max_u16
}
__device__ __forceinline__ u32 amax15_fold(u32 w)
{
    const u32 lo = w & 0xFFFFu, hi = w >> 16;
    return lo > hi ? lo : hi;
}

// eight bf16 (one uint4) times a power of two -> eight e2m1 codes in one dword
__device__ __forceinline__ u32 cvt8(uint4 v, float mul)
{
    u32 r = 0;
    r = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(r, bf16_bits_to_f32(v.x & 0xFFFFu) * mul,
                                                 bf16_bits_to_f32(v.x >> 16) * mul, 1.0f, 0);
    r = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(r, bf16_bits_to_f32(v.y & 0xFFFFu) * mul,
                                                 bf16_bits_to_f32(v.y >> 16) * mul, 1.0f, 1);
    r = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(r, bf16_bits_to_f32(v.z & 0xFFFFu) * mul,
                                                 bf16_bits_to_f32(v.z >> 16) * mul, 1.0f, 2);
    r = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(r, bf16_bits_to_f32(v.w & 0xFFFFu) * mul,
                                                 bf16_bits_to_f32(v.w >> 16) * mul, 1.0f, 3);
    return r;
}

// e8m0 scale byte of a block whose largest bf16 magnitude pattern is am: 2^(floor(log2 amax) - 2), byte 0 for amax < 2^-124
__device__ __forceinline__ u32 mx_scale_byte(u32 am)
{
    int ex = (int)(am >> 7);                             // biased exponent of amax (bf16: 8 exponent bits)
    u32 e8 = (u32)(ex > 2 ? ex - 2 : 0);
    return e8 > 254u ? 254u : e8;
}
// x / 2^(e8-127) = x * 2^(127-e8): exponent field 254-e8 is in [1, 254], always a normal float
__device__ __forceinline__ float mx_inv_scale(u32 e8) { return __builtin_bit_cast(float, (254u - e8) << 23); }

__device__ __forceinline__ int lane_id() { return threadIdx.x & (WAVE - 1); }

// compile-time loop: f(std::integral_constant<int, 0>{}), ..., f(std::integral_constant<int, N-1>{})
template <typename F, int... Is>
__device__ __forceinline__ __attribute__((always_inline)) void static_for_impl(F&& f, std::integer_sequence<int, Is...>)
{
    (f(std::integral_constant<int, Is>{}), ...);
}
template <int N, typename F>
__device__ __forceinline__ void static_for(F&& f)
{
    static_for_impl(f, std::make_integer_sequence<int, N>{});
}
