// Dynamic MXFP4 quantisation of bf16 activations: one e8m0 scale per 32 elements,
// scale = 2^(floor(log2(amax)) - 2), values rounded to nearest-even e2m1, saturating at 6.
// (The reference gets this step from aiter.get_hip_quant(QuantType.per_1x32):
//  tests/contrib/moe/test_moe.py:664-679,732-744.)
//
// Output layout (internal to this library, consumed by the grouped GEMM):
//   q  [rows, K/2]  row-major, low nibble = even element
//   s  [rows, SK]   SK = ceil(K/512)*16 bytes.  Inside every 16-byte group (16 consecutive
//                   32-element blocks = 4 MFMA K-steps of 128) the bytes are stored transposed:
//                   byte (kb*4 + i) holds the scale of block (4*i + kb).  The MFMA lane that owns
//                   K-block kb of a row then reads ONE dword (offset kb*4) and selects the byte of
//                   K-step i with the instruction's op_sel.
#include "common.h"

#define QUANT_THREADS 256

// one thread per 32-element block; 16 consecutive threads own one 16-byte scale group
extern "C" __global__ void __launch_bounds__(QUANT_THREADS)
    moe_act_quant_mxfp4_kernel(const uint16_t* __restrict__ x, long long ldx, uint8_t* __restrict__ q,
                               uint8_t* __restrict__ s, long long rows, int K, int SK,
                               const u32* __restrict__ rows_limit)
{
    if(rows_limit)
    {
        long long lim = (long long)*rows_limit;
        rows          = rows < lim ? rows : lim;
    }
    const long long id = (long long)blockIdx.x * QUANT_THREADS + threadIdx.x;
    const long long row = id / SK;
    const int j         = (int)(id - row * SK);          // block index inside the row (may be padding)
    if(row >= rows)                                      // whole 16-thread groups leave together
        return;
    u32 e8 = 0;
    if(j * 32 < K)
    {
        const uint4* src = (const uint4*)(x + row * ldx + (long long)j * 32);
        uint4 v0 = src[0], v1 = src[1], v2 = src[2], v3 = src[3];
        u32 am = 0;
        am = amax15(am, v0.x); am = amax15(am, v0.y); am = amax15(am, v0.z); am = amax15(am, v0.w);
        am = amax15(am, v1.x); am = amax15(am, v1.y); am = amax15(am, v1.z); am = amax15(am, v1.w);
        am = amax15(am, v2.x); am = amax15(am, v2.y); am = amax15(am, v2.z); am = amax15(am, v2.w);
        am = amax15(am, v3.x); am = amax15(am, v3.y); am = amax15(am, v3.z); am = amax15(am, v3.w);
        e8        = mx_scale_byte(am);
        float mul = mx_inv_scale(e8);
        uint4 o;
        o.x = cvt8(v0, mul);
        o.y = cvt8(v1, mul);
        o.z = cvt8(v2, mul);
        o.w = cvt8(v3, mul);
        *(uint4*)(q + row * (long long)(K / 2) + (long long)j * 16) = o;
    }
    // 4x4 byte transpose of the 16 scales of this group through lane shuffles
    const int jj = j & 15;
    u32 b0 = __shfl(e8, 0 + (jj & 3), 16), b1 = __shfl(e8, 4 + (jj & 3), 16);
    u32 b2 = __shfl(e8, 8 + (jj & 3), 16), b3 = __shfl(e8, 12 + (jj & 3), 16);
    if(jj < 4)
        *(u32*)(s + row * (long long)SK + (j & ~15) + jj * 4) = b0 | (b1 << 8) | (b2 << 16) | (b3 << 24);
}

extern "C" int64_t pyhip_moe_act_scale_stride(int K) { return ((int64_t)K + 511) / 512 * 16; }

extern "C" int pyhip_moe_act_quant_mxfp4(const void* x_bf16, int64_t row_stride_elems, int64_t rows, int K,
                                         uint8_t* q, uint8_t* scales, const uint32_t* rows_limit,
                                         hipStream_t stream)
{
    PYHIP_REQUIRE(x_bf16 && q && scales, "act_quant: null pointer");
    PYHIP_REQUIRE(K > 0 && K % 32 == 0, "act_quant: K=%d must be a positive multiple of 32", K);
    PYHIP_REQUIRE(row_stride_elems >= K && row_stride_elems % 8 == 0,
                  "act_quant: row stride %lld must be >= K and a multiple of 8 elements", (long long)row_stride_elems);
    PYHIP_REQUIRE(((uintptr_t)x_bf16 % 16) == 0 && ((uintptr_t)q % 16) == 0 && ((uintptr_t)scales % 4) == 0,
                  "act_quant: pointers must be 16-byte aligned");
    if(rows <= 0)
        return PYHIP_OK;
    int SK          = (int)pyhip_moe_act_scale_stride(K);
    long long total = rows * SK;
    long long grid  = (total + QUANT_THREADS - 1) / QUANT_THREADS;
    PYHIP_REQUIRE(grid < (1ll << 31), "act_quant: too many rows");
    hipLaunchKernelGGL(moe_act_quant_mxfp4_kernel, dim3((unsigned)grid), dim3(QUANT_THREADS), 0, stream,
                       (const uint16_t*)x_bf16, (long long)row_stride_elems, q, scales, (long long)rows, K, SK,
                       rows_limit);
    PYHIP_CHECK_LAUNCH("moe_act_quant_mxfp4_kernel");
    return PYHIP_OK;
}
