// Device part of the dynamic MXFP4 quantisation of bf16 activations, shared by the stand-alone kernel
// (moe_quant.hip) and by the sort launches that carry it along (moe_sort.hip).
#pragma once
#include "common.h"

struct QuantArgs
{
    const uint16_t* x;         // bf16 [rows, K], row stride ldx elements
    long long ldx;
    uint8_t* q;                // [rows, K/2]
    uint8_t* s;                // [rows, SK]
    long long rows;            // 0: nothing to do
    int K, SK;
    const u32* rows_limit;     // device scalar or null
};

// One thread per 32-element block (id = row * SK + block; blocks past K are padding); 16 consecutive threads own
// one 16-byte scale group, so ids must be handed out in multiples of 16 per wave.
__device__ __forceinline__ void act_quant_block(const QuantArgs& a, long long id)
{
    long long rows = a.rows;
    if(a.rows_limit)
    {
        long long lim = (long long)*a.rows_limit;
        rows          = rows < lim ? rows : lim;
    }
    const long long row = id / a.SK;
    const int j         = (int)(id - row * a.SK);        // block index inside the row (may be padding)
    if(row >= rows)                                      // whole 16-thread groups leave together
        return;
    u32 e8 = 0;
    if(j * 32 < a.K)
    {
        const uint4* src = (const uint4*)(a.x + row * a.ldx + (long long)j * 32);
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
        *(uint4*)(a.q + row * (long long)(a.K / 2) + (long long)j * 16) = o;
    }
    // 4x4 byte transpose of the 16 scales of this group through lane shuffles
    const int jj = j & 15;
    u32 b0 = __shfl(e8, 0 + (jj & 3), 16), b1 = __shfl(e8, 4 + (jj & 3), 16);
    u32 b2 = __shfl(e8, 8 + (jj & 3), 16), b3 = __shfl(e8, 12 + (jj & 3), 16);
    if(jj < 4)
        *(u32*)(a.s + row * (long long)a.SK + (j & ~15) + jj * 4) = b0 | (b1 << 8) | (b2 << 16) | (b3 << 24);
}

// argument checks and the filled-in struct, shared by the entry points that quantise
int pyhip_make_quant_args(const char* name, const void* x_bf16, int64_t row_stride_elems, int64_t rows, int K,
                          uint8_t* q, uint8_t* scales, const uint32_t* rows_limit, QuantArgs* out);
