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
#include "quant_device.h"

#define QUANT_THREADS 256

extern "C" __global__ void __launch_bounds__(QUANT_THREADS) moe_act_quant_mxfp4_kernel(QuantArgs a)
{
    act_quant_block(a, (long long)blockIdx.x * QUANT_THREADS + threadIdx.x);
}

extern "C" int64_t pyhip_moe_act_scale_stride(int K) { return ((int64_t)K + 511) / 512 * 16; }

int pyhip_make_quant_args(const char* name, const void* x_bf16, int64_t row_stride_elems, int64_t rows, int K,
                          uint8_t* q, uint8_t* scales, const uint32_t* rows_limit, QuantArgs* out)
{
    PYHIP_REQUIRE(x_bf16 && q && scales, "%s: null pointer", name);
    PYHIP_REQUIRE(K > 0 && K % 32 == 0, "%s: K=%d must be a positive multiple of 32", name, K);
    PYHIP_REQUIRE(row_stride_elems >= K && row_stride_elems % 8 == 0,
                  "%s: row stride %lld must be >= K and a multiple of 8 elements", name, (long long)row_stride_elems);
    PYHIP_REQUIRE(((uintptr_t)x_bf16 % 16) == 0 && ((uintptr_t)q % 16) == 0 && ((uintptr_t)scales % 4) == 0,
                  "%s: pointers must be 16-byte aligned", name);
    out->x = (const uint16_t*)x_bf16; out->ldx = (long long)row_stride_elems; out->q = q; out->s = scales;
    out->rows = rows > 0 ? (long long)rows : 0; out->K = K; out->SK = (int)pyhip_moe_act_scale_stride(K);
    out->rows_limit = rows_limit;
    PYHIP_REQUIRE(out->rows * out->SK < (1ll << 40), "%s: too many rows", name);
    return PYHIP_OK;
}

extern "C" int pyhip_moe_act_quant_mxfp4(const void* x_bf16, int64_t row_stride_elems, int64_t rows, int K,
                                         uint8_t* q, uint8_t* scales, const uint32_t* rows_limit,
                                         hipStream_t stream)
{
    QuantArgs a;
    int rc = pyhip_make_quant_args("act_quant", x_bf16, row_stride_elems, rows, K, q, scales, rows_limit, &a);
    if(rc)
        return rc;
    if(a.rows == 0)
        return PYHIP_OK;
    long long grid = (a.rows * a.SK + QUANT_THREADS - 1) / QUANT_THREADS;
    PYHIP_REQUIRE(grid < (1ll << 31), "act_quant: too many rows");
    hipLaunchKernelGGL(moe_act_quant_mxfp4_kernel, dim3((unsigned)grid), dim3(QUANT_THREADS), 0, stream, a);
    PYHIP_CHECK_LAUNCH("moe_act_quant_mxfp4_kernel");
    return PYHIP_OK;
}
