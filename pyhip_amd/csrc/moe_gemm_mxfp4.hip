// Grouped MXFP4 x MXFP4 GEMMs of the fused-MoE layer on the gfx950 scaled MFMA
// (v_mfma_scale_f32_16x16x128_f8f6f4 with cbsz = blgp = 4: e2m1 values, one e8m0 scale per
// 32-element K block on both operands, fp32 accumulation).
//
//   stage 1 (gate_up): a2[p, c] = bf16( silu(x_p . Wg[c] + bg[c]) * (x_p . Wu[c] + bu[c]) )
//                      x = activations gathered by sorted token id, p = sorted position
//   stage 2 (down)   : out3[token, slot, h] = bf16( (a2_p . Wd[h] + bd[h]) * routing_weight_p )
// (Reference kernels with the same contract: src/contrib/moe_gemm_mxfp4.py:972-1333.)
//
// Work decomposition.  One workgroup (4 waves) owns BM = 16*MT sorted rows of one expert and 256
// weight rows (stage 1: 128 gate rows and the matching 128 up rows, so SiLU(gate)*up stays in
// registers).  Wave w owns ALL BM rows and 64 of the weight rows.  Weight tiles are therefore
// private to a wave and go HBM -> VGPR -> MFMA directly: the pre-shuffled weight layout
// ([N/16][Kb/64][lane][16 B], src/misc.py:116-130) is exactly the operand layout, one coalesced
// 1 KB load per 16x128 tile.  Activation tiles are shared by the 4 waves and are staged in LDS in
// operand order (lane-linear 1 KB blocks, conflict-free ds_read_b128).
//
// The weight tile is the MFMA's first operand and the activation tile the second, so a lane ends
// up with 4 consecutive output channels of one row (lane%16 = row, lane/16*4.. = channels).
#include "common.h"

#define GEMM_THREADS 256

struct GemmArgs
{
    const uint8_t* a_q;        // activations, e2m1 pairs  [a_rows, K/2]
    const uint8_t* a_s;        // activation scales        [a_rows, SK]  (layout: moe_quant.hip)
    const uint8_t* w;          // weights, pre-shuffled    [E, N, K/2]
    const uint8_t* w_s;        // weight scales, shuffled  [E*N (padded to 256), SC]
    const uint16_t* bias;      // bf16 [E, N] or null
    const u32* sorted_ids;     // [n_blk * BM]
    const float* sorted_w;     // [n_blk * BM]
    const u32* sorted_e;       // [n_blk]
    const u32* num_valid;      // [2]
    void* out;                 // stage 1: bf16 [n_blk*BM, N/2]; stage 2: bf16 [T, topk, N]
    int T, topk, K, N, SK, SC, n_blk, n_tiles;
};

template <int OPW, int OPA>
__device__ __forceinline__ v4f mfma_fp4(v4i w, v4i a, v4f c, int w_scale, int a_scale)
{
    v8i W = {w.x, w.y, w.z, w.w, 0, 0, 0, 0};
    v8i A = {a.x, a.y, a.z, a.w, 0, 0, 0, 0};
    return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(W, A, c, 4, 4, OPW, w_scale, OPA, a_scale);
}

// STAGE 1 = gate_up, 2 = down.  MT = row groups of 16 per tile.
template <int STAGE, int MT>
__global__ void __launch_bounds__(GEMM_THREADS) moe_gemm_mxfp4_kernel(GemmArgs g)
{
    constexpr int BM = MT * 16;
    __shared__ __attribute__((aligned(16))) uint8_t lds_a[MT * 1024];
    __shared__ int lds_row[BM];

    const int m_blk = blockIdx.x / g.n_tiles;
    const int nt    = blockIdx.x - m_blk * g.n_tiles;
    if((u32)(m_blk * BM) >= g.num_valid[0])
        return;
    const int e    = (int)g.sorted_e[m_blk];
    const int tid  = threadIdx.x;
    const int wave = tid / WAVE, lane = tid % WAVE;
    const int r = lane & 15, kb = lane >> 4;
    const int Kb = g.K / 2;
    const int I  = g.N / 2;   // stage 1 only

    // source row of every tile row (stage 1: gathered token; stage 2: the sorted position itself)
    for(int i = tid; i < BM; i += GEMM_THREADS)
    {
        int p = m_blk * BM + i;
        if(STAGE == 1)
        {
            u32 id    = g.sorted_ids[p];
            int tok   = (int)(id & 0xFFFFFFu);
            lds_row[i] = ((int)(id >> 24) < g.topk && tok < g.T) ? tok : 0;   // padding rows read row 0; never stored
        }
        else
            lds_row[i] = p;
    }
    __syncthreads();

    // the 4 weight row groups (16 rows each) of this wave, as row indices inside the expert
    int wrow[4];
#pragma unroll
    for(int j = 0; j < 4; j++)
        wrow[j] = (STAGE == 1) ? ((j >> 1) * I + nt * 128 + wave * 32 + (j & 1) * 16) : (nt * 256 + wave * 64 + j * 16);

    const uint8_t* wptr[4];
#pragma unroll
    for(int j = 0; j < 4; j++)
        wptr[j] = g.w + ((size_t)e * g.N + wrow[j]) * Kb + lane * 16;   // (row/16) * (Kb/64) * 1024 = row * Kb
    // scale dwords: rows wrow[0], wrow[1] share a 32-row tile, so do wrow[2], wrow[3]
    const uint8_t* wsptr[2];
#pragma unroll
    for(int h = 0; h < 2; h++)
    {
        size_t R  = (size_t)e * g.N + wrow[2 * h];
        wsptr[h]  = g.w_s + (R / 32) * (size_t)(g.SC / 8) * 256 + lane * 4;
    }
    const uint8_t* asptr[MT];
    const uint8_t* aqptr[(MT + 3) / 4];
#pragma unroll
    for(int mt = 0; mt < MT; mt++)
        asptr[mt] = g.a_s + (size_t)lds_row[mt * 16 + r] * g.SK + kb * 4;
#pragma unroll
    for(int i = 0; i < (MT + 3) / 4; i++)
    {
        int mt   = wave + i * 4;
        aqptr[i] = g.a_q + (size_t)lds_row[(mt < MT ? mt : 0) * 16 + r] * Kb + kb * 16;
    }

    v4f acc[4][MT];
#pragma unroll
    for(int j = 0; j < 4; j++)
#pragma unroll
        for(int mt = 0; mt < MT; mt++)
            acc[j][mt] = (v4f){0.f, 0.f, 0.f, 0.f};

    const int ksteps = g.K / 512;
    for(int ks = 0; ks < ksteps; ks++)
    {
        int a_sc[MT];
#pragma unroll
        for(int mt = 0; mt < MT; mt++)
            a_sc[mt] = *(const int*)(asptr[mt] + ks * 16);
        int w_sc[2][2];
#pragma unroll
        for(int h = 0; h < 2; h++)
#pragma unroll
            for(int c = 0; c < 2; c++)
                w_sc[h][c] = *(const int*)(wsptr[h] + (size_t)(ks * 2 + c) * 256);

        static_for<4>([&](auto U) {
            constexpr int u = decltype(U)::value;
            const int kt = ks * 4 + u;
            __syncthreads();
#pragma unroll
            for(int i = 0; i < (MT + 3) / 4; i++)
            {
                int mt = wave + i * 4;
                if(mt < MT)
                    *(v4i*)(lds_a + mt * 1024 + lane * 16) = *(const v4i*)(aqptr[i] + kt * 64);
            }
            v4i wf[4];
#pragma unroll
            for(int j = 0; j < 4; j++)
                wf[j] = *(const v4i*)(wptr[j] + (size_t)kt * 1024);
            __syncthreads();
#pragma unroll
            for(int mt = 0; mt < MT; mt++)
            {
                v4i af = *(const v4i*)(lds_a + mt * 1024 + lane * 16);
                // weight-scale byte = (kt%2)*2 + (row%32)/16 ; activation-scale byte = kt%4
                acc[0][mt] = mfma_fp4<(u & 1) * 2 + 0, u>(wf[0], af, acc[0][mt], w_sc[0][u >> 1], a_sc[mt]);
                acc[1][mt] = mfma_fp4<(u & 1) * 2 + 1, u>(wf[1], af, acc[1][mt], w_sc[0][u >> 1], a_sc[mt]);
                acc[2][mt] = mfma_fp4<(u & 1) * 2 + 0, u>(wf[2], af, acc[2][mt], w_sc[1][u >> 1], a_sc[mt]);
                acc[3][mt] = mfma_fp4<(u & 1) * 2 + 1, u>(wf[3], af, acc[3][mt], w_sc[1][u >> 1], a_sc[mt]);
            }
        });
    }

    // ---------------------------------------------------------------- epilogue
    if(STAGE == 1)
    {
        uint16_t* out = (uint16_t*)g.out;
#pragma unroll
        for(int j = 0; j < 2; j++)
        {
            const int ch = nt * 128 + wave * 32 + j * 16 + kb * 4;
            float bg[4] = {0, 0, 0, 0}, bu[4] = {0, 0, 0, 0};
            if(g.bias)
            {
#pragma unroll
                for(int i = 0; i < 4; i++)
                {
                    bg[i] = bf16_bits_to_f32(g.bias[(size_t)e * g.N + ch + i]);
                    bu[i] = bf16_bits_to_f32(g.bias[(size_t)e * g.N + I + ch + i]);
                }
            }
#pragma unroll
            for(int mt = 0; mt < MT; mt++)
            {
                const int p  = m_blk * BM + mt * 16 + r;
                const u32 id = g.sorted_ids[p];
                const bool ok = (int)(id >> 24) < g.topk;
                float v[4];
#pragma unroll
                for(int i = 0; i < 4; i++)
                    v[i] = ok ? silu_f32(acc[j][mt][i] + bg[i]) * (acc[j + 2][mt][i] + bu[i]) : 0.f;
                uint2 o = make_uint2(pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3]));
                *(uint2*)(out + (size_t)p * I + ch) = o;
            }
        }
    }
    else
    {
        uint16_t* out = (uint16_t*)g.out;
#pragma unroll
        for(int mt = 0; mt < MT; mt++)
        {
            const int p  = m_blk * BM + mt * 16 + r;
            const u32 id = g.sorted_ids[p];
            const int tok = (int)(id & 0xFFFFFFu), slot = (int)(id >> 24);
            if(slot >= g.topk || tok >= g.T)
                continue;
            const float rw = g.sorted_w[p];
#pragma unroll
            for(int j = 0; j < 4; j++)
            {
                const int ch = nt * 256 + wave * 64 + j * 16 + kb * 4;
                float b[4] = {0, 0, 0, 0};
                if(g.bias)
#pragma unroll
                    for(int i = 0; i < 4; i++)
                        b[i] = bf16_bits_to_f32(g.bias[(size_t)e * g.N + ch + i]);
                uint2 o = make_uint2(pack_bf16x2((acc[j][mt][0] + b[0]) * rw, (acc[j][mt][1] + b[1]) * rw),
                                     pack_bf16x2((acc[j][mt][2] + b[2]) * rw, (acc[j][mt][3] + b[3]) * rw));
                *(uint2*)(out + ((size_t)tok * g.topk + slot) * g.N + ch) = o;
            }
        }
    }
}

template <int STAGE>
static int launch_gemm(const GemmArgs& g, int block_m, hipStream_t stream)
{
    dim3 grid((unsigned)(g.n_tiles * g.n_blk)), block(GEMM_THREADS);
    switch(block_m)
    {
    case 16: hipLaunchKernelGGL((moe_gemm_mxfp4_kernel<STAGE, 1>), grid, block, 0, stream, g); break;
    case 32: hipLaunchKernelGGL((moe_gemm_mxfp4_kernel<STAGE, 2>), grid, block, 0, stream, g); break;
    case 64: hipLaunchKernelGGL((moe_gemm_mxfp4_kernel<STAGE, 4>), grid, block, 0, stream, g); break;
    case 128: hipLaunchKernelGGL((moe_gemm_mxfp4_kernel<STAGE, 8>), grid, block, 0, stream, g); break;
    case 256: hipLaunchKernelGGL((moe_gemm_mxfp4_kernel<STAGE, 16>), grid, block, 0, stream, g); break;
    default: pyhip_set_error("moe_gemm: block_m=%d not in {16,32,64,128,256}", block_m); return PYHIP_ERR_INVALID;
    }
    PYHIP_CHECK_LAUNCH("moe_gemm_mxfp4_kernel");
    return PYHIP_OK;
}

static int check_common(const char* name, const void* a_q, const void* a_s, const void* w, const void* w_s,
                        const void* sorted_ids, const void* sorted_e, const void* num_valid, const void* out,
                        int K, int block_m, int64_t n_blk)
{
    PYHIP_REQUIRE(a_q && a_s && w && w_s && sorted_ids && sorted_e && num_valid && out, "%s: null pointer", name);
    PYHIP_REQUIRE(K > 0 && K % 512 == 0, "%s: K=%d must be a positive multiple of 512", name, K);
    PYHIP_REQUIRE(block_m == 16 || block_m == 32 || block_m == 64 || block_m == 128 || block_m == 256,
                  "%s: block_m=%d not in {16,32,64,128,256}", name, block_m);
    PYHIP_REQUIRE(n_blk >= 0 && n_blk < (1 << 24), "%s: n_blk=%lld", name, (long long)n_blk);
    PYHIP_REQUIRE(((uintptr_t)a_q % 16) == 0 && ((uintptr_t)a_s % 4) == 0 && ((uintptr_t)w % 16) == 0 &&
                      ((uintptr_t)w_s % 4) == 0 && ((uintptr_t)out % 8) == 0,
                  "%s: unaligned pointer", name);
    return PYHIP_OK;
}

extern "C" int pyhip_moe_gemm1_mxfp4(const uint8_t* a_q, const uint8_t* a_scale, const uint8_t* w1,
                                     const uint8_t* w1_scale, const void* bias1_bf16, const uint32_t* sorted_ids,
                                     const uint32_t* sorted_expert_ids, const uint32_t* num_valid_ids, void* a2_bf16,
                                     int tokens, int topk, int experts, int hidden, int inter, int block_m,
                                     int64_t n_blk, hipStream_t stream)
{
    int rc = check_common("moe_gemm1", a_q, a_scale, w1, w1_scale, sorted_ids, sorted_expert_ids, num_valid_ids,
                          a2_bf16, hidden, block_m, n_blk);
    if(rc)
        return rc;
    PYHIP_REQUIRE(inter > 0 && inter % 128 == 0, "moe_gemm1: inter=%d must be a multiple of 128", inter);
    PYHIP_REQUIRE(tokens > 0 && topk > 0 && experts > 0, "moe_gemm1: bad sizes");
    if(n_blk == 0)
        return PYHIP_OK;
    GemmArgs g;
    g.a_q = a_q; g.a_s = a_scale; g.w = w1; g.w_s = w1_scale; g.bias = (const uint16_t*)bias1_bf16;
    g.sorted_ids = sorted_ids; g.sorted_w = nullptr; g.sorted_e = sorted_expert_ids; g.num_valid = num_valid_ids;
    g.out = a2_bf16;
    g.T = tokens; g.topk = topk; g.K = hidden; g.N = 2 * inter;
    g.SK = (hidden + 511) / 512 * 16;
    g.SC = (hidden / 32 + 7) / 8 * 8;
    g.n_blk = (int)n_blk; g.n_tiles = inter / 128;
    return launch_gemm<1>(g, block_m, stream);
}

extern "C" int pyhip_moe_gemm2_mxfp4(const uint8_t* a2_q, const uint8_t* a2_scale, const uint8_t* w2,
                                     const uint8_t* w2_scale, const void* bias2_bf16, const uint32_t* sorted_ids,
                                     const float* sorted_weights, const uint32_t* sorted_expert_ids,
                                     const uint32_t* num_valid_ids, void* out3_bf16, int tokens, int topk,
                                     int experts, int hidden, int inter, int block_m, int64_t n_blk,
                                     hipStream_t stream)
{
    int rc = check_common("moe_gemm2", a2_q, a2_scale, w2, w2_scale, sorted_ids, sorted_expert_ids, num_valid_ids,
                          out3_bf16, inter, block_m, n_blk);
    if(rc)
        return rc;
    PYHIP_REQUIRE(sorted_weights, "moe_gemm2: null sorted_weights");
    PYHIP_REQUIRE(hidden > 0 && hidden % 256 == 0, "moe_gemm2: hidden=%d must be a multiple of 256", hidden);
    PYHIP_REQUIRE(tokens > 0 && topk > 0 && experts > 0, "moe_gemm2: bad sizes");
    if(n_blk == 0)
        return PYHIP_OK;
    GemmArgs g;
    g.a_q = a2_q; g.a_s = a2_scale; g.w = w2; g.w_s = w2_scale; g.bias = (const uint16_t*)bias2_bf16;
    g.sorted_ids = sorted_ids; g.sorted_w = sorted_weights; g.sorted_e = sorted_expert_ids;
    g.num_valid = num_valid_ids; g.out = out3_bf16;
    g.T = tokens; g.topk = topk; g.K = inter; g.N = hidden;
    g.SK = (inter + 511) / 512 * 16;
    g.SC = (inter / 32 + 7) / 8 * 8;
    g.n_blk = (int)n_blk; g.n_tiles = hidden / 256;
    return launch_gemm<2>(g, block_m, stream);
}
