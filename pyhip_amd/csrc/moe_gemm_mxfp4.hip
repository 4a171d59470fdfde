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
// 1 KB load per 16x128 tile, prefetched four K-steps ahead in a register ring.  Activation tiles
// are shared by the 4 waves: they are DMA'd (buffer_load ... lds, 16 B per lane) three K-steps
// ahead into a ring of four LDS stages, already in operand order (lane-linear 1 KB blocks), so
// the ds_read_b128 of a tile is conflict-free and needs no swizzle.
//
// The weight tile is the MFMA's first operand and the activation tile the second, so a lane ends
// up with 4 consecutive output channels of one row (lane%16 = row, lane/16*4.. = channels).
#include "common.h"

#define GEMM_THREADS 256
#define LDS_PTR(p) ((__attribute__((address_space(3))) void*)(p))

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
    int T, topk, K, N, SK, SC, n_blk, n_tiles, a_rows;
};

template <int OPW, int OPA>
__device__ __forceinline__ v4f mfma_fp4(v4i w, v4i a, v4f c, int w_scale, int a_scale)
{
    v8i W = {w.x, w.y, w.z, w.w, 0, 0, 0, 0};
    v8i A = {a.x, a.y, a.z, a.w, 0, 0, 0, 0};
    return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(W, A, c, 4, 4, OPW, w_scale, OPA, a_scale);
}

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* p, u32 bytes)
{
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, bytes, 0x00020000);
}

template <int N>
__device__ __forceinline__ void wait_vmcnt_barrier()
{
    // own DMA writes complete (all but the N youngest VMEM ops), own LDS reads complete, then meet
    asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(N) : "memory");
}

// STAGE 1 = gate_up, 2 = down.  MT = row groups of 16 per tile.
template <int STAGE, int MT>
__global__ void __launch_bounds__(GEMM_THREADS, (MT <= 8 ? 2 : 1)) moe_gemm_mxfp4_kernel(GemmArgs g)
{
#if defined(__HIP_DEVICE_COMPILE__)   // the host pass only needs the launch stub
    constexpr int BM    = MT * 16;
    constexpr int NA    = (MT + 3) / 4;       // activation tiles DMA'd per wave per K-step
    constexpr int SLOTS = NA * 4;             // tile slots per LDS stage (slots >= MT are never read)
    __shared__ __attribute__((aligned(16))) uint8_t lds_a0[SLOTS * 1024];
    __shared__ __attribute__((aligned(16))) uint8_t lds_a1[SLOTS * 1024];
    __shared__ __attribute__((aligned(16))) uint8_t lds_a2[SLOTS * 1024];
    __shared__ __attribute__((aligned(16))) uint8_t lds_a3[SLOTS * 1024];
    __shared__ __attribute__((aligned(16))) uint8_t lds_s0[SLOTS * 256];   // activation scales of a K-group
    __shared__ __attribute__((aligned(16))) uint8_t lds_s1[SLOTS * 256];
    __shared__ int lds_row[SLOTS * 16];

    const int m_blk = blockIdx.x / g.n_tiles;
    const int nt    = blockIdx.x - m_blk * g.n_tiles;
    if((u32)(m_blk * BM) >= g.num_valid[0])
        return;
    const int e    = (int)g.sorted_e[m_blk];
    const int tid  = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid / WAVE);   // wave-uniform: keeps descriptors and LDS bases scalar
    const int lane = tid % WAVE;
    const int r = lane & 15, kb = lane >> 4;
    const int Kb = g.K / 2;
    const int I  = g.N / 2;   // stage 1 only

    // source row of every tile row (stage 1: gathered token; stage 2: the sorted position itself)
    for(int i = tid; i < SLOTS * 16; i += GEMM_THREADS)
    {
        int row = 0;
        if(i < BM)
        {
            int p = m_blk * BM + i;
            if(STAGE == 1)
            {
                u32 id  = g.sorted_ids[p];
                int tok = (int)(id & 0xFFFFFFu);
                row     = ((int)(id >> 24) < g.topk && tok < g.T) ? tok : 0;   // padding rows read row 0; never stored
            }
            else
                row = p;
        }
        lds_row[i] = row;
    }
    __syncthreads();

    // ---- weight operand: 4 row groups of 16 rows, one buffer resource each (range = the row
    // group's K extent, so prefetches past the end of K are dropped by the bounds check)
    int wrow[4];
#pragma unroll
    for(int j = 0; j < 4; j++)
        wrow[j] = (STAGE == 1) ? ((j >> 1) * I + nt * 128 + wave * 32 + (j & 1) * 16) : (nt * 256 + wave * 64 + j * 16);
    __amdgpu_buffer_rsrc_t wrs[4];
#pragma unroll
    for(int j = 0; j < 4; j++)
        wrs[j] = make_rsrc(g.w + ((size_t)e * g.N + wrow[j]) * Kb, (u32)(16 * Kb));
    // weight scales: rows wrow[0], wrow[1] share a 32-row tile, so do wrow[2], wrow[3]
    const uint8_t* wsptr[2];
#pragma unroll
    for(int h = 0; h < 2; h++)
    {
        size_t R = (size_t)e * g.N + wrow[2 * h];
        wsptr[h] = g.w_s + (R / 32) * (size_t)(g.SC / 8) * 256 + lane * 4;
    }
    // ---- activation operand
    const __amdgpu_buffer_rsrc_t ars  = make_rsrc(g.a_q, (u32)((size_t)g.a_rows * Kb));
    const __amdgpu_buffer_rsrc_t asrs = make_rsrc(g.a_s, (u32)((size_t)g.a_rows * g.SK));
    int a_off[NA];        // byte offset of this lane's 16 B inside a_q for K-step 0, per DMA slot
    int as_off[NA];       // byte offset of this lane's scale dword inside a_s for K-group 0, per DMA slot
#pragma unroll
    for(int i = 0; i < NA; i++)
    {
        const int row = lds_row[(wave + 4 * i) * 16 + r];
        a_off[i]      = row * Kb + kb * 16;
        as_off[i]     = row * g.SK + kb * 4;
    }

    uint8_t* const stage[4]  = {lds_a0, lds_a1, lds_a2, lds_a3};
    uint8_t* const sstage[2] = {lds_s0, lds_s1};
    auto dma_a = [&](auto S, int kt) {
        constexpr int s = decltype(S)::value;
#pragma unroll
        for(int i = 0; i < NA; i++)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(ars, LDS_PTR(stage[s] + (wave + 4 * i) * 1024), 16,
                                                     a_off[i] + kt * 64, 0, 0, 0);
    };
    // one dword per lane: the scales of this lane's (row, K-block) for the 4 K-steps of K-group ks
    auto dma_s = [&](auto S, int ks) {
        constexpr int s = decltype(S)::value;
#pragma unroll
        for(int i = 0; i < NA; i++)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(asrs, LDS_PTR(sstage[s] + (wave + 4 * i) * 256), 4,
                                                     as_off[i] + ks * 16, 0, 0, 0);
    };

    v4f acc[4][MT];
#pragma unroll
    for(int j = 0; j < 4; j++)
#pragma unroll
        for(int mt = 0; mt < MT; mt++)
            acc[j][mt] = (v4f){0.f, 0.f, 0.f, 0.f};

    // ---- prologue: activation tiles of K-steps 0..2 in flight, weight tiles of K-steps 0..3, scales of group 0
    v4i wf[4][4];
    int w_sc[2][4];
    dma_s(std::integral_constant<int, 0>{}, 0);
    dma_a(std::integral_constant<int, 0>{}, 0);
    dma_a(std::integral_constant<int, 1>{}, 1);
    dma_a(std::integral_constant<int, 2>{}, 2);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for(int s = 0; s < 4; s++)
#pragma unroll
        for(int j = 0; j < 4; j++)
            wf[s][j] = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(wrs[j], lane * 16 + s * 1024, 0, 0));
#pragma unroll
    for(int h = 0; h < 2; h++)
#pragma unroll
        for(int c = 0; c < 2; c++)
            w_sc[0][h * 2 + c] = *(const int*)(wsptr[h] + (size_t)c * 256);
    __builtin_amdgcn_sched_barrier(0);
    // scales and stage 0 must have landed: younger ops = 2*NA (DMA) + 16 + 4
    wait_vmcnt_barrier<2 * NA + 16 + 4>();

    const int KS = g.K / 512;
    auto kgroup = [&](auto P, int ks) {
        constexpr int p = decltype(P)::value;     // parity of ks: which scale registers are live
        static_for<4>([&](auto U) {
            constexpr int u = decltype(U)::value;
            const int kt    = ks * 4 + u;
            // (1) activation tile of K-step kt+3 -> stage (u+3)%4 (last read in step kt-1)
            dma_a(std::integral_constant<int, (u + 3) % 4>{}, kt + 3);
            // (2) scales of the next K-group
            if(u == 0)
            {
                const int kn = ks + 1 < KS ? ks + 1 : ks;
                dma_s(std::integral_constant<int, p ^ 1>{}, kn);
#pragma unroll
                for(int h = 0; h < 2; h++)
#pragma unroll
                    for(int c = 0; c < 2; c++)
                        w_sc[p ^ 1][h * 2 + c] = *(const int*)(wsptr[h] + (size_t)(kn * 2 + c) * 256);
            }
            __builtin_amdgcn_sched_barrier(0);
            // (3) MFMAs of K-step kt.  Activation scales of the whole tile first (one dword per 16-row group, the
            //     byte of this K-step is picked by op_sel), then tile operands two reads ahead of their MFMAs.
            int asc[MT];
#pragma unroll
            for(int mt = 0; mt < MT; mt++)
                asc[mt] = *(const int*)(sstage[p] + mt * 256 + lane * 4);
            __builtin_amdgcn_sched_barrier(0);
            v4i af[MT];
#pragma unroll
            for(int mt = 0; mt < MT; mt++)
                af[mt] = *(const v4i*)(stage[u] + mt * 1024 + lane * 16);
#pragma unroll
            for(int mt = 0; mt < MT; mt++)
            {
                // weight-scale byte = (kt%2)*2 + (row%32)/16 ; activation-scale byte = kt%4
                acc[0][mt] = mfma_fp4<(u & 1) * 2 + 0, u>(wf[u][0], af[mt], acc[0][mt], w_sc[p][0 + (u >> 1)], asc[mt]);
                acc[1][mt] = mfma_fp4<(u & 1) * 2 + 1, u>(wf[u][1], af[mt], acc[1][mt], w_sc[p][0 + (u >> 1)], asc[mt]);
                acc[2][mt] = mfma_fp4<(u & 1) * 2 + 0, u>(wf[u][2], af[mt], acc[2][mt], w_sc[p][2 + (u >> 1)], asc[mt]);
                acc[3][mt] = mfma_fp4<(u & 1) * 2 + 1, u>(wf[u][3], af[mt], acc[3][mt], w_sc[p][2 + (u >> 1)], asc[mt]);
            }
            __builtin_amdgcn_sched_group_barrier(0x100, MT < 2 ? MT : 2, 0);
#pragma unroll
            for(int mt = 0; mt < MT; mt++)
            {
                __builtin_amdgcn_sched_group_barrier(0x008, 4, 0);
                if(mt + 2 < MT)
                    __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
            // (4) weight tiles of K-step kt+4 into the registers just consumed
#pragma unroll
            for(int j = 0; j < 4; j++)
                wf[u][j] = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(wrs[j], lane * 16 + (kt + 4) * 1024, 0, 0));
            __builtin_amdgcn_sched_barrier(0);
            // (5) the activation tile of K-step kt+1 was DMA'd in step kt-2; VMEM ops certainly issued
            //     after it: 4 (kt-2) + NA+S(u-1)+4 (kt-1) + NA+S(u)+4 (kt), S = scale loads (u == 0 only)
            constexpr int S = NA + 4;
            wait_vmcnt_barrier<12 + 2 * NA + ((u == 0 || u == 1) ? S : 0)>();
        });
    };
    for(int ks = 0; ks < KS; ks += 2)
    {
        kgroup(std::integral_constant<int, 0>{}, ks);
        if(ks + 1 < KS)
            kgroup(std::integral_constant<int, 1>{}, ks + 1);
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
#endif
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
                        int K, int block_m, int64_t n_blk, int64_t a_rows)
{
    PYHIP_REQUIRE(a_q && a_s && w && w_s && sorted_ids && sorted_e && num_valid && out, "%s: null pointer", name);
    PYHIP_REQUIRE(K > 0 && K % 512 == 0, "%s: K=%d must be a positive multiple of 512", name, K);
    PYHIP_REQUIRE(block_m == 16 || block_m == 32 || block_m == 64 || block_m == 128 || block_m == 256,
                  "%s: block_m=%d not in {16,32,64,128,256}", name, block_m);
    PYHIP_REQUIRE(n_blk >= 0 && n_blk < (1 << 24), "%s: n_blk=%lld", name, (long long)n_blk);
    PYHIP_REQUIRE(a_rows > 0 && a_rows * (int64_t)(K / 2) < (1ll << 32),
                  "%s: activation matrix of %lld rows x %d exceeds the 4 GiB buffer range", name, (long long)a_rows, K);
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
                          a2_bf16, hidden, block_m, n_blk, tokens);
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
    g.n_blk = (int)n_blk; g.n_tiles = inter / 128; g.a_rows = tokens;
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
                          out3_bf16, inter, block_m, n_blk, n_blk * block_m);
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
    g.n_blk = (int)n_blk; g.n_tiles = hidden / 256; g.a_rows = (int)(n_blk * block_m);
    return launch_gemm<2>(g, block_m, stream);
}
