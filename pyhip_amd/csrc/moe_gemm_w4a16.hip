// Grouped GEMMs of the fused-MoE layer with bf16 activations and MXFP4 weights ("w4a16"): the weights are
// expanded to bf16 in registers (e2m1 value times its e8m0 block scale is exact in bf16) and multiplied with
// the bf16 MFMA.  This is the variant the reference runs when few tokens are routed
// (src/contrib/moe.py:362-787, moe_2stage_splitk with fp4 weights, driven by
// tests/contrib/moe/test_moe.py:347-374); at such sizes the layer only streams weights, so the kernel is kept
// simple: one workgroup per (row block, weight tile), the K loop software-pipelined one K-step ahead.
// Three mappings of a workgroup's waves:
//   SPLIT = 0 : four waves, tile of 256 weight rows, wave w owns 64 of them over the whole K range;
//   SPLIT = 4 : four waves share a tile of 64 weight rows, wave w takes K-steps w, w+4, ... and the four
//               partial sums meet in LDS (the reference's split-K arrangement, src/contrib/moe.py:362-500).
//               Four times as many workgroups: used when the layer would otherwise not fill the GPU.
//   SPLIT = 16: the same with sixteen waves per workgroup, for a long K with so few tiles that even the four-way
//               split leaves most CUs without a wave (Mixtral's down GEMM at one token: 128 tiles of 112 K-steps;
//               every wave is a chain of dependent K-steps, and the chain, not the bandwidth, sets the time).
//
// Operand mapping.  A pre-shuffled 1 KB weight block (src/misc.py:116-130) gives lane (row = l % 16,
// kb = l / 16) the 32 consecutive K-elements kb*32 .. kb*32+31 of its row.  The bf16 MFMA 16x16x32 wants 8
// K-elements per lane, so one block feeds four MFMAs; in MFMA i the lane contributes elements
// kb*32 + i*8 .. +7, and the token side loads the same elements of its activation row (16 contiguous bytes).
// Any fixed pairing of K-elements is a valid contraction order.  Weights are src A and tokens src B, so a lane
// ends with 4 consecutive output channels of token l % 16, as in the MXFP4-activation kernel.
#include "common.h"

#define W4A16_THREADS 256

struct W4A16Args
{
    const uint16_t* a;         // activations bf16: stage 1 [T, K] (token order); stage 2 [n_blk*BM, K] (sorted order)
    const uint8_t* w;          // weights, pre-shuffled    [E, N, K/2]
    const uint8_t* w_s;        // weight scales, shuffled  [E*N (padded to 256), SC]
    const uint16_t* bias;      // bf16 [E, N] or null
    const u32* sorted_ids;     // [n_blk * BM]
    const float* sorted_w;     // [n_blk * BM] (stage 2)
    const u32* sorted_e;       // [n_blk]
    const u32* num_valid;      // [2]
    uint16_t* out;             // stage 1: bf16 [n_blk*BM, N/2]; stage 2: bf16 [T, topk, N]
    int T, topk, K, N, SC, n_tiles;
    GatedAct act;              // stage 1: the gated activation (common.h)
    // One token, no sort (the *_token entry points): block b is the token's slot b, with one real row.  The kernels read
    // the routing themselves: the expert of the slot, whether the slot takes part (the sort's drop rule) and the local
    // id of its expert under an expert mask.  sorted_ids / sorted_w / sorted_e / num_valid are not used then.
    const int* token_ids     = nullptr;   // [topk] expert ids of the token's slots
    const float* token_w     = nullptr;   // [topk] routing weights (stage 2)
    const int* expert_mask   = nullptr;   // [experts] or null
    const int* num_local_tok = nullptr;   // device scalar or null: 0 = the token is not this rank's
    int experts              = 0;
};

// 32 e2m1 values (4 dwords) times 2^(scale byte - 127) -> four MFMA operands of 8 bf16
__device__ __forceinline__ void expand_fp4(const v4i& w, u32 scale_byte, v8bf (&o)[4])
{
    const float sc = __builtin_bit_cast(float, scale_byte << 23);
#pragma unroll
    for(int i = 0; i < 4; i++)
    {
        const u32 d = (u32)w[i];
        v2bf p0 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(d, sc, 0);
        v2bf p1 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(d, sc, 1);
        v2bf p2 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(d, sc, 2);
        v2bf p3 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(d, sc, 3);
        o[i] = (v8bf){p0[0], p0[1], p1[0], p1[1], p2[0], p2[1], p3[0], p3[1]};
    }
}

// STAGE 1 = gate_up (+ SiLU(gate) * up), 2 = down (* routing weight).  MT = row groups of 16 per tile.
// SPLIT = 0: every wave owns 64 weight rows over the whole K.  4 / 16: that many waves share a 64-row weight tile and
// split K.  32 (down GEMM only): sixteen waves share a 32-row weight tile, and every wave keeps three K-steps of
// operands in flight instead of two.  For the down GEMM of a layer with few experts and a long K at one or two tokens
// (Mixtral shape: 2 experts x 16 tiles of 256 rows, K = 14336) the sixteen-wave split starts 128 workgroups on 256 CUs,
// and a wave walks its seven K-steps one memory latency at a time; half as wide a tile fills the chip, and the
// narrower tile leaves the registers for the third K-step.
template <int STAGE, int MT, int SPLIT>
__global__ void __launch_bounds__(SPLIT >= 16 ? 1024 : W4A16_THREADS) moe_gemm_w4a16_kernel(W4A16Args g)
{
    constexpr int BM      = MT * 16;
    constexpr bool SPLITK = SPLIT != 0;
    constexpr bool DEEP   = SPLIT == 32;
    constexpr int NW      = DEEP ? 16 : SPLIT;    // waves that split K
    constexpr int RG      = DEEP ? 2 : 4;         // 16-row weight row groups of a wave
    // K-steps of operands in registers: three where a wave's K loop is a chain of a few memory latencies (the 16-row
    // tile under a K split; 151-153 registers, three waves per SIMD instead of four: Mixtral shape, 1 / 4 tokens - 3 %,
    // nothing lost elsewhere), two otherwise
    constexpr int NB      = (DEEP || (SPLIT == 4 && MT == 1)) ? 3 : 2;
    static_assert(!DEEP || STAGE == 2, "the 32-row tile exists for the down GEMM");
    __shared__ float red[SPLITK ? NW * RG * MT * WAVE * 4 : 1];  // [wave][j][mt][lane][4]
    const int tid = threadIdx.x, lane = tid % WAVE;
    const int wave = __builtin_amdgcn_readfirstlane(tid / WAVE);
    const int r = lane & 15, kb = lane >> 4;
    const int m_blk = blockIdx.x / g.n_tiles, nt = blockIdx.x - m_blk * g.n_tiles;
    const bool one_token = g.token_ids != nullptr;
    int e;
    if(one_token)
    {
        if(m_blk >= g.topk || (g.num_local_tok && *g.num_local_tok < 1))
            return;
        const int eg = g.token_ids[m_blk];
        if(!moe_pair_is_kept(eg, g.experts, g.expert_mask))
            return;
        e = eg;
        if(g.expert_mask)                     // local id: the experts this rank holds before this one
        {
            e = 0;
            for(int i0 = 0; i0 < eg; i0 += WAVE)
                e += __builtin_popcountll(__ballot(i0 + lane < eg && g.expert_mask[i0 + lane] != 0));
            e = __builtin_amdgcn_readfirstlane(e);
        }
    }
    else
    {
        if((u32)(m_blk * BM) >= g.num_valid[0])
            return;
        e = (int)g.sorted_e[m_blk];
    }
    // sorted id of position p: (slot << 24) | token; positions without a row carry slot = topk
    auto sorted_id = [&](int p) __attribute__((always_inline)) -> u32 {
        if(one_token)
            return p == m_blk * BM ? (u32)m_blk << 24 : ((u32)g.topk << 24) | (u32)g.T;
        return g.sorted_ids[p];
    };
    const int Kb = g.K / 2, I = g.N / 2;
    // first output channel of this wave's rows (stage 1: within the gate half; the up half is I further)
    const int chbase = STAGE == 1 ? (SPLITK ? nt * 32 : nt * 128 + wave * 32) : (SPLITK ? nt * (16 * RG) : nt * 256 + wave * 64);

    // weight row groups of this wave: j = 0..3 (stage 1: j>>1 selects gate / up)
    const uint8_t* wp[RG];
    const uint8_t* sp[RG];     // scale tile row (32 weight rows) of row group j
    int sbyte_row[RG];         // which 16-row half of the 32-row scale tile
    const size_t sc_tile = (size_t)(g.SC / 8) * 256;
#pragma unroll
    for(int j = 0; j < RG; j++)
    {
        const size_t row = STAGE == 1 ? (size_t)e * g.N + (j >> 1) * I + chbase + (j & 1) * 16
                                      : (size_t)e * g.N + chbase + j * 16;
        wp[j]        = g.w + row * Kb + lane * 16;
        sp[j]        = g.w_s + (row / 32) * sc_tile + lane * 4;
        sbyte_row[j] = (int)((row / 16) & 1);
    }
    // activation rows of this lane, one per row group
    const uint16_t* ap[MT];
    bool ok[MT];
    u32 ids[MT];
    const int tok0 = STAGE == 1 ? (int)(sorted_id(m_blk * BM) & 0xFFFFFFu) : 0;
#pragma unroll
    for(int mt = 0; mt < MT; mt++)
    {
        const int p  = m_blk * BM + mt * 16 + r;
        ids[mt]      = sorted_id(p);
        const int tok = (int)(ids[mt] & 0xFFFFFFu), slot = (int)(ids[mt] >> 24);
        ok[mt]       = slot < g.topk && tok < g.T;
        // padding rows compute nothing that is stored: they all read the row of the block's first position, which
        // always holds a routed row and is read anyway, so the loads coalesce and a sparsely filled block does
        // not pull 16 distinct rows through the L2 per K-step
        const size_t row = STAGE == 1 ? (size_t)(ok[mt] ? tok : tok0) : (size_t)(ok[mt] ? p : m_blk * BM);
        ap[mt]       = g.a + row * g.K + kb * 32;
    }

    v4f acc[RG][MT];
#pragma unroll
    for(int j = 0; j < RG; j++)
#pragma unroll
        for(int mt = 0; mt < MT; mt++)
            acc[j][mt] = (v4f){0.f, 0.f, 0.f, 0.f};

    const int KT = g.K / 128;
    constexpr int KSTRIDE = SPLITK ? NW : 1;
    v4i wf[NB][RG];
    v4i af[NB][MT][4];
    u32 wsc[NB][RG];           // scale dwords (one covers the two K-steps of a 256-K column tile), loaded with
                               // the K-step's weights: fetched only when needed, their latency would add to every step
    auto load_step = [&](auto BB, int kt) __attribute__((always_inline)) {
        constexpr int buf = decltype(BB)::value;
#pragma unroll
        for(int j = 0; j < RG; j++)
            wsc[buf][j] = *(const u32*)(sp[j] + (size_t)(kt >> 1) * 256);
#pragma unroll
        for(int j = 0; j < RG; j++)
            wf[buf][j] = __builtin_nontemporal_load((const v4i*)(wp[j] + (size_t)kt * 1024));
#pragma unroll
        for(int mt = 0; mt < MT; mt++)
#pragma unroll
            for(int i = 0; i < 4; i++)
                af[buf][mt][i] = *(const v4i*)(ap[mt] + kt * 128 + i * 8);
    };
    // the MFMAs of one K-step from register set P
    auto mfma_step = [&](auto PP, int kt) __attribute__((always_inline)) {
        constexpr int P = decltype(PP)::value;
#pragma unroll
        for(int j = 0; j < RG; j++)
        {
            // scale byte of (K-step parity, 16-row half): tests/contrib/moe/test_fused_moe.py:222-236
            const int kpar = SPLITK ? (kt & 1) : P;          // without the split the parity is the register set
            const u32 sb   = (wsc[P][j] >> (8 * (kpar * 2 + sbyte_row[j]))) & 0xFFu;
            v8bf wq[4];
            expand_fp4(wf[P][j], sb, wq);
#pragma unroll
            for(int mt = 0; mt < MT; mt++)
#pragma unroll
                for(int i = 0; i < 4; i++)
                    acc[j][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wq[i], __builtin_bit_cast(v8bf, af[P][mt][i]),
                                                                       acc[j][mt], 0, 0, 0);
        }
    };
    const int kt0 = SPLITK ? wave : 0;
    if constexpr(NB == 3)
    {
        // ring of three: a register set is refilled, three K-steps of this wave ahead, as soon as its MFMAs are issued
        using B0 = std::integral_constant<int, 0>;
        using B1 = std::integral_constant<int, 1>;
        using B2 = std::integral_constant<int, 2>;
        load_step(B0{}, kt0);
        if(kt0 + KSTRIDE < KT)
            load_step(B1{}, kt0 + KSTRIDE);
        if(kt0 + 2 * KSTRIDE < KT)
            load_step(B2{}, kt0 + 2 * KSTRIDE);
        auto ring_step = [&](auto BB, int kt) __attribute__((always_inline)) {
            mfma_step(BB, kt);
            if(kt + 3 * KSTRIDE < KT)
                load_step(BB, kt + 3 * KSTRIDE);
        };
        for(int kt = kt0; kt < KT; kt += 3 * KSTRIDE)
        {
            ring_step(B0{}, kt);
            if(kt + KSTRIDE < KT)
                ring_step(B1{}, kt + KSTRIDE);
            if(kt + 2 * KSTRIDE < KT)
                ring_step(B2{}, kt + 2 * KSTRIDE);
        }
    }
    else
    {
        // one K-step from register set P while the next one loads into set 1 - P (K / 128 is even)
        auto k_step = [&](auto PP, int kt) __attribute__((always_inline)) {
            constexpr int P = decltype(PP)::value;
            if(kt + KSTRIDE < KT)
                load_step(std::integral_constant<int, 1 - P>{}, kt + KSTRIDE);
            mfma_step(PP, kt);
        };
        load_step(std::integral_constant<int, 0>{}, kt0);
        for(int kt = kt0; kt < KT; kt += 2 * KSTRIDE)
        {
            k_step(std::integral_constant<int, 0>{}, kt);
            if(kt + KSTRIDE < KT)                                          // a wave's share of K-steps may be odd
                k_step(std::integral_constant<int, 1>{}, kt + KSTRIDE);
        }
    }
    // which row groups this wave finishes: all four of its own, or (split K) the w-th of the shared ones
    // (stage 1: gate group w and its up group w + 2, waves 0 and 1 only)
    if(SPLITK)
    {
#pragma unroll
        for(int j = 0; j < RG; j++)
#pragma unroll
            for(int mt = 0; mt < MT; mt++)
                *(v4f*)&red[(((wave * RG + j) * MT + mt) * WAVE + lane) * 4] = acc[j][mt];
        __syncthreads();
        if(wave >= (STAGE == 1 ? 2 : RG))
            return;
#pragma unroll
        for(int j = 0; j < RG; j++)
#pragma unroll
            for(int mt = 0; mt < MT; mt++)
            {
                v4f sum = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for(int w = 0; w < NW; w++)
                    sum += *(const v4f*)&red[(((w * RG + j) * MT + mt) * WAVE + lane) * 4];
                acc[j][mt] = sum;
            }
    }
    auto mine = [&](int j) __attribute__((always_inline)) {
        return !SPLITK || (STAGE == 1 ? (j & 1) == wave : j == wave);
    };

    // ---- epilogue: lane (r, kb) holds channels kb*4 .. kb*4+3 of row group j for token row r
    if(g.bias)
    {
#pragma unroll
        for(int j = 0; j < RG; j++)
#pragma unroll
            for(int i = 0; i < 4; i++)
            {
                const int ch = STAGE == 1 ? (j >> 1) * I + chbase + (j & 1) * 16 + kb * 4 + i
                                          : chbase + j * 16 + kb * 4 + i;
                const float b = bf16_bits_to_f32(g.bias[(size_t)e * g.N + ch]);
#pragma unroll
                for(int mt = 0; mt < MT; mt++)
                    acc[j][mt][i] += b;
            }
    }
#pragma unroll
    for(int mt = 0; mt < MT; mt++)
    {
        const int p = m_blk * BM + mt * 16 + r;
        if constexpr(STAGE == 1)
        {
#pragma unroll
            for(int j = 0; j < 2; j++)
            {
                if(!mine(j))
                    continue;
                float v[4];
#pragma unroll
                for(int i = 0; i < 4; i++)
                    v[i] = ok[mt] ? gated_act_f32(g.act, acc[j][mt][i], acc[j + 2][mt][i]) : 0.f;
                uint2 o = make_uint2(pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3]));
                *(uint2*)(g.out + (size_t)p * I + chbase + j * 16 + kb * 4) = o;
            }
        }
        else if(ok[mt])
        {
            const int tok = (int)(ids[mt] & 0xFFFFFFu), slot = (int)(ids[mt] >> 24);
            const float rw = one_token ? g.token_w[m_blk] : g.sorted_w[p];
#pragma unroll
            for(int j = 0; j < RG; j++)
            {
                if(!mine(j))
                    continue;
                uint2 o = make_uint2(pack_bf16x2(acc[j][mt][0] * rw, acc[j][mt][1] * rw),
                                     pack_bf16x2(acc[j][mt][2] * rw, acc[j][mt][3] * rw));
                *(uint2*)(g.out + ((size_t)tok * g.topk + slot) * g.N + chbase + j * 16 + kb * 4) = o;
            }
        }
    }
}

// split_k: 0 = decide here, 1 = never, 4 / 16 = always that many waves per 64-row tile, 32 = sixteen waves per 32-row
// tile with three K-steps in flight (down GEMM; the gate_up GEMM takes 16 instead)
template <int STAGE>
static int launch_w4a16(W4A16Args g, int block_m, int64_t n_blk, int64_t rows, int experts, int split_k,
                        hipStream_t stream)
{
    // upper bound of the row blocks that hold rows: one per routed row, and one partly filled block per expert
    int64_t blocks = rows < n_blk ? rows : n_blk;
    if(experts + rows / block_m < blocks)
        blocks = experts + rows / block_m;
    int split = split_k == 1 ? 0 : split_k;
    if(STAGE == 1 && split == 32)       // (the 32-row tile exists for the down GEMM: gate_up takes sixteen waves, or four)
        split = g.K >= 2048 ? 16 : 4;
    if(split_k == 0 && blocks * g.n_tiles < 2048)
        // sixteen waves when the four-way split would still start fewer workgroups than there are CUs and the K loop
        // is long enough to matter (Mixtral shape, one token: the layer 54.0 -> 49.7 us; forced onto the gate_up GEMM as well,
        // which already starts 896 workgroups there, 57.5 us)
        // (the down GEMM then takes the sixteen-wave split on 32-row tiles with three K-steps in flight, split 32:
        // Mixtral shape, one token, the down GEMM 16.9 -> see the measurements in the kernel's comment)
        split = (blocks * g.n_tiles * 4 < 256 && g.K >= 8192 && block_m == 16) ? (STAGE == 2 ? 32 : 16) : 4;
    // (sixteen waves of a workgroup share the register file four to a SIMD: 128 registers each, which only the 16-row
    // tile fits into; and every wave needs a K-step of its own)
    if(split >= 16 && (g.K < 2048 || block_m != 16))
    {
        pyhip_set_error("moe_gemm_w4a16: split_k=16 / 32 need K >= 2048 and block_m = 16 (K=%d, block_m=%d)", g.K, block_m);
        return PYHIP_ERR_INVALID;
    }
    if(split)
        g.n_tiles *= split == 32 ? 8 : 4;
    // blocks past the bound cannot hold rows (the sort fills blocks from 0 upwards): no workgroups for them
    dim3 grid((unsigned)(blocks * g.n_tiles)), block(split >= 16 ? 1024 : W4A16_THREADS);
    if constexpr(STAGE == 2)
        if(split == 32)
        {
            hipLaunchKernelGGL((moe_gemm_w4a16_kernel<2, 1, 32>), grid, block, 0, stream, g);
            PYHIP_CHECK_LAUNCH("moe_gemm_w4a16_kernel");
            return PYHIP_OK;
        }
#define W4A16_CASE(BMV, MTV, SPV) \
    case BMV * 32 + SPV: hipLaunchKernelGGL((moe_gemm_w4a16_kernel<STAGE, MTV, SPV>), grid, block, 0, stream, g); break;
    switch(block_m * 32 + split)
    {
        W4A16_CASE(16, 1, 0) W4A16_CASE(16, 1, 4) W4A16_CASE(16, 1, 16)
        W4A16_CASE(32, 2, 0) W4A16_CASE(32, 2, 4)
        W4A16_CASE(64, 4, 0) W4A16_CASE(64, 4, 4)
    default: pyhip_set_error("moe_gemm_w4a16: block_m=%d not in {16,32,64}", block_m); return PYHIP_ERR_INVALID;
    }
#undef W4A16_CASE
    PYHIP_CHECK_LAUNCH("moe_gemm_w4a16_kernel");
    return PYHIP_OK;
}

static int check_w4a16(const char* name, const void* a, const void* w, const void* w_s, const void* sorted_ids,
                       const void* sorted_e, const void* num_valid, const void* out, int K, int block_m,
                       int64_t n_blk, int64_t n_tiles)
{
    PYHIP_REQUIRE(a && w && w_s && sorted_ids && sorted_e && num_valid && out, "%s: null pointer", name);
    PYHIP_REQUIRE(K > 0 && K % 512 == 0, "%s: K=%d must be a positive multiple of 512", name, K);
    PYHIP_REQUIRE(block_m == 16 || block_m == 32 || block_m == 64, "%s: block_m=%d not in {16,32,64}", name, block_m);
    PYHIP_REQUIRE(n_blk >= 0 && n_blk * n_tiles * 4 < (1ll << 31), "%s: n_blk=%lld", name, (long long)n_blk);
    PYHIP_REQUIRE(((uintptr_t)a % 16) == 0 && ((uintptr_t)w % 16) == 0 && ((uintptr_t)w_s % 4) == 0 &&
                      ((uintptr_t)out % 8) == 0,
                  "%s: unaligned pointer", name);
    return PYHIP_OK;
}

extern "C" int pyhip_moe_gemm1_w4a16(const void* hidden_bf16, const uint8_t* w1, const uint8_t* w1_scale,
                                     const void* bias1_bf16, const uint32_t* sorted_ids,
                                     const uint32_t* sorted_expert_ids, const uint32_t* num_valid_ids, void* a2_bf16,
                                     int tokens, int topk, int experts, int hidden, int inter, int block_m,
                                     int64_t n_blk, int split_k, int activation, float swiglu_limit,
                                     hipStream_t stream)
{
    PYHIP_REQUIRE(split_k == 0 || split_k == 1 || split_k == 4 || split_k == 16 || split_k == 32, "moe_gemm1_w4a16: split_k=%d not in {0,1,4,16,32}", split_k);
    PYHIP_REQUIRE(activation == 0 || (activation == 1 && swiglu_limit > 0.f),
                  "moe_gemm1_w4a16: activation=%d (0 SiLU, 1 SwiGLU with a positive limit)", activation);
    int rc = check_w4a16("moe_gemm1_w4a16", hidden_bf16, w1, w1_scale, sorted_ids, sorted_expert_ids, num_valid_ids,
                         a2_bf16, hidden, block_m, n_blk, inter / 128);
    if(rc)
        return rc;
    PYHIP_REQUIRE(inter > 0 && inter % 128 == 0, "moe_gemm1_w4a16: inter=%d must be a multiple of 128", inter);
    PYHIP_REQUIRE(tokens > 0 && topk > 0 && experts > 0, "moe_gemm1_w4a16: bad sizes");
    if(n_blk == 0)
        return PYHIP_OK;
    W4A16Args g;
    g.a = (const uint16_t*)hidden_bf16; g.w = w1; g.w_s = w1_scale; g.bias = (const uint16_t*)bias1_bf16;
    g.sorted_ids = sorted_ids; g.sorted_w = nullptr; g.sorted_e = sorted_expert_ids; g.num_valid = num_valid_ids;
    g.out = (uint16_t*)a2_bf16; g.T = tokens; g.topk = topk; g.K = hidden; g.N = 2 * inter;
    g.SC = (hidden / 32 + 7) / 8 * 8; g.n_tiles = inter / 128;
    g.act = make_gated_act(activation, swiglu_limit);
    return launch_w4a16<1>(g, block_m, n_blk, (int64_t)tokens * topk, experts, split_k, stream);
}

// The two GEMMs for a single token without the routing sort: the kernels read topk_ids / topk_weights themselves, one
// 16-row block per slot (the rows of a2 and the blocks are those a sort with block_size 16 would produce when every
// slot has an expert of its own: a2 bf16 [topk * 16, inter], row slot * 16).  Slots the sort would drop (expert id outside
// [0, experts), masked expert, num_local_tokens < 1) are left out; their out3 rows keep what the buffer held, as
// with the sorted entry points.  One launch fewer on the critical path of single-token decode, where the sort's 6 us
// are an eighth of the layer.  Results are those of the sorted entry points, bit for bit.
extern "C" int pyhip_moe_gemm1_w4a16_token(const void* hidden_bf16, const uint8_t* w1, const uint8_t* w1_scale,
                                           const void* bias1_bf16, const int32_t* topk_ids, const int32_t* expert_mask,
                                           const int32_t* num_local_tokens, void* a2_bf16, int topk, int experts,
                                           int hidden, int inter, int split_k, int activation, float swiglu_limit,
                                           hipStream_t stream)
{
    PYHIP_REQUIRE(split_k == 0 || split_k == 1 || split_k == 4 || split_k == 16 || split_k == 32, "moe_gemm1_w4a16_token: split_k=%d not in {0,1,4,16,32}", split_k);
    PYHIP_REQUIRE(activation == 0 || (activation == 1 && swiglu_limit > 0.f),
                  "moe_gemm1_w4a16_token: activation=%d (0 SiLU, 1 SwiGLU with a positive limit)", activation);
    PYHIP_REQUIRE(hidden_bf16 && w1 && w1_scale && topk_ids && a2_bf16, "moe_gemm1_w4a16_token: null pointer");
    PYHIP_REQUIRE(hidden > 0 && hidden % 512 == 0 && inter > 0 && inter % 128 == 0,
                  "moe_gemm1_w4a16_token: hidden=%d must be a multiple of 512, inter=%d of 128", hidden, inter);
    PYHIP_REQUIRE(topk > 0 && topk < 256 && experts > 0, "moe_gemm1_w4a16_token: bad sizes");
    PYHIP_REQUIRE(((uintptr_t)hidden_bf16 % 16) == 0 && ((uintptr_t)w1 % 16) == 0 && ((uintptr_t)w1_scale % 4) == 0 &&
                      ((uintptr_t)a2_bf16 % 8) == 0,
                  "moe_gemm1_w4a16_token: unaligned pointer");
    W4A16Args g;
    g.a = (const uint16_t*)hidden_bf16; g.w = w1; g.w_s = w1_scale; g.bias = (const uint16_t*)bias1_bf16;
    g.sorted_ids = nullptr; g.sorted_w = nullptr; g.sorted_e = nullptr; g.num_valid = nullptr;
    g.out = (uint16_t*)a2_bf16; g.T = 1; g.topk = topk; g.K = hidden; g.N = 2 * inter;
    g.SC = (hidden / 32 + 7) / 8 * 8; g.n_tiles = inter / 128;
    g.act = make_gated_act(activation, swiglu_limit);
    g.token_ids = topk_ids; g.expert_mask = expert_mask; g.num_local_tok = num_local_tokens; g.experts = experts;
    return launch_w4a16<1>(g, 16, topk, topk, experts, split_k, stream);
}

extern "C" int pyhip_moe_gemm2_w4a16_token(const void* a2_bf16, const uint8_t* w2, const uint8_t* w2_scale,
                                           const void* bias2_bf16, const int32_t* topk_ids, const float* topk_weights,
                                           const int32_t* expert_mask, const int32_t* num_local_tokens, void* out3_bf16,
                                           int topk, int experts, int hidden, int inter, int split_k, hipStream_t stream)
{
    PYHIP_REQUIRE(split_k == 0 || split_k == 1 || split_k == 4 || split_k == 16 || split_k == 32, "moe_gemm2_w4a16_token: split_k=%d not in {0,1,4,16,32}", split_k);
    PYHIP_REQUIRE(a2_bf16 && w2 && w2_scale && topk_ids && topk_weights && out3_bf16, "moe_gemm2_w4a16_token: null pointer");
    PYHIP_REQUIRE(inter > 0 && inter % 512 == 0 && hidden > 0 && hidden % 256 == 0,
                  "moe_gemm2_w4a16_token: inter=%d must be a multiple of 512, hidden=%d of 256", inter, hidden);
    PYHIP_REQUIRE(topk > 0 && topk < 256 && experts > 0, "moe_gemm2_w4a16_token: bad sizes");
    PYHIP_REQUIRE(((uintptr_t)a2_bf16 % 16) == 0 && ((uintptr_t)w2 % 16) == 0 && ((uintptr_t)w2_scale % 4) == 0 &&
                      ((uintptr_t)out3_bf16 % 8) == 0,
                  "moe_gemm2_w4a16_token: unaligned pointer");
    W4A16Args g;
    g.a = (const uint16_t*)a2_bf16; g.w = w2; g.w_s = w2_scale; g.bias = (const uint16_t*)bias2_bf16;
    g.sorted_ids = nullptr; g.sorted_w = nullptr; g.sorted_e = nullptr; g.num_valid = nullptr;
    g.out = (uint16_t*)out3_bf16; g.T = 1; g.topk = topk; g.K = inter;
    g.N = hidden; g.SC = (inter / 32 + 7) / 8 * 8; g.n_tiles = hidden / 256;
    g.act = make_gated_act(0, 0.f);
    g.token_ids = topk_ids; g.token_w = topk_weights; g.expert_mask = expert_mask; g.num_local_tok = num_local_tokens;
    g.experts = experts;
    return launch_w4a16<2>(g, 16, topk, topk, experts, split_k, stream);
}

extern "C" int pyhip_moe_gemm2_w4a16(const void* a2_bf16, const uint8_t* w2, const uint8_t* w2_scale,
                                     const void* bias2_bf16, const uint32_t* sorted_ids, const float* sorted_weights,
                                     const uint32_t* sorted_expert_ids, const uint32_t* num_valid_ids, void* out3_bf16,
                                     int tokens, int topk, int experts, int hidden, int inter, int block_m,
                                     int64_t n_blk, int split_k, hipStream_t stream)
{
    PYHIP_REQUIRE(split_k == 0 || split_k == 1 || split_k == 4 || split_k == 16 || split_k == 32, "moe_gemm2_w4a16: split_k=%d not in {0,1,4,16,32}", split_k);
    int rc = check_w4a16("moe_gemm2_w4a16", a2_bf16, w2, w2_scale, sorted_ids, sorted_expert_ids, num_valid_ids,
                         out3_bf16, inter, block_m, n_blk, hidden / 256);
    if(rc)
        return rc;
    PYHIP_REQUIRE(sorted_weights, "moe_gemm2_w4a16: null sorted_weights");
    PYHIP_REQUIRE(hidden > 0 && hidden % 256 == 0, "moe_gemm2_w4a16: hidden=%d must be a multiple of 256", hidden);
    PYHIP_REQUIRE(tokens > 0 && topk > 0 && experts > 0, "moe_gemm2_w4a16: bad sizes");
    if(n_blk == 0)
        return PYHIP_OK;
    W4A16Args g;
    g.a = (const uint16_t*)a2_bf16; g.w = w2; g.w_s = w2_scale; g.bias = (const uint16_t*)bias2_bf16;
    g.sorted_ids = sorted_ids; g.sorted_w = sorted_weights; g.sorted_e = sorted_expert_ids;
    g.num_valid = num_valid_ids; g.out = (uint16_t*)out3_bf16; g.T = tokens; g.topk = topk; g.K = inter;
    g.N = hidden; g.SC = (inter / 32 + 7) / 8 * 8; g.n_tiles = hidden / 256;
    g.act = make_gated_act(0, 0.f);
    return launch_w4a16<2>(g, block_m, n_blk, (int64_t)tokens * topk, experts, split_k, stream);
}
