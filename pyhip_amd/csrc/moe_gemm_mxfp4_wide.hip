// The 256-row tile of the MXFP4 x MXFP4 grouped GEMMs with BOTH operands staged through LDS: eight waves, one
// workgroup per CU, a tile of 256 sorted rows x 256 weight rows.  (The reference's prefill kernel has this shape:
// src/contrib/moe_gemm_mxfp4.py:318-637, an eight-wave 256 x 256 tile whose two groups of four waves alternate between
// loading and computing.)  Same contract, same argument block, same epilogues as the four-wave kernels in
// moe_gemm_mxfp4.hip; what differs is how the operands reach the matrix pipeline.
//
// Waves.  wave = wr * 4 + wc: wave column wc owns 64 of the tile's weight rows (stage 1: 32 gate rows and the matching 32
// up rows), wave row wr owns 128 of the tile's rows (8 row groups of 16).  A wave therefore has the same 4 x 8 accumulator
// tiles, in the same hand-numbered accumulation registers, as a wave of the 128-row kernel, and two waves share a SIMD.
//
// Operands.  Per K-step (128 K elements) the workgroup needs 16 weight tiles and 16 activation tiles of 1 KB.  All 32 are
// brought by LDS-DMA (buffer_load ... lds), four per wave: a pre-shuffled weight tile is 1 KB contiguous in memory and
// lands in operand order; an activation tile is gathered row by row, 64 contiguous bytes per four lanes, into the
// XOR-swizzled row-major block that the 128-row kernel uses.  Every weight tile is read by the two waves of its column,
// every activation tile by the four waves of its row: 128 B per MFMA pass through the CU's vector-memory path where the
// 128-row kernel moves 192 B, and a weight tile has one reader per 256 rows instead of one per 128.
//
// Pipeline.  LDS holds a ring of five one-K-step stages of weight tiles and a ring of three of activation tiles: while
// K-step n is computed, the weight tiles of K-step n+4 (they come from HBM) and the activation tiles of K-step n+2 (they
// come from the L2, which 16 workgroups read them through) are on their way, each into the stage that K-step n-1 has
// just left.  The wave rows run half a K-step apart: every wave meets every barrier, two per K-step, but a wave row
// starts a K-step (the point where it has nothing read from LDS yet) while the other is in the middle of one, so a SIMD
// always holds one wave with operands in registers.  Row 0 issues its vector-memory operations in the second half of
// its K-step, row 1 in the first half of its own: both fall between the same two barriers, after the last reader of the
// stages they overwrite.  The wait for the data of the next K-step is made by all waves at the barrier at which row 0
// starts that K-step.
//
// Measured (DeepSeek-V3 shape, 6144 tokens, every expert one 256-row block; whole layer): 1.86 ms against 1.70 ms for the
// four-wave 256-row tile of moe_gemm_mxfp4.hip, with the same HBM traffic (4.2 GB per gate_up launch, the algorithmic
// amount).  Taking things away from this kernel: no barriers 1.84; weights of one expert only (cache hits) 1.64; no
// weight fetches 1.49; no fetches and no barriers 1.12.  The kernel is therefore not the default for any launch; it is
// reached through pyhip_moe_gemm1_mxfp4_lds / pyhip_moe_gemm2_mxfp4_lds.
#include "gemm_device.h"

#define WIDE_THREADS 512
#define WIDE_BM 256
#define WIDE_E_MAX 512      // experts whose schedule (row-block prefixes, local ids) fits next to the stages

// all but the N youngest vector-memory operations have completed (the weight-scale registers named are (re)defined here,
// so their consumers cannot be scheduled above the wait), optionally the wave's own LDS reads too, then the barrier
template <int N, bool LGKM>
__device__ __forceinline__ void wide_wait_barrier(int& a, int& b, int& c, int& d)
{
    if(LGKM)
        asm volatile("s_waitcnt vmcnt(%4) lgkmcnt(0)\n\ts_barrier" : "+v"(a), "+v"(b), "+v"(c), "+v"(d) : "n"(N) : "memory");
    else
        asm volatile("s_waitcnt vmcnt(%4)\n\ts_barrier" : "+v"(a), "+v"(b), "+v"(c), "+v"(d) : "n"(N) : "memory");
}
template <bool LGKM>
__device__ __forceinline__ void wide_barrier()
{
    if(LGKM)
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    else
        asm volatile("s_barrier" ::: "memory");
}

// STAGE 1 = gate_up, 2 = down; ACT as in moe_gemm_mxfp4_kernel
template <int STAGE, int ACT>
__global__ void __launch_bounds__(WIDE_THREADS) moe_gemm_mxfp4_wide_kernel(GemmArgs g)
{
#if defined(__HIP_DEVICE_COMPILE__)   // the host pass only needs the launch stub
    constexpr int MT   = 8;           // row groups per wave
    constexpr int BM   = WIDE_BM;
    constexpr int NG   = BM / 16;     // row groups per tile
    constexpr int NID  = BM / 64;     // DMA operations that bring one tile's sorted ids (same for the routing weights)
    constexpr int MPAD = BM;          // words per meta array
    asm volatile("" ::: "a0", "a127");   // the accumulators, named by hand in mfma_row_group
    constexpr int RW = 5, RA = 3;     // LDS stages (one K-step each) of the weight ring and of the activation ring
    constexpr int WST = 16 * 1024, AST = NG * 1024;                         // bytes of a stage
    __shared__ __attribute__((aligned(16))) uint8_t lds_w[RW][WST];         // [stage][weight tile wc*4+j][1 KB]
    __shared__ __attribute__((aligned(16))) uint8_t lds_a[RA][AST];         // [stage][row group][1 KB]
    __shared__ __attribute__((aligned(16))) uint8_t lds_s[2][NG * 256];     // activation scales of a K-group [parity]
    __shared__ u32 lds_meta[3][2 * MPAD];     // per tile: sorted ids | routing weights; ring of 3 tiles
    __shared__ __attribute__((aligned(16))) u32 lds_dummy[256];   // where switched-off DMA operations put their zeros
    __shared__ u32 lds_pre[WIDE_E_MAX + 1];   // the schedule: row blocks before every expert (and their total),
    __shared__ u32 lds_lid[WIDE_E_MAX];       //   local id of every expert

    const int tid  = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid / WAVE);
    const int lane = tid % WAVE;
    const int wc = wave & 3, wr = wave >> 2;
    const int r = lane & 15, kb = lane >> 4;
    const int Kb = g.K / 2;
    const int KS = g.K / 512;
    const int I  = g.N / 2;   // stage 1 only

    // ---- tile iterator: the persistent schedule of moe_gemm_mxfp4_kernel (tiles ordered expert -> weight tile -> row
    // block, cut into 8 equal runs, workgroup w serves XCD w % 8 and walks its run with stride gridDim / 8)
    const int xcd     = blockIdx.x & 7;
    const u32 qstride = gridDim.x >> 3;
    u32 q             = blockIdx.x >> 3;
    u32 q_end         = 0;
    int ei            = 0;
    for(int i = tid; i <= g.E; i += WIDE_THREADS)
    {
        lds_pre[i] = g.sched[i];
        if(i < g.E)
            lds_lid[i] = g.sched[g.E + 1 + i];
    }
    __syncthreads();
    auto uni = [](u32 v) __attribute__((always_inline)) { return (u32)__builtin_amdgcn_readfirstlane((int)v); };
    auto uni4 = [](v4i v) __attribute__((always_inline)) {
        return (v4i){__builtin_amdgcn_readfirstlane(v.x), __builtin_amdgcn_readfirstlane(v.y),
                     __builtin_amdgcn_readfirstlane(v.z), __builtin_amdgcn_readfirstlane(v.w)};
    };
    {
        const u32 tiles = uni(lds_pre[g.E]) * (u32)g.n_tiles;
        const u32 chunk = (tiles + 7u) >> 3;
        q += (u32)xcd * chunk;
        q_end = (u32)(xcd + 1) * chunk < tiles ? (u32)(xcd + 1) * chunk : tiles;
        if(q < q_end)
        {
            int lo = 0, hi = g.E - 1;
            while(lo < hi)
            {
                const int mid = (lo + hi) >> 1;
                if(uni(lds_pre[mid + 1]) * (u32)g.n_tiles > q)
                    hi = mid;
                else
                    lo = mid + 1;
            }
            ei = lo;
        }
    }
    auto decode = [&](TileId& t) __attribute__((always_inline)) {
        t.valid = false;
        if(q >= q_end)
            return;
        while(q >= uni(lds_pre[ei + 1]) * (u32)g.n_tiles)
            ei++;
        const u32 p0    = uni(lds_pre[ei]);
        const u32 nb    = uni(lds_pre[ei + 1]) - p0;
        const u32 local = q - p0 * (u32)g.n_tiles;
        t.nt            = (int)(local / nb);
        t.m_blk         = (int)(p0 + (local - (u32)t.nt * nb));
        t.e             = (int)uni(lds_lid[ei]);
        q += qstride;
        t.valid = true;
    };

    // ---- load side.  `_p`: descriptors and lane offsets of the K-group that is being prefetched (the next one of this
    // tile, or the first one of the workgroup's next tile): every weight DMA uses them (weights run a whole K-group
    // ahead).  The activation DMAs run two K-steps ahead, so those of K-steps 2 and 3 of a K-group still belong to the
    // tile being computed: its lane offsets are kept in `a_c`.  A tile that does not exist is prefetched with offsets
    // beyond every buffer: the hardware drops the accesses, the instruction stream stays the same.
    constexpr u32 OOB = 0xFFFF0000u;
    const int dma_row   = lane >> 2;
    const int dma_chunk = (lane & 3) ^ ((lane >> 3) & 3);
    const int rd_a      = r * 64 + ((kb ^ ((r >> 1) & 3)) * 16);   // operand read offset inside a 1 KB activation block
    const int rd_s      = (r * 4 + kb) * 4;                        // scale dword read offset inside a 256 B block
    v4i wd_p[2];                // this wave's two weight tiles per K-step: tile t = wave + 8*s = (column t/4, group t%4)
    int wv_p;                   // lane offset inside a weight tile (lane * 16, or OOB)
    v4i wsd[2];                 // scale tiles of the wave column's weight rows (prefetched K-group)
    int wsv;                    // lane offset inside them (lane * 4, or OOB)
    int a_c[2], a_p[2], as_p[2];   // this wave's two activation row groups g = wave + 8*s: lane offsets in a_q / a_s
    const v4i ars  = make_rsrc(g.a_q, (u32)((size_t)g.a_rows * Kb));
    const v4i asrs = make_rsrc(g.a_s, (u32)((size_t)g.a_rows * g.SK));
    const int ws_half = (STAGE == 2) ? (g.SC / 8) * 256 : 0;
    auto setup_pre_null = [&]() __attribute__((always_inline)) {
        wv_p = wsv = (int)OOB;
        a_p[0] = a_p[1] = as_p[0] = as_p[1] = (int)OOB;
    };
    // ids: the tile's sorted ids, in LDS (meta ring) or in global memory
    auto setup_pre = [&](const TileId& t, const u32* ids) __attribute__((always_inline)) {
        const size_t sc_tile = (size_t)(g.SC / 8) * 256;           // bytes of one 32-row scale tile
#pragma unroll
        for(int s = 0; s < 2; s++)
        {
            const int tt = wave + 8 * s, c = tt >> 2, j = tt & 3;
            const size_t row = STAGE == 1 ? (size_t)t.e * g.N + (j >> 1) * I + t.nt * 128 + c * 32 + (j & 1) * 16
                                          : (size_t)t.e * g.N + t.nt * 256 + c * 64 + j * 16;
            wd_p[s] = make_rsrc(g.w + row * Kb, (u32)(16 * Kb));
        }
        wv_p = lane * 16;
        if(STAGE == 1)
        {
#pragma unroll
            for(int h = 0; h < 2; h++)
            {
                const size_t row = (size_t)t.e * g.N + h * I + t.nt * 128 + wc * 32;
                wsd[h]           = make_rsrc(g.w_s + (row / 32) * sc_tile, (u32)sc_tile);
            }
        }
        else
        {
            const size_t row = (size_t)t.e * g.N + t.nt * 256 + wc * 64;
            wsd[0] = wsd[1] = make_rsrc(g.w_s + (row / 32) * sc_tile, (u32)(2 * sc_tile));
        }
        wsv = lane * 4;
#pragma unroll
        for(int s = 0; s < 2; s++)
        {
            const int gi  = wave + 8 * s;
            const u32 id  = ids[gi * 16 + dma_row];
            const int tok = (int)(id & 0xFFFFFFu);
            int row       = -1;                     // padding rows fetch nothing
            if((int)(id >> 24) < g.topk && tok < g.T)
                row = STAGE == 1 ? tok : t.m_blk * BM + gi * 16 + dma_row;
            a_p[s]  = row < 0 ? (int)OOB : row * Kb + dma_chunk * 16;
            as_p[s] = row < 0 ? (int)OOB : row * g.SK + (lane & 3) * 4;
        }
    };
    auto take_pre = [&]() __attribute__((always_inline)) {
        a_c[0] = a_p[0]; a_c[1] = a_p[1];
    };
    // row groups of a tile that hold at least one real row (the sort pads at the end of a block: a prefix)
    auto count_groups = [&](const u32* ids) __attribute__((always_inline)) -> int {
        const u32 id  = ids[(lane < NG ? lane : 0) * 16];
        const bool ok = lane < NG && (int)(id >> 24) < g.topk && (int)(id & 0xFFFFFFu) < g.T;
        return __builtin_popcountll(__ballot(ok));
    };

    const u32 ldsw0 = lds_addr_of(&lds_w[0][0]), ldsa0 = lds_addr_of(&lds_a[0][0]), ldss0 = lds_addr_of(&lds_s[0][0]);
    // Operand DMAs of one K-step, two per wave and operand, into the ring stage with index st (wave-uniform, run time):
    // weights of K-step kt of the prefetched K-group's tile (non-temporal: a weight tile has this one reader), activations
    // of K-step kt with the given lane offsets
    auto dma_w = [&](auto OP, int st, int kt) __attribute__((always_inline)) {
        constexpr int op = decltype(OP)::value;
        vm_dma_b128<0, op * 8 * 1024, true>(wv_p, wd_p[op], kt * 1024, ldsw0 + (u32)(st * WST + wave * 1024));
    };
    auto dma_a = [&](auto OP, int st, const int (&ao)[2], int kt) __attribute__((always_inline)) {
        constexpr int op = decltype(OP)::value;
        vm_dma_b128<0, op * 8 * 1024>(ao[op], ars, kt * 64, ldsa0 + (u32)(st * AST + wave * 1024));
    };
    int w_sc[4], w_sc_nxt[4];  // weight-scale dwords of the K-group being computed / prefetched
    int par = 0;               // activation-scale stage of the K-group being computed
    // the operations a wave issues once per K-group, for the K-group kpre that is prefetched: 1 of the 8 that bring the
    // next tile's sorted ids and routing weights (first K-group of a tile only), the scales of its 2 activation row
    // groups, the 4 scale dwords of its weight rows
    constexpr int NGRP = 7;
    auto group_op = [&](auto OP, int kpre, bool meta_on, const TileId& mt_tile, int mb_dst) __attribute__((always_inline)) {
        constexpr int op = decltype(OP)::value;
        if constexpr(op == 0)
        {
            const bool wts  = wave >= NID;
            const int oo    = wts ? wave - NID : wave;
            const bool real = meta_on && (!wts || g.sorted_w != nullptr);
            const v4i rid   = make_rsrc(g.sorted_ids + (size_t)mt_tile.m_blk * BM, BM * 4);
            const v4i rwt   = make_rsrc(g.sorted_w + (size_t)mt_tile.m_blk * BM, BM * 4);
            const v4i rs    = uni4(real ? (wts ? rwt : rid) : make_rsrc(g.sorted_ids, 0));
            const u32 dst   = uni(real ? lds_addr_of(&lds_meta[mb_dst][(wts ? MPAD : 0) + oo * 64]) : lds_addr_of(lds_dummy));
            vm_dma_b32_fresh_sgprs((oo * 64 + lane) * 4, rs, dst);
        }
        else if constexpr(op < 3)
            vm_dma_b32<0, (op - 1) * 8 * 256>(as_p[op - 1], asrs, kpre * 16, ldss0 + (u32)((par ^ 1) * NG * 256 + wave * 256));
        else
        {
            constexpr int h = (op - 3) / 2, c = (op - 3) % 2;
            vm_load_b32<0>(w_sc_nxt[h * 2 + c], wsv + c * 256, wsd[h], kpre * 512 + h * ws_half);
        }
    };

    // accumulators and epilogue: gemm_device.h (a wave's rows start wr * 128 rows into the tile)
    auto zero_acc = [&]() __attribute__((always_inline)) { gemm_zero_acc<MT>(); };
    auto epilogue = [&](const TileId& t, const u32* meta, int ma_t) __attribute__((always_inline)) {
        if(g.bias)
            gemm_epilogue<STAGE, MT, ACT, false, true>(g, t.e, t.nt, t.m_blk * BM + wr * MT * 16, wc, meta + wr * MT * 16, MPAD,
                                                        ma_t - wr * MT, r, kb);
        else
            gemm_epilogue<STAGE, MT, ACT, false, false>(g, t.e, t.nt, t.m_blk * BM + wr * MT * 16, wc, meta + wr * MT * 16, MPAD,
                                                         ma_t - wr * MT, r, kb);
    };

    // ---------------------------------------------------------------- pipeline
    TileId cur, nxt;
    decode(cur);
    if(!cur.valid)
        return;
    int mb = 0;
    setup_pre(cur, g.sorted_ids + (size_t)cur.m_blk * BM);
    take_pre();
    int ma     = count_groups(g.sorted_ids + (size_t)cur.m_blk * BM);
    int ma_nxt = ma;
    // prologue: this tile's ids / routing weights, scales of K-group 0 (group_op fills the stage and the registers of the
    // NEXT K-group: they change roles below), activations of K-steps 0, 1, weights of K-steps 0 .. 3
    {
        static_for<NGRP>([&](auto OP) __attribute__((always_inline)) { group_op(OP, 0, true, cur, 0); });
        static_for<RA - 1>([&](auto ST) __attribute__((always_inline)) {
            static_for<2>([&](auto OP) __attribute__((always_inline)) { dma_a(OP, decltype(ST)::value, a_c, decltype(ST)::value); });
        });
        static_for<RW - 1>([&](auto ST) __attribute__((always_inline)) {
            static_for<2>([&](auto OP) __attribute__((always_inline)) { dma_w(OP, decltype(ST)::value, decltype(ST)::value); });
        });
    }
    wide_wait_barrier<0, true>(w_sc_nxt[0], w_sc_nxt[1], w_sc_nxt[2], w_sc_nxt[3]);
    auto next_group_scales = [&]() __attribute__((always_inline)) {
#pragma unroll
        for(int i = 0; i < 4; i++)
            w_sc[i] = w_sc_nxt[i];
        par ^= 1;
    };
    next_group_scales();
    decode(nxt);
    zero_acc();
    int ks = 0;
    int iw = 0, ia = 0;        // ring stages that hold the K-step being computed
    // wave row 1 runs half a K-step behind wave row 0
    if(wr == 1)
        wide_barrier<false>();

    // one K-group (four K-steps); WR = this wave's row.  Returns false when the workgroup has no more work.
    auto kgroup = [&](auto WRR) __attribute__((always_inline)) -> bool {
        constexpr int wrow = decltype(WRR)::value;
        const bool last  = ks == KS - 1;
        const int kpre   = last ? 0 : ks + 1;
        const int mb_nxt = mb == 2 ? 0 : mb + 1;
        if(last)
        {
            if(nxt.valid)
            {
                setup_pre(nxt, lds_meta[mb_nxt]);
                ma_nxt = count_groups(lds_meta[mb_nxt]);
            }
            else
                setup_pre_null();
        }
        const bool meta_on = ks == 0 && nxt.valid;
        int asc[MT];
        static_for<4>([&](auto U) __attribute__((always_inline)) {
            constexpr int u = decltype(U)::value;
            // vector-memory operations of this K-step, in issue order: at u = 0 the NGRP operations of the K-group; then
            // the activations of the K-step two ahead (u < 2: of this K-group) and the weights of the K-step four ahead
            // (K-step u of the prefetched K-group), each into the stage its ring's previous K-step has just left
            constexpr int NOPS = u == 0 ? NGRP + 4 : 4;
            const int iw_prev = iw == 0 ? RW - 1 : iw - 1, ia_prev = ia == 0 ? RA - 1 : ia - 1;
            auto vm_op = [&](auto KK) __attribute__((always_inline)) {
                constexpr int k = decltype(KK)::value, k0 = u == 0 ? NGRP : 0;
                if constexpr(k < k0)
                    group_op(KK, kpre, meta_on, nxt, mb_nxt);
                else if constexpr(k - k0 < 2)
                {
                    if constexpr(u < 2)
                        dma_a(std::integral_constant<int, k - k0>{}, ia_prev, a_c, ks * 4 + u + 2);
                    else
                        dma_a(std::integral_constant<int, k - k0>{}, ia_prev, a_p, kpre * 4 + u - 2);
                }
                else
                    dma_w(std::integral_constant<int, k - k0 - 2>{}, iw_prev, kpre * 4 + u);
            };
            // younger than the activations of the NEXT K-step (the youngest data it needs) at the barrier where all waves
            // wait for them: the two weight operations that followed them and the operations of this K-step
            constexpr int YOUNGER = NOPS + 2;
            constexpr int PPM     = (NOPS + 3) / 4;           // operations issued after each of the four row groups
            const uint8_t* sw = &lds_w[0][0] + iw * WST + (wc * 4) * 1024 + lane * 16;
            const uint8_t* sa = &lds_a[0][0] + ia * AST + (wrow * MT) * 1024 + rd_a;
            v4i wq[4], af_r[3];
#pragma unroll
            for(int j = 0; j < 4; j++)
                wq[j] = *(const v4i*)(sw + j * 1024);
            auto lds_read = [&](auto MM) __attribute__((always_inline)) {
                constexpr int mm = decltype(MM)::value;
                af_r[mm % 3] = *(const v4i*)(sa + mm * 1024);
                if constexpr(u == 0)
                    asc[mm] = *(const int*)(&lds_s[0][0] + par * (NG * 256) + (wrow * MT + mm) * 256 + rd_s);
            };
            lds_read(std::integral_constant<int, 0>{});
            lds_read(std::integral_constant<int, 1>{});
            __builtin_amdgcn_sched_barrier(0);
            static_for<MT>([&](auto M) __attribute__((always_inline)) {
                constexpr int mt = decltype(M)::value;
                if constexpr(mt + 2 < MT)
                    lds_read(std::integral_constant<int, mt + 2>{});
                const v4i af = af_r[mt % 3];
                __builtin_amdgcn_sched_barrier(0);
                mfma_row_group<u, mt, MT>(wq[0], wq[1], wq[2], wq[3], af, w_sc[0 + (u >> 1)], w_sc[2 + (u >> 1)], asc[mt]);
                // wave row 0 issues its operations after row groups 4..7, wave row 1 after row groups 0..3
                constexpr int slot = wrow == 0 ? mt - 4 : mt;
                if constexpr(slot >= 0 && slot < 4)
                    static_for<PPM>([&](auto Q) __attribute__((always_inline)) {
                        constexpr int k = slot * PPM + decltype(Q)::value;
                        if constexpr(k < NOPS)
                            vm_op(std::integral_constant<int, k>{});
                    });
                __builtin_amdgcn_sched_barrier(0);
                if constexpr(mt == 3)
                {
                    // the barrier in the middle of this wave's K-step is the one at which the other wave row ends a K-step
                    if constexpr(wrow == 0)
                        wide_barrier<false>();
                    else
                        wide_wait_barrier<YOUNGER, false>(w_sc_nxt[0], w_sc_nxt[1], w_sc_nxt[2], w_sc_nxt[3]);
                    __builtin_amdgcn_sched_barrier(0);
                }
            });
            if constexpr(wrow == 0)
                wide_wait_barrier<YOUNGER, true>(w_sc_nxt[0], w_sc_nxt[1], w_sc_nxt[2], w_sc_nxt[3]);
            else
                wide_barrier<true>();
            iw = iw == RW - 1 ? 0 : iw + 1;
            ia = ia == RA - 1 ? 0 : ia + 1;
            __builtin_amdgcn_sched_barrier(0);
        });
        take_pre();
        next_group_scales();
        ks++;
        if(last)
        {
            // the last MFMAs were issued from assembly: give their results the documented distance to the first VALU read
            asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
            epilogue(cur, lds_meta[mb], ma);
            if(!nxt.valid)
                return false;
            cur = nxt;
            ma  = ma_nxt;
            mb  = mb_nxt;
            ks  = 0;
            zero_acc();
            decode(nxt);
        }
        return true;
    };
    if(wr == 0)
    {
        using W0 = std::integral_constant<int, 0>;
        while(kgroup(W0{}))
            ;
        wide_barrier<false>();      // the barrier at which wave row 1 ends its last K-step
    }
    else
    {
        using W1 = std::integral_constant<int, 1>;
        while(kgroup(W1{}))
            ;
    }
#endif
}

// Launch for launch_gemm (moe_gemm_mxfp4.hip).  The kernel serves layers with a schedule from the sort, at least two
// K-groups per tile and at most WIDE_E_MAX experts; -1 when it does not apply.
int pyhip_launch_gemm_wide(int stage, const GemmArgs& g, int act, hipStream_t stream)
{
    if(!g.sched || g.K < 1024 || g.E > WIDE_E_MAX)
        return -1;
    unsigned nwg            = (unsigned)(g.n_tiles * g.n_blk);
    const unsigned resident = (unsigned)device_cu_count() / 8u * 8u;
    nwg                     = nwg < resident ? (nwg + 7u) / 8u * 8u : resident;
    dim3 grid(nwg), block(WIDE_THREADS);
    if(stage == 1 && act == 1)
        hipLaunchKernelGGL((moe_gemm_mxfp4_wide_kernel<1, 1>), grid, block, 0, stream, g);
    else if(stage == 1)
        hipLaunchKernelGGL((moe_gemm_mxfp4_wide_kernel<1, 0>), grid, block, 0, stream, g);
    else
        hipLaunchKernelGGL((moe_gemm_mxfp4_wide_kernel<2, 0>), grid, block, 0, stream, g);
    PYHIP_CHECK_LAUNCH("moe_gemm_mxfp4_wide_kernel");
    return PYHIP_OK;
}
