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
// are shared by the 4 waves: they are DMA'd (buffer_load ... lds, 16 B per lane) one K-group (four
// K-steps) ahead into two LDS stages, row-major with an XOR swizzle of the 16 B chunks, so that both
// the DMA (64 contiguous bytes per four lanes) and the ds_read_b128 of an operand are at full rate.
//
// The weight tile is the MFMA's first operand and the activation tile the second, so a lane ends
// up with 4 consecutive output channels of one row (lane%16 = row, lane/16*4.. = channels).
#include "gemm_device.h"

// most experts a persistent launch can serve: the schedule (E + 1 block prefixes, E local ids) sits in LDS next to the
// activation stages, and two workgroups of the 128-row tile must still fit one CU (2 x 80 KB), three of the 16-row
// tile (40 KB each)
#define SCHED_E_MAX 704
#define SCHED_E_MAX_16 512

// STAGE 1 = gate_up, 2 = down, 3 = down with the top-k reduction done by the workgroup that stores a token's last
// slot (gemm_arrive_reduce in gemm_device.h; an option that was built to be measured against stage 2 + the reduction
// kernel, not what the layer call uses).  MT = row groups of 16 per tile.
//
// The kernel is one flat software pipeline over (tile, K-group) pairs: while the MFMAs of K-group ks of a
// tile run, the activation DMA of K-group ks+1 and the weight loads of K-steps 4(ks+1)..4(ks+1)+3 are in
// flight; in the last K-group of a tile those prefetches already belong to the workgroup's NEXT tile, so
// the memory pipeline never drains between tiles.  One barrier per K-group (512 K elements).  Everything
// a tile boundary needs (schedule tables, sorted ids, routing weights) is read from LDS, so no wait on the
// vector-memory counter ever covers the prefetches in flight.
// NT: the weight loads are marked non-temporal (the launch decides: set when nearly every expert has a single row
// block, so that no other workgroup reads the same weight tile)
// ATOMIC (down GEMM only): the epilogue adds bf16(acc * routing weight) into out[token, :] with packed bf16 atomics
// instead of storing it to out3[token, slot, :] for the top-k reduction: the reference's atomic variant
// (src/contrib/moe_gemm_mxfp4.py:1334-1398).  The sum then depends on the order in which the slots arrive.
template <int STAGE, int MT, int ACT, bool NT, bool ATOMIC = false>
__global__ void __launch_bounds__(GEMM_THREADS, (MT > 8 ? 1 : 2)) moe_gemm_mxfp4_kernel(GemmArgs g)
{
#if defined(__HIP_DEVICE_COMPILE__)   // the host pass only needs the launch stub
    constexpr int BM    = MT * 16;
    // The accumulators live in the accumulation registers a0 .. a[16*MT-1], named by hand in the instruction text
    // (mfma_row_group); the clobber reserves that range for the kernel.
    if constexpr(MT >= 16) asm volatile("" ::: "a0", "a255");
    if constexpr(MT == 12) asm volatile("" ::: "a0", "a191");
    if constexpr(MT == 10) asm volatile("" ::: "a0", "a159");
    if constexpr(MT == 8) asm volatile("" ::: "a0", "a127");
    if constexpr(MT == 4) asm volatile("" ::: "a0", "a63");
    if constexpr(MT == 2) asm volatile("" ::: "a0", "a31");
    if constexpr(MT == 1) asm volatile("" ::: "a0", "a15");
    constexpr int NA    = (MT + 3) / 4;       // activation row groups DMA'd per wave
    // The 288-row tile (MT = 18) is the largest that fits the CU at all: its two activation stages take 144 of the 160 KB
    // of LDS.  It therefore has exactly MT slots per stage (the DMA operations of the two slots that do not exist go to
    // a dummy area), a ring of two tiles' sorted ids instead of three (filled one K-group later, see meta_on), reads
    // the schedule from global memory with scalar loads instead of keeping it in LDS, and keeps the accumulator tiles
    // that the 256 accumulation registers do not hold in ordinary registers (xacc).
    constexpr bool TALL = MT == 18;
    constexpr int SLOTS = TALL ? MT : NA * 4;  // row-group slots per LDS stage (slots >= MT are never read)
    constexpr int MR    = TALL ? 2 : 3;        // tiles in the ring of sorted ids / routing weights
    constexpr int NID   = (BM + 63) / 64;     // DMA ops that bring one tile's sorted ids (same for weights)
    constexpr int MPAD  = NID * 64;           // words per meta array
    constexpr int NM    = (2 * NID + 3) / 4;  // DMA ops per wave that bring a tile's sorted ids and routing weights
    // VMEM operations per wave and K-group: NPF prefetch operations (5*NA activation, 4 weight-scale) and 16 weight
    // tiles, in the fixed order of VmSchedule (gemm_device.h), which is what the hand-counted waits rely on.  The
    // operations that bring the next tile's sorted ids are issued once per tile, ahead of a K-group's schedule, and are
    // not counted: an operation the counts do not know of only makes a wait cover more than it must.
    constexpr int NPF = 5 * NA + 4;
    // one LDS stage = the activation tile of a whole K-group (4 K-steps of 128) + its scales
    __shared__ __attribute__((aligned(16))) uint8_t lds_a0[4 * SLOTS * 1024];
    __shared__ __attribute__((aligned(16))) uint8_t lds_a1[4 * SLOTS * 1024];
    __shared__ __attribute__((aligned(16))) uint8_t lds_s0[SLOTS * 256];
    __shared__ __attribute__((aligned(16))) uint8_t lds_s1[SLOTS * 256];
    __shared__ u32 lds_meta[MR][2 * MPAD];    // per tile: sorted ids | routing weights; ring of MR tiles
    __shared__ __attribute__((aligned(16))) u32 lds_dummy[TALL ? 256 : 64];   // where switched-off DMA operations put their zeros
    constexpr int SCHED_E = TALL ? 0 : MT == 1 ? SCHED_E_MAX_16 : SCHED_E_MAX;
    __shared__ u32 lds_pre[SCHED_E + 1];      // the schedule: row blocks before every expert (and their total),
    __shared__ u32 lds_lid[SCHED_E + 1];      //   local id of every expert
    __shared__ u32 lds_tab[TALL ? 1 : 128];   // the workgroup's next 64 tiles, decoded (the 288-row tile keeps them in registers)

    const int tid  = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid / WAVE);   // wave-uniform: keeps descriptors and LDS bases scalar
    const int lane = tid % WAVE;
    const int r = lane & 15, kb = lane >> 4;
    const int Kb = g.K / 2;
    const int KS = g.K / 512;
    const int I  = g.N / 2;   // stage 1 only

    // ---- tile iterator.  With a schedule the grid is persistent.  All tiles, ordered expert -> weight tile -> row
    // block (the row blocks that share a weight tile next to each other), form one list; it is cut into 8 equal
    // runs, one per XCD, so every XCD (its own L2) gets the same number of tiles however unevenly the router loads
    // the experts, and an expert's data still meets in one L2 (two where a cut falls inside an expert).  Workgroup w
    // serves XCD w % 8 (the hardware deals consecutive workgroup ids round-robin to the XCDs) and walks that XCD's
    // run with stride gridDim/8.
    // Without a schedule (or when K has a single K-group): one tile per workgroup, weight tile fastest.
    const bool persistent = g.sched != nullptr;
    const int xcd         = blockIdx.x & 7;
    const u32 qstride     = gridDim.x >> 3;
    u32 q                 = blockIdx.x >> 3;
    u32 q_end             = 0;
    if(persistent && !TALL)
    {
        for(int i = tid; i <= g.E; i += GEMM_THREADS)
        {
            lds_pre[i] = g.sched[i];
            if(i < g.E)
                lds_lid[i] = g.sched[g.E + 1 + i];
        }
        __syncthreads();
    }
    auto uni = [](u32 v) __attribute__((always_inline)) { return (u32)__builtin_amdgcn_readfirstlane((int)v); };
    // the schedule: row blocks before expert i (i = E: their total) and the local id of expert i; from LDS, or (288-row
    // tile, which has no LDS to spare) from global memory
    auto sched_pre = [&](int i) __attribute__((always_inline)) -> u32 { return TALL ? g.sched[i] : lds_pre[i]; };
    auto sched_lid = [&](int i) __attribute__((always_inline)) -> u32 { return TALL ? g.sched[g.E + 1 + i] : lds_lid[i]; };
    auto uni4 = [](v4i v) __attribute__((always_inline)) {
        return (v4i){__builtin_amdgcn_readfirstlane(v.x), __builtin_amdgcn_readfirstlane(v.y),
                     __builtin_amdgcn_readfirstlane(v.z), __builtin_amdgcn_readfirstlane(v.w)};
    };
    // The workgroup's first 64 tiles are decoded before the pipeline starts, one per lane (a binary search over the block
    // prefixes and a division): stepping to the next tile is then two register (288-row tile: v_readlane) or LDS reads
    // instead of a dependent chain of schedule reads between two tiles, where nothing else is there to cover them.
    // (Every wave computes the same table; in LDS they overwrite each other with equal values.  The tiles up to 128 rows
    // run two workgroups per CU on 128 registers and have none to spare for it.  Tiles beyond the 64th, which only very
    // large calls have, are decoded one at a time with uniform reads of the schedule.)
    u32 tab_blk = 0xFFFFFFFFu, tab_nte = 0;       // lane i: row block and weight tile | expert << 16
    int tab_i   = 0;                              // next entry; 64: the table is used up
    int ei      = -1;                             // beyond the table: cursor into the expert list (q only grows)
    auto build_table = [&]() __attribute__((always_inline)) {
        const u32 qi = q + (u32)lane * qstride;
        tab_blk      = 0xFFFFFFFFu;
        tab_nte      = 0;
        if(qi < q_end && qi >= q)                 // (qi >= q: no wrap-around)
        {
            int lo = 0, hi = g.E - 1;             // first expert whose tiles end beyond qi
            while(lo < hi)
            {
                const int mid = (lo + hi) >> 1;
                if(sched_pre(mid + 1) * (u32)g.n_tiles > qi)
                    hi = mid;
                else
                    lo = mid + 1;
            }
            const u32 p0    = sched_pre(lo);
            const u32 nb    = sched_pre(lo + 1) - p0;
            const u32 local = qi - p0 * (u32)g.n_tiles;
            const u32 nt    = local / nb;
            tab_blk         = p0 + (local - nt * nb);
            tab_nte         = nt | (sched_lid(lo) << 16);
        }
        if constexpr(!TALL)
        {
            lds_tab[lane]      = tab_blk;
            lds_tab[64 + lane] = tab_nte;
            tab_blk = tab_nte = 0;                // (not kept in registers)
        }
    };
    if(persistent)
    {
        const u32 tiles = uni(sched_pre(g.E)) * (u32)g.n_tiles;
        const u32 chunk = (tiles + 7u) >> 3;
        // (Every workgroup of the launch takes part, also when the last round of an XCD's run is nearly empty.  Letting only
        // as many take part as make the rounds even (113 tiles on 96 workgroups: 57 with two tiles each) was measured and is
        // slower everywhere: DeepSeek-V3 shape at 16 tokens 0.379 -> 0.412 ms, Mixtral shape at 4096 tokens 0.790 -> 0.831 ms.
        // More workgroups keep more loads in flight, and that is worth more than even rounds.)
        q += (u32)xcd * chunk;
        q_end = (u32)(xcd + 1) * chunk < tiles ? (u32)(xcd + 1) * chunk : tiles;
        if(q < q_end)
            build_table();
    }
    auto decode = [&](TileId& t) __attribute__((always_inline)) {
        t.valid = false;
        if(persistent)
        {
            if(q >= q_end)
                return;
            if(tab_i < 64)
            {
                const u32 blk = TALL ? (u32)__builtin_amdgcn_readlane((int)tab_blk, tab_i) : uni(lds_tab[tab_i]);
                const u32 nte = TALL ? (u32)__builtin_amdgcn_readlane((int)tab_nte, tab_i) : uni(lds_tab[64 + tab_i]);
                tab_i++;
                t.m_blk = (int)blk;
                t.nt    = (int)(nte & 0xFFFFu);
                t.e     = (int)(nte >> 16);
            }
            else
            {
                auto pre_u = [&](int i) __attribute__((always_inline)) -> u32 {
                    typedef const __attribute__((address_space(4))) u32* sched_ptr;    // scalar loads
                    return TALL ? ((sched_ptr)(unsigned long long)g.sched)[i] : uni(lds_pre[i]);
                };
                if(ei < 0)
                    ei = 0;
                while(q >= pre_u(ei + 1) * (u32)g.n_tiles)
                    ei++;
                const u32 p0    = pre_u(ei);
                const u32 nb    = pre_u(ei + 1) - p0;
                const u32 local = q - p0 * (u32)g.n_tiles;
                t.nt            = (int)(local / nb);
                t.m_blk         = (int)(p0 + (local - (u32)t.nt * nb));
                t.e             = (int)(TALL ? pre_u(g.E + 1 + ei) : uni(lds_lid[ei]));
            }
            q += qstride;
        }
        else
        {
            if(q == 0xFFFFFFFFu)
                return;
            t.m_blk = blockIdx.x / g.n_tiles;
            t.nt    = blockIdx.x - t.m_blk * g.n_tiles;
            q       = 0xFFFFFFFFu;
            if((u32)(t.m_blk * BM) >= uni(g.num_valid[0]))
                return;
            t.e = (int)uni(g.sorted_e[t.m_blk]);
        }
        t.valid = true;
    };
    // ---- load side of the pipeline: descriptors and per-lane offsets of the tile being prefetched
    // (every prefetch is issued unconditionally; when there is no tile left to prefetch the descriptors get
    // a zero range, so the hardware drops the accesses and the instruction stream stays the same)
    v4i wrs[2];    // weight rows of this wave: stage 1 [0] gate, [1] up (2 row groups each); stage 2 [0] all 4 groups
    v4i wsrs[2];   // their scale tiles, same split (rows j = 0,1 share a 32-row scale tile, so do j = 2,3)
    // activations and their scales: the same for every tile (rows that fetch nothing carry an out-of-range offset)
    const v4i ars  = make_rsrc(g.a_q, (u32)((size_t)g.a_rows * Kb));
    const v4i asrs = make_rsrc(g.a_s, (u32)((size_t)g.a_rows * g.SK));
    int a_off[NA], as_off[NA];        // this lane's byte offsets inside a_q / a_s at K = 0, per DMA slot
    // DMA lane mapping: four consecutive lanes fetch the 64 contiguous bytes of one row and K-step (a gather
    // with one row per lane costs four times the address-pipeline cycles).  LDS therefore holds a (row group,
    // K-step) block row-major, 16 rows x 64 B; the 16 B chunk c of row r sits in slot c ^ ((r / 2) % 4), which makes
    // the operand reads (lane = K-block * 16 + row) conflict-free: measured 4 LDS cycles per ds_read_b128, against
    // 8 for c ^ (r / 4) or for no swizzle at all.
    // (Eight lanes per row, the 128 B line that a row contributes to a pair of K-steps, was built and measured as well:
    // the same time, bit-identical, and one more offset register per slot, which the 128-row tile does not have.)
    const int dma_row   = lane >> 2;
    const int dma_chunk = (lane & 3) ^ ((lane >> 3) & 3);
    const int rd_a      = r * 64 + ((kb ^ ((r >> 1) & 3)) * 16);   // operand read offset inside a 1 KB block
    const int rd_s      = (r * 4 + kb) * 4;                  // scale dword read offset inside a 256 B block
    auto setup_null = [&]() __attribute__((always_inline)) {
        wrs[0] = wrs[1] = make_rsrc(g.w, 0);
        wsrs[0] = wsrs[1] = make_rsrc(g.w_s, 0);
#pragma unroll
        for(int i = 0; i < NA; i++)
            a_off[i] = as_off[i] = (int)0xFFFF0000u;
    };
    // Row groups of a tile that hold at least one real row.  The sort pads every expert's rows at the END of
    // its last block, so the real rows of a block are a prefix.  Padded rows send their activation fetches out
    // of the descriptor's range, where the hardware drops them, and the epilogue leaves padded row groups out.
    // Their MFMAs are still issued: the K-group body exists once (see mfma_row_group for what skipping them costs).
    // (Instantiating the body per count of active row groups and branching between the instances in C++ is NOT safe
    // with this pipeline: the register allocator then gives the weight-tile registers different homes in different
    // instances and copies them at the joins, while loads into them are still in flight, which it cannot know.
    // Measured: wrong results in tiles that run short K-groups.  tests/test_build_checks.py looks for such copies in
    // the generated code.)
    constexpr u32 OOB = 0xFFFF0000u;               // beyond every activation buffer (checked by the launcher)
    auto count_groups = [&](const u32* ids) __attribute__((always_inline)) -> int {
        const u32 id  = ids[(lane < MT ? lane : 0) * 16];
        const bool ok = lane < MT && (int)(id >> 24) < g.topk && (int)(id & 0xFFFFFFu) < g.T;
        const int n   = __builtin_popcountll(__ballot(ok));
        return n < 1 ? 1 : n;
    };
    // ids: the tile's sorted ids, either in LDS (meta buffer) or in global memory
    auto setup_load = [&](const TileId& t, const u32* ids) __attribute__((always_inline)) {
        const size_t sc_tile = (size_t)(g.SC / 8) * 256;           // bytes of one 32-row scale tile
        if(STAGE == 1)
        {
#pragma unroll
            for(int h = 0; h < 2; h++)
            {
                const size_t row = (size_t)t.e * g.N + h * I + t.nt * 128 + wave * 32;
                const bool real  = t.nt * 128 + wave * 32 < I - g.n_pad;       // (rows of padding: nothing to fetch)
                wrs[h]           = make_rsrc(g.w + row * Kb, real ? (u32)(32 * Kb) : 0u);
                wsrs[h]          = make_rsrc(g.w_s + (row / 32) * sc_tile, real ? (u32)sc_tile : 0u);
            }
        }
        else
        {
            const size_t row = (size_t)t.e * g.N + t.nt * 256 + wave * 64;
            const bool real  = t.nt * 256 + wave * 64 < g.N - g.n_pad;
            wrs[0] = wrs[1] = make_rsrc(g.w + row * Kb, real ? (u32)(64 * Kb) : 0u);
            wsrs[0] = wsrs[1] = make_rsrc(g.w_s + (row / 32) * sc_tile, real ? (u32)(2 * sc_tile) : 0u);
        }
        // (all the reads first, from a clamped position and without a branch between them: one LDS round trip instead of
        // one per slot)
        u32 idv[NA];
#pragma unroll
        for(int i = 0; i < NA; i++)
        {
            const int slot = wave + 4 * i;
            idv[i]         = ids[(slot < MT ? slot : MT - 1) * 16 + dma_row];
        }
#pragma unroll
        for(int i = 0; i < NA; i++)
        {
            const int slot = wave + 4 * i;
            const int tok  = (int)(idv[i] & 0xFFFFFFu);
            // padding rows and unused slots fetch nothing
            const bool ok  = slot < MT && (int)(idv[i] >> 24) < g.topk && tok < g.T;
            const int row  = STAGE == 1 ? tok : t.m_blk * BM + slot * 16 + dma_row;
            a_off[i]       = ok ? row * Kb + dma_chunk * 16 : (int)OOB;
            as_off[i]      = ok ? row * g.SK + (lane & 3) * 4 : (int)OOB;
        }
    };

    uint8_t* const stage[2]  = {lds_a0, lds_a1};
    uint8_t* const sstage[2] = {lds_s0, lds_s1};
    // activation tile + scales of K-group ks -> LDS stage s.  Lane (r, kb) fetches 16 B of row r, so the
    // 1 KB block of a (row group, K-step) lands in MFMA operand order; 5*NA VMEM ops per wave.
    const u32 lds_a[2] = {lds_addr_of(lds_a0 + wave * 1024), lds_addr_of(lds_a1 + wave * 1024)};
    const u32 lds_s[2] = {lds_addr_of(lds_s0 + wave * 256), lds_addr_of(lds_s1 + wave * 256)};
    // (288-row tile: the last of a wave's five slots, wave + 16, only exists for waves 0 and 1; the operations of the
    // other two waves, whose lane offsets are out of range anyway, put their zeros into the dummy area.  LDS_IMM is the
    // offset the DMA helper adds to the base it is given.)
    const bool last_slot_ok = !TALL || wave + 4 * (NA - 1) < MT;
    const u32 lds_dummy_a   = lds_addr_of(lds_dummy);
    auto slot_base = [&](auto II, auto IMM, u32 normal) __attribute__((always_inline)) -> u32 {
        if constexpr(TALL && decltype(II)::value == NA - 1)
            return last_slot_ok ? normal : lds_dummy_a - (u32)decltype(IMM)::value;
        else
            return normal;
    };
    v4i wf[4][4];
    int w_sc[2][4];
    // per-lane offsets of the wave's row groups inside wrs[] / of its scale dwords inside wsrs[]; the half that
    // is uniform (stage 2: row groups 2, 3 sit 32 rows further in the same descriptor) goes into the scalar offset,
    // which the hardware does not range-check: it stays inside the rows the descriptor covers
    const int w_voff[2]  = {lane * 16, lane * 16 + 16 * Kb};                    // row groups j = 2h, 2h+1
    const int w_half     = (STAGE >= 2) ? 32 * Kb : 0;
    const int ws_half    = (STAGE >= 2) ? (g.SC / 8) * 256 : 0;
    // The 16- and 32-row tiles are bound by the weight stream: there, lanes whose 32 columns of a K-step are all padding
    // fetch nothing (their offset is pushed out of the descriptor's range; the register gets the zeros the padding holds).
    const int k_real = g.K - g.k_pad;
    auto load_wtile = [&](auto U, auto J, int kt) __attribute__((always_inline)) {
        constexpr int u = decltype(U)::value, j = decltype(J)::value;
        if constexpr(MT <= 2)
        {
            const int away = kt * 128 + kb * 32 >= k_real ? (int)0x80000000u : 0;
            vm_load_b128<0, NT>(wf[u][j], w_voff[j & 1] + away, wrs[j >> 1], kt * 1024 + (j >> 1) * w_half);
        }
        else
            vm_load_b128<0, NT>(wf[u][j], w_voff[j & 1], wrs[j >> 1], kt * 1024 + (j >> 1) * w_half);
    };
    auto load_wtiles = [&](auto U, int kt) __attribute__((always_inline)) {
        static_for<4>([&](auto J) __attribute__((always_inline)) { load_wtile(U, J, kt); });
    };

    // accumulators and epilogue: gemm_device.h
    v4f xacc[TALL ? MT - ACC_SPILL_MT0 : 1];      // the accumulator tiles beyond the accumulation registers (288-row tile)
    auto zero_acc = [&]() __attribute__((always_inline)) { gemm_zero_acc<MT>(xacc); };
    // free_lds: the LDS stage that the tile's last K-group has just finished reading (stage 3 keeps a list there)
    auto epilogue = [&](const TileId& t, const u32* meta, int ma_t, uint8_t* free_lds) __attribute__((always_inline)) {
        if(g.bias)
            gemm_epilogue<STAGE, MT, ACT, ATOMIC, true>(g, t.e, t.nt, t.m_blk * BM, wave, meta, MPAD, ma_t, r, kb, xacc);
        else
            gemm_epilogue<STAGE, MT, ACT, ATOMIC, false>(g, t.e, t.nt, t.m_blk * BM, wave, meta, MPAD, ma_t, r, kb, xacc);
        if constexpr(STAGE == 3)
            gemm_arrive_reduce<MT>(g, t.nt, meta, ma_t, (u32*)free_lds);
    };

    // ---------------------------------------------------------------- pipeline
    constexpr int MA = MT;                    // row groups that take part in the MFMAs
    // One wave per SIMD (the tiles above 128 rows): the K-group's prefetches are spread over two K-steps and every
    // instruction that is not an MFMA sits in a gap between two MFMAs.  (Measured per K-step of the 288-row tile,
    // DeepSeek-V3 shape, 8192 tokens, in clocks, 1152 being the MFMAs alone: a K-step that only issues its four weight
    // tiles takes 1275-1300; every LDS-DMA operation adds about 40 wherever it sits, which gap of the row group included:
    // all 29 in K-step 0: 2705 + 3 x 1300; over two K-steps 1700 + 1950 + 2 x 1290; over three 1545 + 1770 + 1790 + 1275.
    // The same loads into registers instead of LDS add 10 each: the cost is in the DMA's write to LDS, not in the
    // fetch.  Two K-steps leave the last operation a K-step and a half to land before the barrier.)
    // Two or more waves per SIMD fill each other's gaps: there the four MFMAs of a row group stay back to back, the
    // other instructions follow them, and the prefetches all go out during K-step 0 (measured against the spread form
    // at 128 rows: gpt-oss shape, 4096 tokens, layer 0.573 against 0.597 ms; Mixtral shape, 512 tokens, 0.216 against
    // 0.224 ms).
    constexpr bool SPREAD = MT > 8;
    // the last GUARDED row groups of a tall tile are jumped over when they hold no real rows (mfma_row_group_guarded)
    constexpr int GUARDED = MT == 18 ? 2 : MT > 8 ? 3 : 0;
    using VS = VmSchedule<MA, NPF, SPREAD ? 2 : 1>;
    static_assert(VS::younger(0) <= 63 && VS::younger(1) <= 63 && VS::younger(2) <= 63 && VS::younger(3) <= 63,
                  "the vector-memory counter has six bits");
    // sorted ids and routing weights of a tile's rows -> LDS meta buffer `buf` (DMA, 64 rows per operation, spread over
    // the four waves)
    auto dma_meta = [&](const TileId& t, int buf) __attribute__((always_inline)) {
        const v4i rid = make_rsrc(g.sorted_ids + (size_t)t.m_blk * BM, BM * 4);
        const v4i rwt = make_rsrc(g.sorted_w + (size_t)t.m_blk * BM, BM * 4);
#pragma unroll
        for(int i = 0; i < NM; i++)
        {
            const int o    = wave + 4 * i;               // op index: [0, NID) ids, [NID, 2*NID) weights, beyond: nothing
            const bool wts = o >= NID;
            const int oo   = wts ? o - NID : o;
            if(o < 2 * NID && (!wts || g.sorted_w != nullptr))
                vm_dma_b32_fresh_sgprs((oo * 64 + lane) * 4, uni4(wts ? rwt : rid),
                                       uni(lds_addr_of(&lds_meta[buf][(wts ? MPAD : 0) + oo * 64])));
        }
    };
    // prefetch operation K (0 <= K < NPF) of a K-group: TS = the LDS stage / scale register set it fills, kpre = the
    // K-group it fetches
    auto prefetch_op = [&](auto KK, auto TS, int kpre) __attribute__((always_inline)) {
        constexpr int k = decltype(KK)::value, ts = decltype(TS)::value;
        if constexpr(k < 5 * NA)
        {
            constexpr int i = k / 5, sub = k % 5;
            using II = std::integral_constant<int, i>;
            if constexpr(sub < 4)
            {
                constexpr int imm = (sub * SLOTS + 4 * i) * 1024;
                vm_dma_b128<sub * 64, imm>(a_off[i], ars, kpre * 256, slot_base(II{}, std::integral_constant<int, imm>{}, lds_a[ts]));
            }
            else
                vm_dma_b32<0, 4 * i * 256>(as_off[i], asrs, kpre * 16, slot_base(II{}, std::integral_constant<int, 4 * i * 256>{}, lds_s[ts]));
        }
        else
        {
            constexpr int h = (k - 5 * NA) / 2, c = (k - 5 * NA) % 2;
            vm_load_b32<0>(w_sc[ts][h * 2 + c], lane * 4 + c * 256, wsrs[h], kpre * 512 + h * ws_half);
        }
    };
    // the vector-memory operations of gap G of row group N (see VmSchedule)
    auto issue_gap = [&](auto N, auto G, auto TS, int kpre) __attribute__((always_inline)) {
        constexpr int n = decltype(N)::value, gp = decltype(G)::value;
        if constexpr(gp < 3)
        {
            if constexpr(VS::is_pgap(gp) && VS::slot_of(n, gp) < VS::NSLOT)
            {
                constexpr int k0 = VS::p_before_slot(VS::slot_of(n, gp)), k1 = VS::p_before_slot(VS::slot_of(n, gp) + 1);
                static_for<k1 - k0>([&](auto Q) __attribute__((always_inline)) {
                    prefetch_op(std::integral_constant<int, k0 + decltype(Q)::value>{}, TS, kpre);
                });
            }
        }
        else
            static_for<12>([&](auto UJ) __attribute__((always_inline)) {
                constexpr int u = decltype(UJ)::value / 4, j = decltype(UJ)::value % 4;
                if constexpr(VS::w_rg(u, j) == n)
                    load_wtile(std::integral_constant<int, u>{}, std::integral_constant<int, j>{}, kpre * 4 + u);
            });
    };

    TileId cur, nxt;
    decode(cur);
    if(!cur.valid)
        return;
    int mb = 0;                                   // meta buffer of the current tile (ring of MR)
    setup_load(cur, g.sorted_ids + (size_t)cur.m_blk * BM);
    int ma     = count_groups(g.sorted_ids + (size_t)cur.m_blk * BM);   // active row groups of the current tile
    int ma_nxt = ma;                                                    // ... and of the next one
    // prologue: a K-group's vector-memory operations in the K-group's issue order, without the MFMAs: this tile's
    // ids / routing weights, activation K-group 0 into stage 0, weight scales and weight tiles of K-steps 0..3
    dma_meta(cur, 0);
    static_for<4 * MA>([&](auto N) __attribute__((always_inline)) {
        static_for<4>([&](auto G) __attribute__((always_inline)) { issue_gap(N, G, std::integral_constant<int, 0>{}, 0); });
    });
    load_wtiles(std::integral_constant<int, 3>{}, 3);
    wait_vmcnt_barrier<VS::younger_end()>();      // everything but the youngest weight tiles has landed
    decode(nxt);                      // (without a schedule there is no next tile)
    zero_acc();
    int ks = 0;

    // one K-group; returns false when the workgroup has no more work
    auto kgroup = [&](auto P) __attribute__((always_inline)) -> bool {
        constexpr int p  = decltype(P)::value;    // parity of the global K-group count: LDS stage / scale registers
        const bool last     = ks == KS - 1;
        const int kpre      = last ? 0 : ks + 1;  // K-group that is prefetched now (of the next tile when last)
        const int mb_nxt    = mb == MR - 1 ? 0 : mb + 1;
        // (0) first K-group of a tile: ids/weights of the NEXT tile into the meta ring (two tiles ahead of the
        //     slot any wave can still be reading in its epilogue)
        // (1) descriptors of what this K-group prefetches: the next K-group of this tile, or K-group 0 of the
        //     next tile (into the other LDS stage, whose readers left at the last barrier)
        if(last)
        {
            // (kept a branch: turned into selects, the set-up would run, and cost its scalar chain, in every K-group)
            asm volatile("" ::: "memory");
            if(nxt.valid)
            {
                setup_load(nxt, lds_meta[mb_nxt]);
                ma_nxt = count_groups(lds_meta[mb_nxt]);
            }
            else
                setup_null();
        }
        // (with a ring of two the slot still belongs to the previous tile, whose epilogue a slower wave may not have
        // finished before the barrier that ends this tile's first K-group: the fetch waits for the second K-group)
        if(ks == (TALL ? 1 : 0) && nxt.valid)
            dma_meta(nxt, mb_nxt);
        using TS = std::integral_constant<int, p ^ 1>;
        // The activation operand of a row group and its scale dword (one per 16-row group and K-group, op_sel picks the
        // K-step's byte) are read RA row groups ahead of the MFMAs that consume them, across K-step boundaries, through
        // a ring of RA + 1 register sets: two ahead with two waves per SIMD, four in the one-wave-per-SIMD 256-row
        // tile, where nothing else covers the LDS latency.
        constexpr int RA = MT > 8 ? 4 : 2;
        v4i af_r[RA + 1];
        int asc_all[MT];                          // the scale dword of a row group serves all four K-steps
        auto lds_read = [&](auto NN) __attribute__((always_inline)) {
            constexpr int n = decltype(NN)::value, uu = n / MA, mm = n % MA;
            af_r[n % (RA + 1)] = *(const v4i*)(stage[p] + (uu * SLOTS + mm) * 1024 + rd_a);
            if constexpr(uu == 0)
                asc_all[mm] = *(const int*)(sstage[p] + mm * 256 + rd_s);
        };
        static_for<RA>([&](auto NN) __attribute__((always_inline)) { lds_read(NN); });
        __builtin_amdgcn_sched_barrier(0);
        static_for<4>([&](auto U) __attribute__((always_inline)) {
            constexpr int u = decltype(U)::value;
            // MFMAs of K-step 4*ks + u.  Its weight tiles (and, at u = 0, the weight scales) were requested one K-group
            // ago; VS::younger counts what has been issued since.
            constexpr int YOUNGER = VS::younger(u);
            wait_vm_tiles<YOUNGER>(wf[u][0], wf[u][1], wf[u][2], wf[u][3]);
            if(u == 0)
                wait_vm_scales<YOUNGER>(w_sc[p][0], w_sc[p][1], w_sc[p][2], w_sc[p][3]);
            static_for<MA>([&](auto M) __attribute__((always_inline)) {
                constexpr int mt = decltype(M)::value;
                constexpr int n  = u * MA + mt;                // position in the K-group's sequence of row groups
                using N = std::integral_constant<int, n>;
                const v4i af  = af_r[n % (RA + 1)];
                const int asc = asc_all[mt];
                __builtin_amdgcn_sched_barrier(0);
                // weight-scale byte = (kt%2)*2 + (row%32)/16 ; activation-scale byte = kt%4
                if constexpr(!SPREAD && n + RA < 4 * MA)
                    lds_read(std::integral_constant<int, n + RA>{});
                if constexpr(SPREAD && mt >= MT - GUARDED)
                {
                    // one of the tile's last row groups, which are padding more often than not: everything else that
                    // belongs to the row group first (same order as always: the waits count on it), then its four MFMAs
                    // behind one test of the tile's number of row groups with real rows
                    if constexpr(n + RA < 4 * MA)
                        lds_read(std::integral_constant<int, n + RA>{});
                    static_for<4>([&](auto G) __attribute__((always_inline)) { issue_gap(N{}, G, TS{}, kpre); });
                    __builtin_amdgcn_sched_barrier(0);
                    v4f* xa = nullptr;
                    if constexpr(acc_in_vgprs<MT, mt>())
                        xa = &xacc[mt - ACC_SPILL_MT0];
                    mfma_row_group_guarded<u, mt, MT>(wf[u][0], wf[u][1], wf[u][2], wf[u][3], af, w_sc[p][u >> 1],
                                                      w_sc[p][2 + (u >> 1)], asc, ma, xa);
                    __builtin_amdgcn_sched_barrier(0);
                }
                else
                static_for<4>([&](auto J) __attribute__((always_inline)) {
                    constexpr int j = decltype(J)::value;
                    v4f* xa = nullptr;
                    if constexpr(acc_in_vgprs<MT, mt>() && j == 3)
                        xa = &xacc[mt - ACC_SPILL_MT0];
                    mfma_one<u, mt, MT, j>(wf[u][j], af, w_sc[p][(j >> 1) * 2 + (u >> 1)], asc, xa);
                    if constexpr(SPREAD)
                    {
                        __builtin_amdgcn_sched_barrier(0);
                        // the gap after the MFMA: the operand read of the row group RA ahead, then this gap's share of
                        // the K-group's vector-memory operations
                        if constexpr(j == 0 && n + RA < 4 * MA)
                            lds_read(std::integral_constant<int, n + RA>{});
                        issue_gap(N{}, J, TS{}, kpre);
                        __builtin_amdgcn_sched_barrier(0);
                    }
                });
                if constexpr(!SPREAD)
                {
                    __builtin_amdgcn_sched_barrier(0);
                    static_for<4>([&](auto G) __attribute__((always_inline)) { issue_gap(N{}, G, TS{}, kpre); });
                    __builtin_amdgcn_sched_barrier(0);
                }
            });
            __builtin_amdgcn_sched_barrier(0);
            if constexpr(u == 3)
                load_wtiles(U, kpre * 4 + u);
            __builtin_amdgcn_sched_barrier(0);
        });
        // the weight tiles issued since the last prefetch operation are the only operations that may still be under way
        wait_vmcnt_barrier<VS::younger_end()>();
        ks++;
        if(last)
        {
            // the last MFMAs were issued from assembly: give their results the documented distance to the
            // first VALU read
            asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
            epilogue(cur, lds_meta[mb], ma, stage[p]);
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
    for(;;)
    {
        if(!kgroup(std::integral_constant<int, 0>{}))
            break;
        if(!kgroup(std::integral_constant<int, 1>{}))
            break;
    }
#endif
}

// the eight-wave 256-row tile (moe_gemm_mxfp4_wide.hip); -1 when it does not serve the launch
int pyhip_launch_gemm_wide(int stage, const GemmArgs& g, int act, hipStream_t stream);

// lds: the launch asks for the eight-wave tile with both operands staged through LDS (block_m 256)
template <int STAGE>
static int launch_gemm(GemmArgs g, int block_m, int act, hipStream_t stream, bool atomic = false, bool lds = false)
{
    if(lds)
    {
        PYHIP_REQUIRE(block_m == 256, "moe_gemm (operands through LDS): block_m=%d, the tile has 256 rows", block_m);
        const int rc = pyhip_launch_gemm_wide(STAGE, g, act, stream);
        PYHIP_REQUIRE(rc >= 0, "moe_gemm (operands through LDS): needs the sort's schedule, K >= 1024 and at most 512 experts "
                               "(K=%d, experts=%d, schedule %s)", g.K, g.E, g.sched ? "given" : "missing");
        return rc;
    }
    unsigned nwg = (unsigned)(g.n_tiles * g.n_blk);
    // a single K-group per tile (no room to prefetch across tiles; the 288-row tile fetches the next tile's sorted ids
    // in its second K-group and needs three) or more experts than the schedule table in LDS holds (the 288-row tile
    // reads the schedule from global memory): one tile per workgroup
    if(block_m == 288 ? g.K < 1536 : (g.K < 1024 || g.E > (block_m == 16 ? SCHED_E_MAX_16 : SCHED_E_MAX)))
        g.sched = nullptr;
    if(g.sched)
    {
        // persistent: as many workgroups per CU as fit (three of the 16- and 32-row tiles: 136-160 registers, 40 KB of LDS;
        // two up to 128 rows; one of the 256-row tile).  The small tiles are bound by the weight stream; what the further
        // workgroups buy is more loads in flight (DeepSeek-V3 shape at 16 tokens: 0.417 ms with two per CU, 0.378 with
        // three).  The 16-row tile is launched with four per CU although only three are resident at a time: the last
        // quarter of the grid starts as the first workgroups leave (per-workgroup time stamps show it) and fills the
        // slots they free with its own, smaller shares of the tile list, which evens out the end of the launch
        // (DeepSeek-V3 shape at 16 tokens 0.378 -> 0.377 ms, gpt-oss shape at 16 tokens 0.139 -> 0.133 ms)
        const int cus = device_cu_count();
        unsigned resident = (unsigned)cus * (block_m == 16 ? 4u : block_m <= 32 ? 3u : block_m <= 128 ? 2u : 1u) / 8u * 8u;
        nwg               = nwg < resident ? (nwg + 7u) / 8u * 8u : resident;
    }
    dim3 grid(nwg), block(GEMM_THREADS);
    // Non-temporal weight loads when the routed rows per expert (T * topk / E on average) stay under three quarters
    // of a row block: nearly every expert then has one block, each weight tile one reader, and lines that are
    // dropped first leave the L2 to the activations.  With several blocks per expert the readers of a tile find
    // each other's lines in the L2 and the marking would throw that away.
    // (The tiles above 128 rows are chosen so that all but a few experts in a hundred have a single block, up to an
    // average of 0.8-0.96 of the block: for them the mark stays on up to 15/16 of the block.)
    const bool nt = block_m > 128 ? (int64_t)g.T * g.topk * 16 <= (int64_t)g.E * block_m * 15
                                  : (int64_t)g.T * g.topk * 4 <= (int64_t)g.E * block_m * 3;
    // ACT (0 SiLU * up, 1 clamped SwiGLU) only exists for the gate_up stage
#define GEMM_LAUNCH(MTV, ACTV, NTV) \
    hipLaunchKernelGGL((moe_gemm_mxfp4_kernel<STAGE, MTV, ACTV, NTV>), grid, block, 0, stream, g)
#define GEMM_CASE(BM, MTV)                                       \
    case BM:                                                     \
        if(STAGE == 1 && act == 1)                               \
        {                                                        \
            if(nt)                                               \
                GEMM_LAUNCH(MTV, (STAGE == 1 ? 1 : 0), true);    \
            else                                                 \
                GEMM_LAUNCH(MTV, (STAGE == 1 ? 1 : 0), false);   \
        }                                                        \
        else if(nt)                                              \
            GEMM_LAUNCH(MTV, 0, true);                           \
        else                                                     \
            GEMM_LAUNCH(MTV, 0, false);                          \
        break;
    if constexpr(STAGE == 2)
        if(atomic)
        {
            // the atomic epilogue exists for the two tile heights that matter for the comparison: decode and prefill
            if(block_m == 16 && nt)
                hipLaunchKernelGGL((moe_gemm_mxfp4_kernel<2, 1, 0, true, true>), grid, block, 0, stream, g);
            else if(block_m == 16)
                hipLaunchKernelGGL((moe_gemm_mxfp4_kernel<2, 1, 0, false, true>), grid, block, 0, stream, g);
            else if(block_m == 128 && nt)
                hipLaunchKernelGGL((moe_gemm_mxfp4_kernel<2, 8, 0, true, true>), grid, block, 0, stream, g);
            else if(block_m == 128)
                hipLaunchKernelGGL((moe_gemm_mxfp4_kernel<2, 8, 0, false, true>), grid, block, 0, stream, g);
            else
            {
                pyhip_set_error("moe_gemm2 (atomic): block_m=%d not in {16,128}", block_m);
                return PYHIP_ERR_INVALID;
            }
            PYHIP_CHECK_LAUNCH("moe_gemm_mxfp4_kernel (atomic)");
            return PYHIP_OK;
        }
    if constexpr(STAGE == 3)
    {
        // built for the tile heights that matter for the comparison with stage 2 + reduction kernel: decode, the
        // two-workgroup prefill tile and the 288-row tile
        switch(block_m)
        {
            GEMM_CASE(16, 1) GEMM_CASE(128, 8) GEMM_CASE(288, 18)
        default: pyhip_set_error("moe_gemm2 (reducing): block_m=%d not in {16,128,288}", block_m); return PYHIP_ERR_INVALID;
        }
    }
    else
        switch(block_m)
        {
            GEMM_CASE(16, 1) GEMM_CASE(32, 2) GEMM_CASE(64, 4) GEMM_CASE(128, 8) GEMM_CASE(160, 10) GEMM_CASE(192, 12)
            GEMM_CASE(256, 16) GEMM_CASE(288, 18)
        default: pyhip_set_error("moe_gemm: block_m=%d not in {16,32,64,128,160,192,256,288}", block_m); return PYHIP_ERR_INVALID;
        }
#undef GEMM_CASE
#undef GEMM_LAUNCH
    PYHIP_CHECK_LAUNCH("moe_gemm_mxfp4_kernel");
    return PYHIP_OK;
}

static int check_common(const char* name, const void* a_q, const void* a_s, const void* w, const void* w_s,
                        const void* sorted_ids, const void* sorted_e, const void* num_valid, const void* out,
                        int K, int block_m, int64_t n_blk, int64_t a_rows)
{
    PYHIP_REQUIRE(a_q && a_s && w && w_s && sorted_ids && sorted_e && num_valid && out, "%s: null pointer", name);
    PYHIP_REQUIRE(K > 0 && K % 512 == 0, "%s: K=%d must be a positive multiple of 512", name, K);
    PYHIP_REQUIRE(block_m == 16 || block_m == 32 || block_m == 64 || block_m == 128 || block_m == 160 || block_m == 192 ||
                      block_m == 256 || block_m == 288,
                  "%s: block_m=%d not in {16,32,64,128,160,192,256,288}", name, block_m);
    PYHIP_REQUIRE(n_blk >= 0 && n_blk < (1 << 24), "%s: n_blk=%lld", name, (long long)n_blk);
    PYHIP_REQUIRE(a_rows > 0 && a_rows * (int64_t)(K / 2) < 0xFFFF0000ll,
                  "%s: activation matrix of %lld rows x %d exceeds the 4 GiB buffer range", name, (long long)a_rows, K);
    PYHIP_REQUIRE(((uintptr_t)a_q % 16) == 0 && ((uintptr_t)a_s % 4) == 0 && ((uintptr_t)w % 16) == 0 &&
                      ((uintptr_t)w_s % 4) == 0 && ((uintptr_t)out % 8) == 0,
                  "%s: unaligned pointer", name);
    return PYHIP_OK;
}

static int gemm1_impl(const uint8_t* a_q, const uint8_t* a_scale, const uint8_t* w1, const uint8_t* w1_scale,
                      const void* bias1_bf16, const uint32_t* sorted_ids, const uint32_t* sorted_expert_ids,
                      const uint32_t* num_valid_ids, const uint32_t* schedule, void* a2_bf16, uint8_t* a2_q,
                      uint8_t* a2_scale, int tokens, int topk, int experts, int hidden, int inter, int hidden_pad,
                      int inter_pad, int block_m, int64_t n_blk, int activation, float swiglu_limit, hipStream_t stream,
                      bool lds)
{
    PYHIP_REQUIRE(hidden_pad >= 0 && hidden_pad < hidden && inter_pad >= 0 && inter_pad < inter,
                  "moe_gemm1: hidden_pad=%d / inter_pad=%d outside [0, hidden=%d) / [0, inter=%d)", hidden_pad, inter_pad,
                  hidden, inter);
    PYHIP_REQUIRE(a2_bf16 || a2_q, "moe_gemm1: no output buffer");
    PYHIP_REQUIRE(activation == 0 || (activation == 1 && swiglu_limit > 0.f),
                  "moe_gemm1: activation=%d (0 SiLU, 1 SwiGLU with a positive limit)", activation);
    PYHIP_REQUIRE((a2_q == nullptr) == (a2_scale == nullptr), "moe_gemm1: a2_q and a2_scale go together");
    PYHIP_REQUIRE(!a2_q || inter % 512 == 0, "moe_gemm1: quantised output needs inter=%d to be a multiple of 512", inter);
    PYHIP_REQUIRE(((uintptr_t)a2_q % 4) == 0 && ((uintptr_t)a2_bf16 % 16) == 0, "moe_gemm1: unaligned output");
    int rc = check_common("moe_gemm1", a_q, a_scale, w1, w1_scale, sorted_ids, sorted_expert_ids, num_valid_ids,
                          a2_bf16 ? a2_bf16 : (void*)a2_q, hidden, block_m, n_blk, tokens);
    if(rc)
        return rc;
    PYHIP_REQUIRE(inter > 0 && inter % 128 == 0, "moe_gemm1: inter=%d must be a multiple of 128", inter);
    PYHIP_REQUIRE(tokens > 0 && topk > 0 && experts > 0, "moe_gemm1: bad sizes");
    if(n_blk == 0)
        return PYHIP_OK;
    GemmArgs g;
    g.a_q = a_q; g.a_s = a_scale; g.w = w1; g.w_s = w1_scale; g.bias = (const uint16_t*)bias1_bf16;
    g.sorted_ids = sorted_ids; g.sorted_w = nullptr; g.sorted_e = sorted_expert_ids; g.num_valid = num_valid_ids;
    g.out = a2_bf16; g.out_q = a2_q; g.out_s = a2_scale; g.OSK = (inter + 511) / 512 * 16;
    g.limit = swiglu_limit;
    g.sched = schedule; g.E = experts;
    g.T = tokens; g.topk = topk; g.K = hidden; g.N = 2 * inter;
    g.SK = (hidden + 511) / 512 * 16;
    g.SC = (hidden / 32 + 7) / 8 * 8;
    g.n_blk = (int)n_blk; g.n_tiles = inter / 128; g.a_rows = tokens;
    g.n_pad = inter_pad; g.k_pad = hidden_pad;
    return launch_gemm<1>(g, block_m, activation, stream, false, lds);
}

extern "C" int pyhip_moe_gemm1_mxfp4(const uint8_t* a_q, const uint8_t* a_scale, const uint8_t* w1,
                                     const uint8_t* w1_scale, const void* bias1_bf16, const uint32_t* sorted_ids,
                                     const uint32_t* sorted_expert_ids, const uint32_t* num_valid_ids,
                                     const uint32_t* schedule, void* a2_bf16, uint8_t* a2_q, uint8_t* a2_scale,
                                     int tokens, int topk, int experts, int hidden, int inter, int hidden_pad,
                                     int inter_pad, int block_m, int64_t n_blk, int activation, float swiglu_limit,
                                     hipStream_t stream)
{
    return gemm1_impl(a_q, a_scale, w1, w1_scale, bias1_bf16, sorted_ids, sorted_expert_ids, num_valid_ids, schedule,
                      a2_bf16, a2_q, a2_scale, tokens, topk, experts, hidden, inter, hidden_pad, inter_pad, block_m, n_blk,
                      activation, swiglu_limit, stream, false);
}

// The gate_up GEMM on the eight-wave 256-row tile whose operands both go through LDS (moe_gemm_mxfp4_wide.hip); the
// sort must have been run with block_size 256 and must have written the schedule.
extern "C" int pyhip_moe_gemm1_mxfp4_lds(const uint8_t* a_q, const uint8_t* a_scale, const uint8_t* w1,
                                         const uint8_t* w1_scale, const void* bias1_bf16, const uint32_t* sorted_ids,
                                         const uint32_t* sorted_expert_ids, const uint32_t* num_valid_ids,
                                         const uint32_t* schedule, void* a2_bf16, uint8_t* a2_q, uint8_t* a2_scale,
                                         int tokens, int topk, int experts, int hidden, int inter, int64_t n_blk,
                                         int activation, float swiglu_limit, hipStream_t stream)
{
    return gemm1_impl(a_q, a_scale, w1, w1_scale, bias1_bf16, sorted_ids, sorted_expert_ids, num_valid_ids, schedule,
                      a2_bf16, a2_q, a2_scale, tokens, topk, experts, hidden, inter, 0, 0, 256, n_blk, activation,
                      swiglu_limit, stream, true);
}

static int gemm2_impl(const uint8_t* a2_q, const uint8_t* a2_scale, const uint8_t* w2, const uint8_t* w2_scale,
                      const void* bias2_bf16, const uint32_t* sorted_ids, const float* sorted_weights,
                      const uint32_t* sorted_expert_ids, const uint32_t* num_valid_ids, const uint32_t* schedule,
                      void* out3_bf16, int tokens, int topk, int experts, int hidden, int inter, int hidden_pad,
                      int inter_pad, int block_m, int64_t n_blk, hipStream_t stream, bool lds)
{
    PYHIP_REQUIRE(hidden_pad >= 0 && hidden_pad < hidden && inter_pad >= 0 && inter_pad < inter,
                  "moe_gemm2: hidden_pad=%d / inter_pad=%d outside [0, hidden=%d) / [0, inter=%d)", hidden_pad, inter_pad,
                  hidden, inter);
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
    g.num_valid = num_valid_ids; g.out = out3_bf16; g.out_q = nullptr; g.out_s = nullptr; g.OSK = 0;
    g.limit = 0.f;
    g.sched = schedule; g.E = experts;
    g.T = tokens; g.topk = topk; g.K = inter; g.N = hidden;
    g.SK = (inter + 511) / 512 * 16;
    g.SC = (inter / 32 + 7) / 8 * 8;
    g.n_blk = (int)n_blk; g.n_tiles = hidden / 256; g.a_rows = (int)(n_blk * block_m);
    g.n_pad = hidden_pad; g.k_pad = inter_pad;
    return launch_gemm<2>(g, block_m, 0, stream, false, lds);
}

extern "C" int pyhip_moe_gemm2_mxfp4(const uint8_t* a2_q, const uint8_t* a2_scale, const uint8_t* w2,
                                     const uint8_t* w2_scale, const void* bias2_bf16, const uint32_t* sorted_ids,
                                     const float* sorted_weights, const uint32_t* sorted_expert_ids,
                                     const uint32_t* num_valid_ids, const uint32_t* schedule, void* out3_bf16,
                                     int tokens, int topk, int experts, int hidden, int inter, int hidden_pad,
                                     int inter_pad, int block_m, int64_t n_blk, hipStream_t stream)
{
    return gemm2_impl(a2_q, a2_scale, w2, w2_scale, bias2_bf16, sorted_ids, sorted_weights, sorted_expert_ids,
                      num_valid_ids, schedule, out3_bf16, tokens, topk, experts, hidden, inter, hidden_pad, inter_pad, block_m,
                      n_blk, stream, false);
}

// the down GEMM on the same tile
extern "C" int pyhip_moe_gemm2_mxfp4_lds(const uint8_t* a2_q, const uint8_t* a2_scale, const uint8_t* w2,
                                         const uint8_t* w2_scale, const void* bias2_bf16, const uint32_t* sorted_ids,
                                         const float* sorted_weights, const uint32_t* sorted_expert_ids,
                                         const uint32_t* num_valid_ids, const uint32_t* schedule, void* out3_bf16,
                                         int tokens, int topk, int experts, int hidden, int inter, int64_t n_blk,
                                         hipStream_t stream)
{
    return gemm2_impl(a2_q, a2_scale, w2, w2_scale, bias2_bf16, sorted_ids, sorted_weights, sorted_expert_ids,
                      num_valid_ids, schedule, out3_bf16, tokens, topk, experts, hidden, inter, 0, 0, 256, n_blk, stream, true);
}

// The down GEMM with the top-k reduction in its epilogue: every (token, slot) result is added into out[token, :]
// (bf16 [tokens, hidden], which the caller has cleared, e.g. with pyhip_moe_zero_fill) with packed bf16 atomics, the
// reference's atomic variant (src/contrib/moe_gemm_mxfp4.py:1334-1398, src/contrib/moe.py:703-787).  No out3, no
// reduction launch; the price is a result that depends on the arrival order of a token's slots (bf16 additions do
// not commute with rounding) and atomic traffic.  block_m 16 or 128.
extern "C" int pyhip_moe_gemm2_mxfp4_atomic(const uint8_t* a2_q, const uint8_t* a2_scale, const uint8_t* w2,
                                            const uint8_t* w2_scale, const void* bias2_bf16, const uint32_t* sorted_ids,
                                            const float* sorted_weights, const uint32_t* sorted_expert_ids,
                                            const uint32_t* num_valid_ids, const uint32_t* schedule, void* out_bf16,
                                            int tokens, int topk, int experts, int hidden, int inter, int block_m,
                                            int64_t n_blk, hipStream_t stream)
{
    int rc = check_common("moe_gemm2_atomic", a2_q, a2_scale, w2, w2_scale, sorted_ids, sorted_expert_ids, num_valid_ids,
                          out_bf16, inter, block_m, n_blk, n_blk * block_m);
    if(rc)
        return rc;
    PYHIP_REQUIRE(sorted_weights, "moe_gemm2_atomic: null sorted_weights");
    PYHIP_REQUIRE(hidden > 0 && hidden % 256 == 0, "moe_gemm2_atomic: hidden=%d must be a multiple of 256", hidden);
    PYHIP_REQUIRE(tokens > 0 && topk > 0 && experts > 0, "moe_gemm2_atomic: bad sizes");
    if(n_blk == 0)
        return PYHIP_OK;
    GemmArgs g;
    g.a_q = a2_q; g.a_s = a2_scale; g.w = w2; g.w_s = w2_scale; g.bias = (const uint16_t*)bias2_bf16;
    g.sorted_ids = sorted_ids; g.sorted_w = sorted_weights; g.sorted_e = sorted_expert_ids;
    g.num_valid = num_valid_ids; g.out = out_bf16; g.out_q = nullptr; g.out_s = nullptr; g.OSK = 0;
    g.limit = 0.f;
    g.sched = schedule; g.E = experts;
    g.T = tokens; g.topk = topk; g.K = inter; g.N = hidden;
    g.SK = (inter + 511) / 512 * 16;
    g.SC = (inter / 32 + 7) / 8 * 8;
    g.n_blk = (int)n_blk; g.n_tiles = hidden / 256; g.a_rows = (int)(n_blk * block_m);
    return launch_gemm<2>(g, block_m, 0, stream, true);
}

// Set-up of the reducing down GEMM (stage 3): arrive[token, weight tile] = the number of the token's slots that take part
// in the layer; a token without any (all its pairs dropped, or past the local token count) is nobody's to complete: its
// output row is written here, as zeros.  One wave per token.
__global__ void __launch_bounds__(256) moe_arrive_init_kernel(const int* topk_ids, const int* expert_mask,
                                                              const int* num_local_tok, int* arrive, void* out, int out_f32,
                                                              int T, int topk, int experts, int n_tiles)
{
    const int tok = blockIdx.x * 4 + threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
    if(tok >= T)
        return;
    int T_local = T;
    if(num_local_tok)
    {
        const int lim = *num_local_tok;
        T_local       = lim < 0 ? 0 : (lim < T ? lim : T);
    }
    int kept = 0;
    if(tok < T_local)
        for(int s = 0; s < topk; s++)
            kept += moe_pair_is_kept(topk_ids[(size_t)tok * topk + s], experts, expert_mask) ? 1 : 0;
    for(int i = lane; i < n_tiles; i += WAVE)
        arrive[(size_t)tok * n_tiles + i] = kept;
    if(kept == 0)
    {
        const int words = n_tiles * 256 / (out_f32 ? 1 : 2);
        u32* row        = (u32*)out + (size_t)tok * words;
        for(int i = lane; i < words; i += WAVE)
            row[i] = 0u;
    }
}

// The down GEMM that also does the top-k reduction: out3 is written as by pyhip_moe_gemm2_mxfp4, and the workgroup that
// stores the last of a token's slots for a 256-channel weight tile sums the slots (fp32, slot order, one rounding: the
// arithmetic of pyhip_moe_topk_reduce_routed, bit for bit) and writes out[tokens, hidden].  No reduction launch and no
// waiting between workgroups; a deterministic alternative to the reference's atomic epilogue
// (src/contrib/moe_gemm_mxfp4.py:1334-1398).  arrive: int32 [tokens * hidden / 256] of scratch, initialised here.
// block_m 16, 128 or 288.  Measured against the two-kernel path, which stays what pyhip_moe_forward uses.
extern "C" int pyhip_moe_gemm2_mxfp4_reduce(const uint8_t* a2_q, const uint8_t* a2_scale, const uint8_t* w2,
                                            const uint8_t* w2_scale, const void* bias2_bf16, const uint32_t* sorted_ids,
                                            const float* sorted_weights, const uint32_t* sorted_expert_ids,
                                            const uint32_t* num_valid_ids, const uint32_t* schedule, void* out3_bf16,
                                            const int32_t* topk_ids, const int32_t* expert_mask,
                                            const int32_t* num_local_tokens, int32_t* arrive, void* out, int out_is_f32,
                                            int tokens, int topk, int experts, int hidden, int inter, int block_m,
                                            int64_t n_blk, hipStream_t stream)
{
    int rc = check_common("moe_gemm2_reduce", a2_q, a2_scale, w2, w2_scale, sorted_ids, sorted_expert_ids, num_valid_ids,
                          out3_bf16, inter, block_m, n_blk, n_blk * block_m);
    if(rc)
        return rc;
    PYHIP_REQUIRE(sorted_weights && topk_ids && arrive && out, "moe_gemm2_reduce: null pointer");
    PYHIP_REQUIRE(hidden > 0 && hidden % 256 == 0, "moe_gemm2_reduce: hidden=%d must be a multiple of 256", hidden);
    PYHIP_REQUIRE(tokens > 0 && tokens < (1 << 24) && topk > 0 && topk < 256 && experts > 0, "moe_gemm2_reduce: bad sizes");
    PYHIP_REQUIRE(((uintptr_t)out3_bf16 % 16) == 0 && ((uintptr_t)out % 16) == 0 && ((uintptr_t)arrive % 4) == 0,
                  "moe_gemm2_reduce: unaligned pointer");
    hipLaunchKernelGGL(moe_arrive_init_kernel, dim3((tokens + 3) / 4), dim3(256), 0, stream, topk_ids, expert_mask,
                       num_local_tokens, arrive, out, out_is_f32, tokens, topk, experts, hidden / 256);
    PYHIP_CHECK_LAUNCH("moe_arrive_init_kernel");
    if(n_blk == 0)
        return PYHIP_OK;
    GemmArgs g;
    g.a_q = a2_q; g.a_s = a2_scale; g.w = w2; g.w_s = w2_scale; g.bias = (const uint16_t*)bias2_bf16;
    g.sorted_ids = sorted_ids; g.sorted_w = sorted_weights; g.sorted_e = sorted_expert_ids;
    g.num_valid = num_valid_ids; g.out = out3_bf16; g.out_q = nullptr; g.out_s = nullptr; g.OSK = 0;
    g.limit = 0.f;
    g.sched = schedule; g.E = experts;
    g.T = tokens; g.topk = topk; g.K = inter; g.N = hidden;
    g.SK = (inter + 511) / 512 * 16;
    g.SC = (inter / 32 + 7) / 8 * 8;
    g.n_blk = (int)n_blk; g.n_tiles = hidden / 256; g.a_rows = (int)(n_blk * block_m);
    g.arrive = arrive; g.topk_ids = topk_ids; g.expert_mask = expert_mask; g.final_out = out; g.final_f32 = out_is_f32;
    g.experts_all = experts;
    return launch_gemm<3>(g, block_m, 0, stream);
}
