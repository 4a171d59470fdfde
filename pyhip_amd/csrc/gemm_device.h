// Device-side building blocks shared by the MXFP4 x MXFP4 GEMM kernels (moe_gemm_mxfp4.hip, moe_gemm_mxfp4_wide.hip):
// the kernel argument block, the scaled MFMA on hand-numbered accumulation registers, the vector-memory primitives
// whose waits are counted by hand, and the lane transposes of the epilogues.
#pragma once
#include "common.h"
#include <stdlib.h>

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
    const u32* sched;          // tile schedule written by the sort (moe_sort.hip: write_schedule) or null
    void* out;                 // stage 1: bf16 [n_blk*BM, N/2] (may be null); stage 2: bf16 [T, topk, N]
    uint8_t* out_q;            // stage 1: MXFP4 of the output, e2m1 pairs [n_blk*BM, N/4], or null
    uint8_t* out_s;            //          and its scales [n_blk*BM, OSK] in the activation-scale layout
    int OSK;
    float limit;               // stage 1, SwiGLU: the clamp
    int T, topk, K, N, SK, SC, n_blk, n_tiles, a_rows, E;
    // stage 3 only (the down GEMM that also reduces over the slots, see gemm_arrive_reduce)
    int* arrive            = nullptr;   // [T, n_tiles] slots of the token that have not been stored yet
    const int* topk_ids    = nullptr;   // [T, topk] the routing ...
    const int* expert_mask = nullptr;   // ... and the expert mask ([experts_all] or null), for the drop rule
    void* final_out        = nullptr;   // [T, N] bf16, or fp32 when final_f32 != 0
    int final_f32 = 0, experts_all = 0;
    // zero padding at the end of the weight matrices (shapes that are not multiples of the tiles arrive padded): the last
    // n_pad rows of every expert's weight matrix (stage 1: of its gate half and of its up half) and the last k_pad
    // columns are zeros.  Waves whose weight rows are all padding fetch nothing (the registers then hold the zeros that
    // an out-of-range fetch returns: the same product), and so do, in the 16- and 32-row tiles, lanes past the real columns.
    int n_pad = 0, k_pad = 0;
};

// acc += W(16 rows x 128 K, e2m1) * A(128 K x 16 rows, e2m1) with per-lane e8m0 block scales.
// The accumulators are the accumulation registers a[(j*MT + mt)*4 .. +3] of (weight row group j, row group mt), named
// in the instruction text: the compiler never sees them as values.  (Declared as ordinary vectors, in either register
// file, about a third of them get renamed on every K-step, get shuffled between the files around the loop and spill.)
// With the register numbers fixed by hand, the kernel reserves the range once (see the clobber at its top) and must keep
// its ordinary register use below the point where the compiler would start parking values there (checked at build time
// by looking for accumulation-register moves outside these helpers).  U = K-step inside the K-group: it selects the byte
// of the scale dwords (weights: (kt%2)*2 + (row%32)/16 through op_sel / op_sel_hi, activations: kt%4).
// (Row groups that hold only padding are NOT skipped.  Measured with a compare and a branch around the four MFMAs
// inside this statement, so that nothing else about the generated code changes: the pair costs more issue time in
// full tiles than the skipped MFMAs save elsewhere: DeepSeek-V3 shape, 8192 tokens, where a fifth of the row groups
// are padding: gate_up 1.30 -> 1.38 ms; Mixtral shape, 4096 tokens, no padding: 0.477 -> 0.503 ms.)
// (The 288-row tile has 72 accumulator tiles, eight more than the 256 accumulation registers hold: those of weight row
// group 3 and row groups ACC_SPILL_MT0 .. 17 are ordinary vectors, handed in as `xacc`.)
#define ACC_SPILL_MT0 10
template <int MT, int MTI>
constexpr bool acc_in_vgprs() { return (3 * MT + MTI) * 4 >= 256; }
// One MFMA of a row group: weight row group J (0..3) of the wave against activation row group MTI, K-step U of the
// K-group.  The four MFMAs of a row group are separate statements so that the kernel can put its other instructions
// (LDS reads, vector-memory issue) into the gaps between them: an MFMA occupies the matrix pipeline for 16 cycles but
// the wave's issue port only for four, and instructions issued in those gaps are free, while the same instructions
// placed after four back-to-back MFMAs delay the next row group (measured on a stream of MFMAs with eight s_nop per
// row group: + 12 % behind the fourth MFMA, nothing between them).
template <int U, int MTI, int MT, int J>
__device__ __forceinline__ void mfma_one(v4i w, v4i a, int ws, int a_scale, v4f* xacc = nullptr)
{
    constexpr int A0 = (J * MT + MTI) * 4;
    static_assert(J == 3 || A0 + 3 < 256, "only weight row group 3 may overflow the accumulation registers");
    constexpr int WB = (U & 1) * 2 + (J & 1);       // weight-scale byte: (kt%2)*2 + (row%32)/16
    if constexpr(acc_in_vgprs<MT, MTI>() && J == 3)
        asm volatile("v_mfma_scale_f32_16x16x128_f8f6f4 %[xa], %[w], %[a], %[xa], %[ws], %[as] op_sel:[%[wl],%[al],0] "
                     "op_sel_hi:[%[wh],%[ah],0] cbsz:4 blgp:4"
                     : [xa] "+v"(*xacc)
                     : [w] "v"(w), [a] "v"(a), [ws] "v"(ws), [as] "v"(a_scale), [wl] "n"(WB & 1), [wh] "n"(WB >> 1),
                       [al] "n"(U & 1), [ah] "n"(U >> 1));
    else
        asm volatile("v_mfma_scale_f32_16x16x128_f8f6f4 a[%[c]:%[e]], %[w], %[a], a[%[c]:%[e]], %[ws], %[as] "
                     "op_sel:[%[wl],%[al],0] op_sel_hi:[%[wh],%[ah],0] cbsz:4 blgp:4"
                     :
                     : [c] "n"(A0), [e] "n"(A0 + 3), [w] "v"(w), [a] "v"(a), [ws] "v"(ws), [as] "v"(a_scale),
                       [wl] "n"(WB & 1), [wh] "n"(WB >> 1), [al] "n"(U & 1), [ah] "n"(U >> 1));
}
// The four MFMAs of a row group behind a test of the tile's number of row groups that hold real rows: a row group at or
// beyond that number is padding (zeros in LDS: its MFMAs add nothing) and is jumped over.  One compare and one branch
// per row group, so it is only used for the last few row groups of the tall tiles, the ones that are empty often: a
// tile height is chosen so that an expert's rows usually fit one block, which leaves the block's tail unused more often
// than not.  (A guard around EVERY row group costs more issue time than the skipped MFMAs save, see above; and what the
// matrix pipeline does not execute it does not draw power for, which on this part is what the memory stream gets.)
template <int U, int MTI, int MT>
__device__ __forceinline__ void mfma_row_group_guarded(v4i w0, v4i w1, v4i w2, v4i w3, v4i a, int ws01, int ws23, int a_scale,
                                                       int groups_with_rows, v4f* xacc = nullptr)
{
    constexpr int A0 = MTI * 4, A1 = (MT + MTI) * 4, A2 = (2 * MT + MTI) * 4, A3 = (3 * MT + MTI) * 4;
    constexpr int WL = U & 1;                         // weight-scale byte (kt%2)*2 + (row%32)/16: op_sel_hi = kt%2 ...
    static_assert(A2 + 3 < 256, "only weight row group 3 may overflow the accumulation registers");
#define PYHIP_MFMA_TXT(ACC, W, WS, LO) \
    "v_mfma_scale_f32_16x16x128_f8f6f4 " ACC ", " W ", %[a], " ACC ", " WS ", %[as] op_sel:[" LO ",%[al],0] op_sel_hi:[%[wh],%[ah],0] cbsz:4 blgp:4\n\t"
    if constexpr(acc_in_vgprs<MT, MTI>())
        asm volatile("s_cmp_le_u32 %[n], %[mti]\n\ts_cbranch_scc1 1f\n\t"
                     PYHIP_MFMA_TXT("a[%[c0]:%[e0]]", "%[w0]", "%[s01]", "0")
                     PYHIP_MFMA_TXT("a[%[c1]:%[e1]]", "%[w1]", "%[s01]", "1")
                     PYHIP_MFMA_TXT("a[%[c2]:%[e2]]", "%[w2]", "%[s23]", "0")
                     PYHIP_MFMA_TXT("%[xa]", "%[w3]", "%[s23]", "1")
                     "1:"
                     : [xa] "+v"(*xacc)
                     : [n] "s"(groups_with_rows), [mti] "n"(MTI), [c0] "n"(A0), [e0] "n"(A0 + 3), [c1] "n"(A1), [e1] "n"(A1 + 3),
                       [c2] "n"(A2), [e2] "n"(A2 + 3), [w0] "v"(w0), [w1] "v"(w1), [w2] "v"(w2), [w3] "v"(w3), [a] "v"(a),
                       [s01] "v"(ws01), [s23] "v"(ws23), [as] "v"(a_scale), [wh] "n"(WL), [al] "n"(U & 1), [ah] "n"(U >> 1)
                     : "scc");
    else
        asm volatile("s_cmp_le_u32 %[n], %[mti]\n\ts_cbranch_scc1 1f\n\t"
                     PYHIP_MFMA_TXT("a[%[c0]:%[e0]]", "%[w0]", "%[s01]", "0")
                     PYHIP_MFMA_TXT("a[%[c1]:%[e1]]", "%[w1]", "%[s01]", "1")
                     PYHIP_MFMA_TXT("a[%[c2]:%[e2]]", "%[w2]", "%[s23]", "0")
                     PYHIP_MFMA_TXT("a[%[c3]:%[e3]]", "%[w3]", "%[s23]", "1")
                     "1:"
                     :
                     : [n] "s"(groups_with_rows), [mti] "n"(MTI), [c0] "n"(A0), [e0] "n"(A0 + 3), [c1] "n"(A1), [e1] "n"(A1 + 3),
                       [c2] "n"(A2), [e2] "n"(A2 + 3), [c3] "n"(A3), [e3] "n"(A3 + 3), [w0] "v"(w0), [w1] "v"(w1), [w2] "v"(w2),
                       [w3] "v"(w3), [a] "v"(a), [s01] "v"(ws01), [s23] "v"(ws23), [as] "v"(a_scale), [wh] "n"(WL), [al] "n"(U & 1),
                       [ah] "n"(U >> 1)
                     : "scc");
#undef PYHIP_MFMA_TXT
}
// the four MFMAs of a row group back to back (the eight-wave kernel, whose two waves per SIMD fill each other's gaps)
template <int U, int MTI, int MT>
__device__ __forceinline__ void mfma_row_group(v4i w0, v4i w1, v4i w2, v4i w3, v4i a, int ws01, int ws23, int a_scale,
                                               v4f* xacc = nullptr)
{
    mfma_one<U, MTI, MT, 0>(w0, a, ws01, a_scale);
    mfma_one<U, MTI, MT, 1>(w1, a, ws01, a_scale);
    mfma_one<U, MTI, MT, 2>(w2, a, ws23, a_scale);
    mfma_one<U, MTI, MT, 3>(w3, a, ws23, a_scale, xacc);
}

// ---- Vector-memory issue schedule of one K-group of the four-wave kernel (moe_gemm_mxfp4.hip).
// A K-group is 4 K-steps x MA row groups; a row group is four MFMAs with a gap after each.  Per wave and K-group the
// kernel issues NPF prefetch operations (sorted ids, activation DMA, scales) and 16 weight tiles.  They are spread
// evenly instead of bunched: the texture-address path takes 16 clocks per 1 KB operation and CU, and a wave that finds
// its queue full stalls at the issue, MFMAs included.
//   prefetch operation k : slot pslot(k) = k * NSLOT / NPF of the NSLOT = PGAPS * PSTEPS * MA slots that the last PGAPS of
//                          the gaps 0..2 of the row groups of K-steps 0 .. PSTEPS-1 offer (the later K-steps leave
//                          the operations time to land)
//   weight tile (u, j)   : the registers are free once K-step u's MFMAs are issued: u < 3: gap 3 of row group
//                          (u + 1) * MA + j * MA / 4; u = 3: after the last row group
// The issue order is the same in every K-group (and in the prologue), which makes "all but the N youngest operations
// have completed" exact: the functions below count N for the waits.
template <int MA, int NPF, int PSTEPS, int PGAPS = 3>
struct VmSchedule
{
    // prefetch operations use the last PGAPS of the gaps 0..2 of a row group (gap 0 also holds the LDS operand read)
    static constexpr int NSLOT = PGAPS * PSTEPS * MA;
    static constexpr int TOTAL = NPF + 16;
    static constexpr int slot_of(int n, int gap) { return n * PGAPS + gap - (3 - PGAPS); }      // gap >= 3 - PGAPS
    static constexpr bool is_pgap(int gap) { return gap >= 3 - PGAPS && gap < 3; }
    static constexpr int p_before_slot(int s)      // prefetch operations in slots < s
    {
        const int c = (s * NPF + NSLOT - 1) / NSLOT;
        return s >= NSLOT ? NPF : c < NPF ? c : NPF;
    }
    static constexpr int w_rg(int u, int j) { return (u + 1) * MA + j * MA / 4; }
    static constexpr int w_before_rg(int n)        // weight tiles (u < 3) issued in row groups < n
    {
        int c = 0;
        for(int u = 0; u < 3; u++)
            for(int j = 0; j < 4; j++)
                c += w_rg(u, j) < n;
        return c;
    }
    static constexpr int before_rg(int n) { return p_before_slot(PGAPS * n < NSLOT ? PGAPS * n : NSLOT) + w_before_rg(n); }
    static constexpr int w_index(int u, int j)
    {
        if(u == 3)
            return NPF + 12 + j;
        const int n = w_rg(u, j);
        return p_before_slot(PGAPS * (n + 1) < NSLOT ? PGAPS * (n + 1) : NSLOT) + 4 * u + j;
    }
    // operations younger than the tiles of K-step u (issued one K-group ago) when K-step u starts
    static constexpr int younger(int u) { return TOTAL - 1 - w_index(u, 3) + before_rg(u * MA); }
    // operations younger than the last prefetch operation at the end of the K-group
    // (the weight tiles in gap 3 of its own row group come after it)
    static constexpr int younger_end() { return 16 - w_before_rg(((NPF - 1) * NSLOT / NPF) / PGAPS); }
};

template <int R>
__device__ __forceinline__ float acc_fixed_read()
{
    float x;
    asm volatile("v_accvgpr_read_b32 %0, a[%1]" : "=v"(x) : "n"(R));
    return x;
}
template <int R>
__device__ __forceinline__ void acc_fixed_zero()
{
    asm volatile("v_accvgpr_write_b32 a[%0], 0" ::"n"(R));
}

// ---- vector-memory primitives.  Every VMEM operation of the pipeline is issued through inline assembly
// and every wait on the VMEM counter is written by hand: the counter retires loads in issue order, the
// issue order below is fixed, so "all but the N youngest operations have completed" is exact.  (Left to
// the compiler, the waits around loop back-edges and around LDS-DMA operations collapse the prefetch
// distance to one or two K-steps.)
__device__ __forceinline__ v4i make_rsrc(const void* p, u32 bytes)
{
    const unsigned long long a = (unsigned long long)p;
    // raw buffer: base[47:0], stride 0, num_records = bytes, word 3 = 32-bit data format
    return (v4i){(int)(u32)a, (int)((a >> 32) & 0xFFFFu), (int)bytes, 0x00020000};
}
// address = rsrc.base + voff + soff + IMM (IMM < 4096); only voff + IMM is range-checked
template <int IMM = 0, bool NT = false>
__device__ __forceinline__ void vm_load_b128(v4i& dst, int voff, v4i rsrc, int soff)
{
    if(NT)      // streamed once: the line is the first to go when the L2 needs room
        asm volatile("buffer_load_dwordx4 %0, %1, %2, %3 offen offset:%4 nt" : "=v"(dst) : "v"(voff), "s"(rsrc), "s"(soff), "n"(IMM) : "memory");
    else
        asm volatile("buffer_load_dwordx4 %0, %1, %2, %3 offen offset:%4" : "=v"(dst) : "v"(voff), "s"(rsrc), "s"(soff), "n"(IMM) : "memory");
}
template <int IMM = 0>
__device__ __forceinline__ void vm_load_b32(int& dst, int voff, v4i rsrc, int soff)
{
    asm volatile("buffer_load_dword %0, %1, %2, %3 offen offset:%4" : "=v"(dst) : "v"(voff), "s"(rsrc), "s"(soff), "n"(IMM) : "memory");
}
// global -> LDS without passing through registers: lane i's bytes land at lds_base + LDS_IMM + i * size.
// (The hardware adds the instruction's immediate offset to the LDS address as well as to the global one, so
// M0 is set to the target minus IMM.)  M0 cannot be named as a clobber: it is a reserved register for the compiler,
// which neither tracks nor preserves it around inline assembly (it says so when asked to).  These helpers are sound
// as long as the compiler's own code never uses M0 in these kernels (on gfx9 LDS instructions do not need it);
// tests/test_build_checks.py checks on the generated code that nothing outside the inline assembly names M0.
template <int IMM, int LDS_IMM, bool NT = false>
__device__ __forceinline__ void vm_dma_b128(int voff, v4i rsrc, int soff, u32 lds_base)
{
    if(NT)      // streamed once: the line is the first to go when the L2 needs room
        asm volatile("s_add_u32 m0, %3, %5\n\ts_nop 0\n\tbuffer_load_dwordx4 %0, %1, %2 offen offset:%4 nt lds"
                     ::"v"(voff), "s"(rsrc), "s"(soff), "s"(lds_base), "n"(IMM), "n"(LDS_IMM - IMM) : "memory", "scc");
    else
        asm volatile("s_add_u32 m0, %3, %5\n\ts_nop 0\n\tbuffer_load_dwordx4 %0, %1, %2 offen offset:%4 lds"
                     ::"v"(voff), "s"(rsrc), "s"(soff), "s"(lds_base), "n"(IMM), "n"(LDS_IMM - IMM) : "memory", "scc");
}
template <int IMM, int LDS_IMM>
__device__ __forceinline__ void vm_dma_b32(int voff, v4i rsrc, int soff, u32 lds_base)
{
    asm volatile("s_add_u32 m0, %3, %5\n\ts_nop 0\n\tbuffer_load_dword %0, %1, %2 offen offset:%4 lds"
                 ::"v"(voff), "s"(rsrc), "s"(soff), "s"(lds_base), "n"(IMM), "n"(LDS_IMM - IMM) : "memory", "scc");
}
// The same for descriptors that were just made uniform with v_readfirstlane: a vector-memory instruction must not
// read a scalar register earlier than 5 wait states after a vector instruction wrote it, and the compiler does
// not look into inline assembly for that (tests/test_build_checks.py scans the generated code for the pattern).
__device__ __forceinline__ void vm_dma_b32_fresh_sgprs(int voff, v4i rsrc, u32 lds_base)
{
    asm volatile("s_nop 4\n\ts_mov_b32 m0, %2\n\ts_nop 0\n\tbuffer_load_dword %0, %1, 0 offen lds"
                 ::"v"(voff), "s"(rsrc), "s"(lds_base) : "memory");
}
__device__ __forceinline__ u32 lds_addr_of(const void* p)
{
    return (u32)(unsigned long long)(__attribute__((address_space(3))) const void*)p;
}
// all but the N youngest VMEM operations have completed; the registers named are (re)defined here, so
// their consumers cannot be scheduled above the wait
template <int N>
__device__ __forceinline__ void wait_vm_tiles(v4i& a, v4i& b, v4i& c, v4i& d)
{
    asm volatile("s_waitcnt vmcnt(%4)" : "+v"(a), "+v"(b), "+v"(c), "+v"(d) : "n"(N));
}
template <int N>
__device__ __forceinline__ void wait_vm_scales(int& a, int& b, int& c, int& d)
{
    asm volatile("s_waitcnt vmcnt(%4)" : "+v"(a), "+v"(b), "+v"(c), "+v"(d) : "n"(N));
}
template <int N>
__device__ __forceinline__ void wait_vmcnt_barrier()
{
    // own DMA writes complete (all but the N youngest VMEM ops), own LDS reads complete, then meet
    asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(N) : "memory");
}

// 4x4 transpose of dwords across the four 16-lane rows of a wave: in: x[j] of lane row kb;
// out: x[c] of lane row q holds what x[q] of lane row c held.  (permlane32_swap exchanges lanes
// 32..63 of its first operand with lanes 0..31 of its second; permlane16_swap exchanges the odd
// 16-lane rows of its first operand with the even rows of its second.)
__device__ __forceinline__ void transpose4x4_rows(u32 (&x)[4])
{
    typedef unsigned v2u __attribute__((ext_vector_type(2)));
    v2u t;
    t = __builtin_amdgcn_permlane32_swap(x[0], x[2], false, false); x[0] = t.x; x[2] = t.y;
    t = __builtin_amdgcn_permlane32_swap(x[1], x[3], false, false); x[1] = t.x; x[3] = t.y;
    t = __builtin_amdgcn_permlane16_swap(x[0], x[1], false, false); x[0] = t.x; x[1] = t.y;
    t = __builtin_amdgcn_permlane16_swap(x[2], x[3], false, false); x[2] = t.x; x[3] = t.y;
}

struct TileId
{
    int m_blk, nt, e;   // row block, weight tile, (local) expert; all wave-uniform
    bool valid;
};

// ---- accumulators and epilogue of one wave's part of a tile.  A wave owns MT row groups of 16 rows x 4 weight row
// groups (stage 1: groups 0, 1 are gate rows, 2, 3 the matching up rows); the accumulator of (weight row group j, row
// group mt) is a[(j*MT + mt)*4 .. +3].
template <int MT>
__device__ __forceinline__ void gemm_zero_acc(v4f* xacc = nullptr)
{
    static_for<(16 * MT < 256 ? 16 * MT : 256)>([&](auto R) __attribute__((always_inline)) { acc_fixed_zero<decltype(R)::value>(); });
    if constexpr(16 * MT > 256)
#pragma unroll
        for(int i = 0; i < (16 * MT - 256) / 4; i++)
            xacc[i] = (v4f){0.f, 0.f, 0.f, 0.f};
}
// the four accumulators of row group MTI, plus bias when the instance has one (bias4(j) = the address of the lane's
// four bf16 biases of weight row group j; re-read per row group to keep the epilogue's register need small)
template <int MT, int MTI, bool BIAS, typename B>
__device__ __forceinline__ void gemm_fetch_row(v4f (&row)[4], B bias4, const v4f* xacc)
{
    static_for<4>([&](auto J) __attribute__((always_inline)) {
        constexpr int j = decltype(J)::value, a0 = (j * MT + MTI) * 4;
        if constexpr(a0 >= 256)
            row[j] = xacc[MTI - ACC_SPILL_MT0];
        else
            row[j] = (v4f){acc_fixed_read<a0>(), acc_fixed_read<a0 + 1>(), acc_fixed_read<a0 + 2>(), acc_fixed_read<a0 + 3>()};
        if constexpr(BIAS)
        {
            const uint2 b = *(const uint2*)bias4(j);
            row[j][0] += bf16_bits_to_f32((uint16_t)b.x);
            row[j][1] += bf16_bits_to_f32((uint16_t)(b.x >> 16));
            row[j][2] += bf16_bits_to_f32((uint16_t)b.y);
            row[j][3] += bf16_bits_to_f32((uint16_t)(b.y >> 16));
        }
    });
}
// e, nt: (local) expert and weight tile; row0: sorted position of the wave's first row; wcol: which 64 (stage 1: 32 + 32)
// of the tile's weight rows the wave owns; meta: the sorted ids of the wave's rows, their routing weights mpad words
// further; ma: how many of the wave's row groups hold real rows (a prefix; may be <= 0).  BIAS: the layer has biases
// (the kernel branches once per tile between the two instances).
//
// With one wave per SIMD (the tiles above 128 rows) nothing else runs while a wave is in its epilogue, so the row groups
// are taken two at a time and everything up to the stores is one stretch of code without branches: the second group's
// accumulator reads, conversions and lane exchanges fill the latencies of the first one's (the transcendental pipeline,
// the exchanges).  The tiles up to 128 rows have two or more waves per SIMD for that, and no registers for a second group.
template <int STAGE, int MT, int ACT, bool ATOMIC, bool BIAS>
__device__ __forceinline__ void gemm_epilogue(const GemmArgs& g, int e, int nt, int row0, int wcol, const u32* meta, int mpad,
                                              int ma, int r, int kb, const v4f* xacc = nullptr)
{
    constexpr int PAIR = MT > 8 ? 2 : 1;
    const int I = g.N / 2;   // stage 1 only
    if(STAGE == 1)
    {
        // lane (r, kb) holds channels j*16 + kb*4 .. +3 (j = 0, 1) of row r.  After one permlane16 swap per
        // packed dword a lane holds 8 consecutive channels: one 16 B store, 64 B contiguous per row and wave.
        typedef unsigned v2u __attribute__((ext_vector_type(2)));
        uint16_t* out = (uint16_t*)g.out;
        const int chw = nt * 128 + wcol * 32;
        auto bz = [&](int j) __attribute__((always_inline)) {
            return g.bias + (size_t)e * g.N + (j >> 1) * I + chw + (j & 1) * 16 + kb * 4;
        };
        // after the swap: lane rows 0..3 hold channel offsets 0, 16, 8, 24
        const int ch_out = chw + (kb & 1) * 16 + (kb >> 1) * 8;
        const int blk = nt * 4 + wcol, jb = blk & 15;              // scale byte: see moe_quant.hip
        const int s_col = (blk & ~15) + (jb & 3) * 4 + (jb >> 2);
        static_for<(MT + PAIR - 1) / PAIR>([&](auto GI) __attribute__((always_inline)) {
            constexpr int m0 = decltype(GI)::value * PAIR;
            constexpr int NP = m0 + PAIR <= MT ? PAIR : MT - m0;       // row groups of this pair
            uint4 o[NP];
            u32 q4[NP], e8[NP];
#pragma unroll
            for(int q = 0; q < NP; q++)
                o[q] = make_uint4(0u, 0u, 0u, 0u);                // row groups that hold only padding store zeros
            if(m0 < ma)                                           // (a pair leaves together: a padding group next to a real one computes)
            {
                u32 ids[NP];
#pragma unroll
                for(int q = 0; q < NP; q++)
                    ids[q] = meta[(m0 + q) * 16 + r];
                static_for<NP>([&](auto Q) __attribute__((always_inline)) {
                    constexpr int q = decltype(Q)::value, mt = m0 + q;
                    v4f row[4];
                    gemm_fetch_row<MT, mt, BIAS>(row, bz, xacc);
                    u32 d[2][2];
#pragma unroll
                    for(int j = 0; j < 2; j++)
                    {
                        float v[4];
#pragma unroll
                        for(int i = 0; i < 4; i++)
                            v[i] = ACT == 0 ? silu_f32(row[j][i]) * row[j + 2][i] : swiglu_f32(row[j][i], row[j + 2][i], g.limit);
                        d[j][0] = pack_bf16x2(v[0], v[1]);
                        d[j][1] = pack_bf16x2(v[2], v[3]);
                    }
                    v2u t0 = __builtin_amdgcn_permlane16_swap(d[0][0], d[1][0], false, false);
                    v2u t1 = __builtin_amdgcn_permlane16_swap(d[0][1], d[1][1], false, false);
                    // even lane rows: x = (kb, j0), y = (kb+1, j0); odd lane rows: x = (kb-1, j1), y = (kb, j1)
                    const bool ok = (int)(ids[q] >> 24) < g.topk;          // padding rows store zeros
                    o[q] = make_uint4(ok ? t0.x : 0u, ok ? t1.x : 0u, ok ? t0.y : 0u, ok ? t1.y : 0u);
                });
            }
            // the wave's 32 channels of a row are exactly one MX block (8 channels in each of the four lane rows): block
            // maximum across the lane rows, then the same arithmetic as the stand-alone quantiser (moe_quant.hip) on the
            // bf16-rounded values, so both paths agree bit for bit
            if(g.out_q)
            {
#pragma unroll
                for(int q = 0; q < NP; q++)
                {
                    u32 am  = amax15_fold(amax15x2(amax15x2(o[q].x, o[q].y), amax15x2(o[q].z, o[q].w)));
                    v2u s16 = __builtin_amdgcn_permlane16_swap(am, am, false, false);
                    am      = s16.x > s16.y ? s16.x : s16.y;
                    v2u s32 = __builtin_amdgcn_permlane32_swap(am, am, false, false);
                    am      = s32.x > s32.y ? s32.x : s32.y;
                    e8[q]   = mx_scale_byte(am);
                    q4[q]   = cvt8(o[q], mx_inv_scale(e8[q]));
                }
#pragma unroll
                for(int q = 0; q < NP; q++)
                {
                    const size_t p = (size_t)(row0 + (m0 + q) * 16 + r);
                    *(u32*)(g.out_q + p * (I / 2) + ch_out / 2) = q4[q];
                    if(kb == 0)
                        g.out_s[p * g.OSK + s_col] = (uint8_t)e8[q];
                }
            }
            if(out)
#pragma unroll
                for(int q = 0; q < NP; q++)
                    *(uint4*)(out + (size_t)(row0 + (m0 + q) * 16 + r) * I + ch_out) = o[q];
            __builtin_amdgcn_sched_barrier(0);      // a pair of row groups at a time: keeps the temporaries few
        });
    }
    else
    {
        // lane (r, kb) holds channels j*16 + kb*4 .. +3 (j = 0..3) of row r.  A 4x4 transpose across the
        // four lane rows gives every lane 16 consecutive channels: 32 B stores, 128 B contiguous per row.
        uint16_t* out = (uint16_t*)g.out;
        const int chw = nt * 256 + wcol * 64;
        auto bz = [&](int j) __attribute__((always_inline)) { return g.bias + (size_t)e * g.N + chw + j * 16 + kb * 4; };
        const int lane_col  = chw + kb * 16;
        const u32 row_bytes = (u32)g.N * 2u;
        static_for<(MT + PAIR - 1) / PAIR>([&](auto GI) __attribute__((always_inline)) {
            constexpr int m0 = decltype(GI)::value * PAIR;
            constexpr int NP = m0 + PAIR <= MT ? PAIR : MT - m0;
            if(m0 >= ma)
                return;
            u32 ids[NP], rws[NP];
#pragma unroll
            for(int q = 0; q < NP; q++)
            {
                ids[q] = meta[(m0 + q) * 16 + r];
                rws[q] = meta[mpad + (m0 + q) * 16 + r];
            }
            u32 lo[NP][4], hi[NP][4];
            static_for<NP>([&](auto Q) __attribute__((always_inline)) {
                constexpr int q = decltype(Q)::value, mt = m0 + q;
                v4f row[4];
                gemm_fetch_row<MT, mt, BIAS>(row, bz, xacc);
                const float rw = __builtin_bit_cast(float, rws[q]);
#pragma unroll
                for(int j = 0; j < 4; j++)
                {
                    lo[q][j] = pack_bf16x2(row[j][0] * rw, row[j][1] * rw);
                    hi[q][j] = pack_bf16x2(row[j][2] * rw, row[j][3] * rw);
                }
                transpose4x4_rows(lo[q]);
                transpose4x4_rows(hi[q]);
                // lane row c now holds channels c*16 + i*4 .. +3 in (lo[i], hi[i])
            });
#pragma unroll
            for(int q = 0; q < NP; q++)
            {
                const u32 tok = ids[q] & 0xFFFFFFu, slot = ids[q] >> 24;
                const bool ok = (int)slot < g.topk && (int)tok < g.T;       // (a padding group next to a real one: all false)
                if(ok && STAGE == 3)
                {
                    // the rows are read by whichever workgroup completes the token (gemm_arrive_reduce), possibly on another
                    // XCD with an L2 of its own: stores at device scope (written through), as the compiler emits them for an
                    // atomic store of that scope
                    const u32 orow               = tok * (u32)g.topk + slot;
                    const unsigned long long dst = (unsigned long long)(out + lane_col) + (unsigned long long)orow * row_bytes;
                    const v4i d0 = {(int)lo[q][0], (int)hi[q][0], (int)lo[q][1], (int)hi[q][1]};
                    const v4i d1 = {(int)lo[q][2], (int)hi[q][2], (int)lo[q][3], (int)hi[q][3]};
                    asm volatile("global_store_dwordx4 %0, %1, off sc1\n\tglobal_store_dwordx4 %0, %2, off offset:16 sc1"
                                 ::"v"(dst), "v"(d0), "v"(d1) : "memory");
                }
                if(ok && !ATOMIC && STAGE != 3)
                {
                    // (plain stores: marked non-temporal they cost the down GEMM 5 % and the reduction, which then finds
                    // nothing of out3 in the last-level cache, another 4 %)
                    const u32 orow = tok * (u32)g.topk + slot;              // row of out3 [tokens * topk, N]
                    uint4* dst = (uint4*)((unsigned long long)(out + lane_col) + (unsigned long long)orow * row_bytes);
                    dst[0]     = make_uint4(lo[q][0], hi[q][0], lo[q][1], hi[q][1]);
                    dst[1]     = make_uint4(lo[q][2], hi[q][2], lo[q][3], hi[q][3]);
                }
                if(ok && ATOMIC)
                {
                    typedef short v2s __attribute__((ext_vector_type(2)));
                    auto* dst = (__attribute__((address_space(1))) v2s*)((unsigned long long)(out + lane_col) + (unsigned long long)tok * row_bytes);
#pragma unroll
                    for(int c = 0; c < 4; c++)
                    {
                        __builtin_amdgcn_global_atomic_fadd_v2bf16(dst + 2 * c, __builtin_bit_cast(v2s, lo[q][c]));
                        __builtin_amdgcn_global_atomic_fadd_v2bf16(dst + 2 * c + 1, __builtin_bit_cast(v2s, hi[q][c]));
                    }
                }
            }
            __builtin_amdgcn_sched_barrier(0);      // a pair of row groups at a time: keeps the temporaries few
        });
    }
}

// Stage 3: the top-k reduction inside the down GEMM, by the last arriver.  g.arrive[token, weight tile] starts at the
// number of the token's slots that take part in the layer (moe_pair_is_kept; written by moe_arrive_init_kernel).  When a
// tile's rows have been stored to out3 (device-scope stores, waited for by every wave, then a workgroup barrier), the
// workgroup takes one off the counter of every real row; the workgroup that takes the last one sums the token's
// slots for these 256 channels from out3 in slot order in fp32 and writes the layer output: the arithmetic of
// moe_topk_reduce_kernel<.., true>, so the result is the same bit for bit and does not depend on who arrives when.
// Nobody waits for anybody.  The counter is a device-scope atomic (it orders the arrivals: whoever reads 1 knows that
// all other slots' stores were complete before their owners decremented), and the rows are read with device-scope
// loads, because the slots of a token come from up to topk different XCDs whose L2s are not coherent with each other.
// lds: at least (1 + rows) words that nobody else touches until the function returns (it ends with a barrier).
template <int MT>
__device__ __forceinline__ void gemm_arrive_reduce(const GemmArgs& g, int nt, const u32* meta, int ma, u32* lds)
{
    const int tid = threadIdx.x;
    if(tid == 0)
        lds[0] = 0;
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");     // this wave's stores of the tile are complete
    __syncthreads();                                     // ... and so are the other waves'
    for(int row = tid; row < ma * 16; row += GEMM_THREADS)
    {
        const u32 id  = meta[row];
        const u32 tok = id & 0xFFFFFFu, slot = id >> 24;
        if((int)slot < g.topk && (int)tok < g.T)
        {
            const int old = __hip_atomic_fetch_sub(g.arrive + (size_t)tok * g.n_tiles + nt, 1, __ATOMIC_RELAXED,
                                                   __HIP_MEMORY_SCOPE_AGENT);
            if(old == 1)
                lds[1 + atomicAdd(&lds[0], 1u)] = tok;
        }
    }
    __syncthreads();
    const int n = (int)lds[0];
    // 32 lanes per token, 8 channels (16 bytes) each
    const int sub = tid & 31;
    for(int i = tid >> 5; i < n; i += GEMM_THREADS / 32)
    {
        const u32 tok = lds[1 + i];
        const int col = nt * 256 + sub * 8;
        float acc[8];
#pragma unroll
        for(int c = 0; c < 8; c++)
            acc[c] = 0.f;
        // NB slots at a time (eight where the tile has registers for it, one in the tiles that run two or more workgroups
        // per CU on 128 registers): their loads go out together and are waited for once.  The loads are unconditional
        // (straight-line code between a load and its wait: nothing for the compiler to copy while the load is in flight); a
        // slot that is left out is read all the same, from memory that nobody wrote, and replaced by +0.0, which leaves
        // every sum unchanged, as in the reduction kernel.
        constexpr int NB = MT > 8 ? 8 : 1;
        for(int s0 = 0; s0 < g.topk; s0 += NB)
        {
            v4i v[NB];
            bool on[NB];
            unsigned long long src[NB];
#pragma unroll
            for(int j = 0; j < NB; j++)
            {
                const int sl = s0 + j < g.topk ? s0 + j : g.topk - 1;
                on[j]  = s0 + j < g.topk && moe_pair_is_kept(g.topk_ids[(size_t)tok * g.topk + sl], g.experts_all, g.expert_mask);
                src[j] = (unsigned long long)((const uint16_t*)g.out + ((size_t)tok * g.topk + sl) * g.N + col);
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for(int j = 0; j < NB; j++)
                asm volatile("global_load_dwordx4 %0, %1, off sc1" : "=&v"(v[j]) : "v"(src[j]) : "memory");
            if constexpr(NB == 8)
                asm volatile("s_waitcnt vmcnt(0)" : "+v"(v[0]), "+v"(v[1]), "+v"(v[2]), "+v"(v[3]), "+v"(v[4]), "+v"(v[5]),
                             "+v"(v[6]), "+v"(v[7])::"memory");
            else
                asm volatile("s_waitcnt vmcnt(0)" : "+v"(v[0])::"memory");
#pragma unroll
            for(int j = 0; j < NB; j++)
#pragma unroll
                for(int c = 0; c < 4; c++)
                {
                    const u32 w = on[j] ? (u32)v[j][c] : 0u;
                    acc[2 * c]     += __builtin_bit_cast(float, w << 16);
                    acc[2 * c + 1] += __builtin_bit_cast(float, w & 0xFFFF0000u);
                }
        }
        if(g.final_f32)
        {
            float4* dst = (float4*)((float*)g.final_out + (size_t)tok * g.N + col);
            dst[0]      = make_float4(acc[0], acc[1], acc[2], acc[3]);
            dst[1]      = make_float4(acc[4], acc[5], acc[6], acc[7]);
        }
        else
            *(uint4*)((uint16_t*)g.final_out + (size_t)tok * g.N + col) =
                make_uint4(pack_bf16x2(acc[0], acc[1]), pack_bf16x2(acc[2], acc[3]), pack_bf16x2(acc[4], acc[5]),
                           pack_bf16x2(acc[6], acc[7]));
    }
    __syncthreads();                                     // the list is somebody's buffer again from here on
}

// compute units of the current device (asked once per device, then remembered)
static inline int device_cu_count()
{
    static int cached[64] = {0};
    int dev = 0;
    if(hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64)
        return 256;
    int cus = __atomic_load_n(&cached[dev], __ATOMIC_RELAXED);
    if(cus == 0)
    {
        if(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
            cus = 256;
        __atomic_store_n(&cached[dev], cus, __ATOMIC_RELAXED);
    }
    return cus;
}

