// Token routing sort: group (token, slot) pairs by expert, keep (token, slot) order inside an
// expert, pad every expert's run to the block size.
//
// Output contract (what the reference's callers read, src/contrib/fused_moe.py:56-100 and
// archive/ck_tile/ck_tile/host/reference/reference_moe_sorting.hpp:13-117):
//   sorted_ids[p]        = (slot << 24) | token, padding = (topk << 24) | num_tokens
//   sorted_weights[p]    = routing weight, padding = 0
//   sorted_expert_ids[b] = (local) expert of block b; 0xFFFFFFFF past the last valid block
//   num_valid_ids        = { padded total, number of (local) tokens }
// The order is deterministic (no atomics decide a position): a pair's position is
//   expert_offset[e] + (#pairs of e in earlier workgroups) + (#pairs of e in earlier waves of this
//   workgroup) + (#pairs of e earlier in this wave's chunk).
//
// Three launches for large inputs (histogram -> scan -> scatter) and one single-workgroup
// launch for small inputs.
#include "common.h"
#include "quant_device.h"
#include "router_device.h"

#define SORT_THREADS 256
#define SORT_WAVES (SORT_THREADS / WAVE)
#define SMALL_THREADS 1024
#define SMALL_WAVES (SMALL_THREADS / WAVE)
#define SMALL_GROUPS 2      // groups of 64 pairs a wave of the single-workgroup sort holds in registers
#define SORT_GROUPS 4       // the same for a wave of the multi-workgroup sort
#define EXPERT_FILL 0xFFFFFFFFu

struct SortArgs
{
    const int* topk_ids;       // [T_all, k]
    const float* topk_w;       // [T_all, k]
    const int* expert_mask;    // [E] or null
    const int* num_local_tok;  // device scalar or null
    u32* sorted_ids;
    float* sorted_w;
    u32* sorted_e;
    u32* num_valid;
    u32* ws;                   // workspace: hist[G][E], then per-expert offset[E]
    u32* sched;                // optional tile schedule for the grouped GEMMs (see write_schedule) or null
    int T_all, k, E, Bm, n_blk, G;
};

// routing done by the sort's own workgroup (single-workgroup sort only): gating scores in, the top-k picks written
// to the buffers the sort then reads its pairs from
struct RouteArgs
{
    const float* gating;       // [T_all, E] (E = 64 * NE) or null: the pairs are given
    float* topk_w;             // [T_all, k] out
    int* topk_ids;             // [T_all, k] out
    int n_group, topk_group, renorm;
};

__device__ __forceinline__ int sort_tokens(const SortArgs& a)
{
    int T = a.T_all;
    if(a.num_local_tok)
    {
        int t = *a.num_local_tok;
        T     = t < 0 ? 0 : (t < T ? t : T);
    }
    return T;
}

// pairs handled by one wave: a multiple of 64 so that waves never share a 64-pair group
__device__ __forceinline__ int wave_chunk(int pairs, int total_waves)
{
    int c = (pairs + total_waves - 1) / total_waves;
    return (c + WAVE - 1) / WAVE * WAVE;
}

// Up to NG groups of 64 consecutive pairs of one wave, held in registers: all their loads are in flight together
// (a loop of load -> use -> load pays one memory round trip per group), and the scatter reuses what the
// histogram loaded.  e < 0 marks a pair that is dropped (out of range, masked expert, past the end).
template <int NG>
struct WavePairs
{
    int e[NG];
    float w[NG];

    // pairs [beg, min(end, beg + NG*64))
    __device__ __forceinline__ void load(const SortArgs& a, int beg, int end, bool with_weights)
    {
        const int lane = lane_id();
#pragma unroll
        for(int g = 0; g < NG; g++)
        {
            const int i = beg + g * WAVE + lane;
            e[g]        = i < end ? a.topk_ids[i] : -1;
            w[g]        = (with_weights && i < end) ? a.topk_w[i] : 0.f;
        }
#pragma unroll
        for(int g = 0; g < NG; g++)
        {
            if(!moe_pair_is_kept(e[g], a.E, a.expert_mask))
                e[g] = -1;
        }
    }

    // histogram into h[E] (LDS) shared with other waves
    __device__ __forceinline__ void hist_atomic(u32* h) const
    {
#pragma unroll
        for(int g = 0; g < NG; g++)
            if(e[g] >= 0)
                atomicAdd(&h[e[g]], 1u);
    }

    // Within a group of 64 pairs every lane finds the lanes that hold the same expert from one ballot per bit of
    // the expert id (a constant number of steps, however many distinct experts the group holds).  Kept per group:
    // the lane's rank among them (bits 0-7), their number (bits 8-15) and whether the lane is the lowest (bit 16).
    u32 rc[NG];
    __device__ __forceinline__ void match(const SortArgs& a, int beg, int end)
    {
        const int lane  = lane_id();
        const u64 lt    = (1ull << lane) - 1ull;
        const int nbits = 32 - __builtin_clz((unsigned)(a.E > 1 ? a.E - 1 : 1));
#pragma unroll
        for(int g = 0; g < NG; g++)
        {
            rc[g] = 0;
            if(beg + g * WAVE >= end)      // uniform
                continue;
            const bool keep = e[g] >= 0;
            u64 m           = __ballot(keep);
            for(int b = 0; b < nbits; b++)
            {
                const bool bit = (e[g] >> b) & 1;
                const u64 bal  = __ballot(keep && bit);
                m &= bit ? bal : ~bal;
            }
            rc[g] = (u32)__popcll(m & lt) | ((u32)__popcll(m) << 8) | ((m & lt) == 0 ? 1u << 16 : 0u);
        }
    }

    // histogram into h[E] (LDS) private to this wave, after match(): the lowest lane of every expert adds the count
    // (no atomics: the experts of a group are distinct addresses, and a wave's LDS operations execute in order)
    __device__ __forceinline__ void hist_private(u32* h) const
    {
#pragma unroll
        for(int g = 0; g < NG; g++)
            if(e[g] >= 0 && (rc[g] >> 16))
                h[e[g]] += (rc[g] >> 8) & 0xFFu;
    }

    // after match(): writes the pairs to their final positions; base[e] (LDS, private to this wave) is the position
    // of the wave's first pair of expert e and is advanced by the lowest lane as groups are consumed
    __device__ __forceinline__ void scatter(const SortArgs& a, u32* base, int beg, int end) const
    {
        const int lane = lane_id();
#pragma unroll
        for(int g = 0; g < NG; g++)
        {
            if(beg + g * WAVE >= end)      // uniform
                break;
            const int i = beg + g * WAVE + lane;
            if(e[g] >= 0)
            {
                const u32 b0      = base[e[g]];
                const u32 pos     = b0 + (rc[g] & 0xFFu);
                const u32 tok     = (u32)(i / a.k);
                const u32 slot    = (u32)(i - (int)tok * a.k);
                a.sorted_ids[pos] = (slot << 24) | tok;
                a.sorted_w[pos]   = w[g];
                if(rc[g] >> 16)                 // every lane of this expert has read base[e] above (one instruction)
                    base[e[g]] = b0 + ((rc[g] >> 8) & 0xFFu);
            }
        }
    }
};

// per-expert padded offsets from per-expert totals; one workgroup, any thread count that is a
// multiple of 64.  tot[e] in, off[e] (exclusive prefix of padded sizes) and lid[e] out; returns
// the padded total to every thread.  scratch: >= blockDim/64 + 1 words of LDS.
__device__ __forceinline__ u32 expert_offsets(const SortArgs& a, const u32* tot, u32* off, u32* lid,
                                              u32* scratch)
{
    const int nw   = blockDim.x / WAVE;
    const int lane = lane_id(), wave = threadIdx.x / WAVE;
    u32 run_pad = 0, run_id = 0;
    for(int e0 = 0; e0 < a.E; e0 += blockDim.x)
    {
        int e     = e0 + threadIdx.x;
        bool on   = moe_pair_is_kept(e, a.E, a.expert_mask);
        u32 pad   = (on && e < a.E) ? (tot[e] + a.Bm - 1) / a.Bm * a.Bm : 0u;
        u32 one   = on ? 1u : 0u;
        // inclusive scan inside the wave (two values packed: padded size, mask count)
        u32 sp = pad, si = one;
        for(int d = 1; d < WAVE; d <<= 1)
        {
            u32 tp = __shfl_up(sp, d), ti = __shfl_up(si, d);
            if(lane >= d)
            {
                sp += tp;
                si += ti;
            }
        }
        __syncthreads();
        if(lane == WAVE - 1)
        {
            scratch[wave]      = sp;
            scratch[nw + wave] = si;
        }
        __syncthreads();
        u32 bp = 0, bi = 0, allp = 0, alli = 0;
        for(int w = 0; w < nw; w++)
        {
            u32 p = scratch[w], q = scratch[nw + w];
            if(w < wave)
            {
                bp += p;
                bi += q;
            }
            allp += p;
            alli += q;
        }
        if(e < a.E)
        {
            off[e] = run_pad + bp + sp - pad;
            lid[e] = a.expert_mask ? run_id + bi + si - one : (u32)e;
        }
        run_pad += allp;
        run_id += alli;
    }
    __syncthreads();
    return run_pad;
}

// Every position of sorted_ids / sorted_weights gets the padding entry.  Depends on nothing the sort computes, so
// it is issued first and overlaps the loads of the pairs; the scatter overwrites the positions that hold pairs
// and must be ordered after it (a later launch, or a device-scope fence and a barrier in between).
__device__ __forceinline__ void fill_padding(const SortArgs& a, int T, u32 tid, u32 nthreads)
{
    const u32 pad_id = ((u32)a.k << 24) | ((u32)T & 0xFFFFFFu);
    const u32 n      = (u32)a.n_blk * (u32)a.Bm;
    for(u32 p = tid; p < n; p += nthreads)
    {
        a.sorted_ids[p] = pad_id;
        a.sorted_w[p]   = 0.f;
    }
}

// the block -> expert table and num_valid; one workgroup, 16 lanes share the blocks of an expert
__device__ __forceinline__ void fill_blocks(const SortArgs& a, const u32* tot, const u32* off, const u32* lid,
                                            u32 padded_total, int T)
{
    const u32 tid = threadIdx.x, nthreads = blockDim.x;
    for(u32 e = tid / 16; e < (u32)a.E; e += nthreads / 16)
    {
        if(tot[e] == 0 || !moe_pair_is_kept((int)e, a.E, a.expert_mask))
            continue;
        const u32 b0 = off[e] / a.Bm, b1 = b0 + (tot[e] + a.Bm - 1) / a.Bm;
        for(u32 b = b0 + tid % 16; b < b1; b += 16)
            a.sorted_e[b] = lid[e];
    }
    for(u32 b = padded_total / a.Bm + tid; b < (u32)a.n_blk; b += nthreads)
        a.sorted_e[b] = EXPERT_FILL;
    if(tid == 0)
    {
        a.num_valid[0] = padded_total;
        a.num_valid[1] = (u32)T;
    }
}

// Tile schedule for the persistent grouped GEMMs: the table from which every workgroup finds its tiles without
// looking at sorted_expert_ids.  Layout (u32 words):
//   sched[e], e = 0..E   : number of row blocks of the experts before e (sched[E] = all row blocks); the row blocks
//                          of expert e are sched[e] .. sched[e+1]-1
//   sched[E + 1 + e]     : local id of expert e (its index among the unmasked experts)
// A GEMM orders its tiles expert -> weight tile -> row block and cuts that list into 8 equal runs, one per XCD
// (moe_gemm_mxfp4.hip), so the XCDs get the same number of tiles however unevenly the router loads the experts.
__device__ __forceinline__ void write_schedule(const SortArgs& a, const u32* off, const u32* lid, u32 padded_total)
{
    if(!a.sched)
        return;
    for(int e = threadIdx.x; e < a.E; e += blockDim.x)
    {
        a.sched[e]           = off[e] / a.Bm;
        a.sched[a.E + 1 + e] = lid[e];
    }
    if(threadIdx.x == 0)
        a.sched[a.E] = padded_total / a.Bm;
}

// ---------------------------------------------------------------------------------------------
// single workgroup: everything in one launch (up to SMALL_GROUPS * 64 pairs per wave)
// LDS: whist[SMALL_WAVES][E] | tot[E] | off[E] | lid[E] | scratch[2*SMALL_WAVES]
// Workgroups past the first quantise activations (qa.rows > 0): the input quantisation of the MXFP4-activation
// path depends on nothing the sort computes, and carrying it in this launch saves a dispatch.
// NE > 0: the workgroup first routes the tokens itself (a wave per token, tokens dealt round-robin to its 16 waves;
// the step before the sort, aiter.fused_topk at tests/contrib/moe/test_fused_moe.py:38,87, costs no launch of its own).
template <int NE, bool GROUPED>
__global__ void __launch_bounds__(SMALL_THREADS) moe_sort_small_kernel(SortArgs a, QuantArgs qa, RouteArgs ra)
{
    if(blockIdx.x > 0)
    {
        act_quant_block(qa, (long long)(blockIdx.x - 1) * SMALL_THREADS + threadIdx.x);
        return;
    }
    extern __shared__ u32 lds[];
    u32* whist   = lds;
    u32* tot     = whist + SMALL_WAVES * a.E;
    u32* off     = tot + a.E;
    u32* lid     = off + a.E;
    u32* scratch = lid + a.E;
    const int T     = sort_tokens(a);
    const int pairs = T * a.k;
    const int wave  = threadIdx.x / WAVE;
    const int cv    = wave_chunk(pairs, SMALL_WAVES);
    const int beg   = min(pairs, wave * cv), end = min(pairs, beg + cv);

    if constexpr(NE > 0)
    {
        const int lane = lane_id();
        for(int t = wave; t < a.T_all; t += SMALL_WAVES)
        {
            float w;
            int id;
            route_token<NE, GROUPED>(ra.gating + (size_t)t * a.E, lane, a.k, ra.n_group, ra.topk_group, ra.renorm, w, id);
            if(lane < a.k)
            {
                ra.topk_w[(size_t)t * a.k + lane]   = w;
                ra.topk_ids[(size_t)t * a.k + lane] = id;
            }
        }
        // the picks reach the L2 before any wave of this workgroup reads them back as the sort's pairs (these
        // addresses have not been read by this kernel before, so no stale line can sit in the CU's cache)
        __threadfence();
        __syncthreads();
    }

    WavePairs<SMALL_GROUPS> wp;
    wp.load(a, beg, end, true);
    fill_padding(a, T, threadIdx.x, SMALL_THREADS);
    for(int i = threadIdx.x; i < SMALL_WAVES * a.E; i += SMALL_THREADS)
        whist[i] = 0;
    __syncthreads();
    wp.match(a, beg, end);
    wp.hist_private(whist + wave * a.E);
    __syncthreads();
    // exclusive prefix over waves, per expert
    for(int e = threadIdx.x; e < a.E; e += SMALL_THREADS)
    {
        u32 run = 0;
        for(int w = 0; w < SMALL_WAVES; w++)
        {
            u32 c             = whist[w * a.E + e];
            whist[w * a.E + e] = run;
            run += c;
        }
        tot[e] = run;
    }
    __syncthreads();
    u32 padded_total = expert_offsets(a, tot, off, lid, scratch);
    fill_blocks(a, tot, off, lid, padded_total, T);
    write_schedule(a, off, lid, padded_total);
    for(int e = threadIdx.x; e < a.E; e += SMALL_THREADS)
        for(int w = 0; w < SMALL_WAVES; w++)
            whist[w * a.E + e] += off[e];
    // the padding entries have landed (a store leaves the counter when the L2 has it) before any wave of this
    // workgroup, which shares that L2, writes a pair over them
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    wp.scatter(a, whist + wave * a.E, beg, end);
}

// ---------------------------------------------------------------------------------------------
// large inputs, launch 1 of 3: per-workgroup histogram -> ws[g][E]; padding entries everywhere
extern "C" __global__ void __launch_bounds__(SORT_THREADS) moe_sort_hist_kernel(SortArgs a)
{
    extern __shared__ u32 lds[];
    const int T     = sort_tokens(a);
    const int pairs = T * a.k;
    const int cv    = wave_chunk(pairs, a.G * SORT_WAVES);
    const int wid   = blockIdx.x * SORT_WAVES + threadIdx.x / WAVE;
    const int beg   = min(pairs, wid * cv), end = min(pairs, beg + cv);
    fill_padding(a, T, blockIdx.x * SORT_THREADS + threadIdx.x, gridDim.x * SORT_THREADS);
    for(int i = threadIdx.x; i < a.E; i += SORT_THREADS)
        lds[i] = 0;
    __syncthreads();
    WavePairs<SORT_GROUPS> wp;
    for(int s = beg; s < end; s += SORT_GROUPS * WAVE)
    {
        wp.load(a, s, end, false);
        wp.hist_atomic(lds);
    }
    __syncthreads();
    for(int i = threadIdx.x; i < a.E; i += SORT_THREADS)
        a.ws[(size_t)blockIdx.x * a.E + i] = lds[i];
}

// launch 2 of 3 (one workgroup): ws[g][e] -> exclusive prefix over g; offsets; tables
// LDS: tot[E] | off[E] | lid[E] | scratch
// Workgroups past the first quantise activations, as in the single-workgroup sort: the scan is one workgroup
// of serial work during which the rest of the GPU would idle.
extern "C" __global__ void __launch_bounds__(SMALL_THREADS) moe_sort_scan_kernel(SortArgs a, QuantArgs qa)
{
    if(blockIdx.x > 0)
    {
        act_quant_block(qa, (long long)(blockIdx.x - 1) * SMALL_THREADS + threadIdx.x);
        return;
    }
    extern __shared__ u32 lds[];
    u32* tot     = lds;
    u32* off     = tot + a.E;
    u32* lid     = off + a.E;
    u32* scratch = lid + a.E;
    const int T  = sort_tokens(a);
    for(int e = threadIdx.x; e < a.E; e += SMALL_THREADS)
    {
        u32 run = 0;
        for(int g0 = 0; g0 < a.G; g0 += 16)      // 16 independent loads in flight, then their prefix
        {
            u32 c[16];
#pragma unroll
            for(int j = 0; j < 16; j++)
                c[j] = g0 + j < a.G ? __builtin_nontemporal_load(&a.ws[(size_t)(g0 + j) * a.E + e]) : 0u;
#pragma unroll
            for(int j = 0; j < 16; j++)
                if(g0 + j < a.G)
                {
                    a.ws[(size_t)(g0 + j) * a.E + e] = run;
                    run += c[j];
                }
        }
        tot[e] = run;
    }
    __syncthreads();
    u32 padded_total = expert_offsets(a, tot, off, lid, scratch);
    u32* g_off       = a.ws + (size_t)a.G * a.E;
    for(int e = threadIdx.x; e < a.E; e += SMALL_THREADS)
        g_off[e] = off[e];
    fill_blocks(a, tot, off, lid, padded_total, T);
    write_schedule(a, off, lid, padded_total);
}

// launch 3 of 3: scatter.  LDS: whist[SORT_WAVES][E]
extern "C" __global__ void __launch_bounds__(SORT_THREADS) moe_sort_scatter_kernel(SortArgs a)
{
    extern __shared__ u32 lds[];
    const int T     = sort_tokens(a);
    const int pairs = T * a.k;
    const int cv    = wave_chunk(pairs, a.G * SORT_WAVES);
    const int wave  = threadIdx.x / WAVE;
    const int wid   = blockIdx.x * SORT_WAVES + wave;
    const int beg   = min(pairs, wid * cv), end = min(pairs, beg + cv);
    for(int i = threadIdx.x; i < SORT_WAVES * a.E; i += SORT_THREADS)
        lds[i] = 0;
    __syncthreads();
    WavePairs<SORT_GROUPS> wp;
    const bool once = end - beg <= SORT_GROUPS * WAVE;      // then the registers still hold the chunk for the scatter
    for(int s = beg; s < end; s += SORT_GROUPS * WAVE)
    {
        wp.load(a, s, end, true);
        wp.match(a, s, end);
        wp.hist_private(lds + wave * a.E);
    }
    __syncthreads();
    const u32* g_off = a.ws + (size_t)a.G * a.E;
    for(int e = threadIdx.x; e < a.E; e += SORT_THREADS)
    {
        u32 run = g_off[e] + a.ws[(size_t)blockIdx.x * a.E + e];
        for(int w = 0; w < SORT_WAVES; w++)
        {
            u32 c            = lds[w * a.E + e];
            lds[w * a.E + e] = run;
            run += c;
        }
    }
    __syncthreads();
    for(int s = beg; s < end; s += SORT_GROUPS * WAVE)
    {
        if(!once)
        {
            wp.load(a, s, end, true);
            wp.match(a, s, end);
        }
        wp.scatter(a, lds + wave * a.E, s, end);
    }
}

// zero fill of the layer output buffer the reference's sorter hands back
extern "C" __global__ void moe_zero_kernel(uint4* p, size_t n16, unsigned char* tail, int ntail)
{
    size_t i      = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    size_t stride = (size_t)gridDim.x * blockDim.x;
    for(; i < n16; i += stride)
        p[i] = make_uint4(0, 0, 0, 0);
    if(blockIdx.x == 0 && (int)threadIdx.x < ntail)
        tail[threadIdx.x] = 0;
}

// zero fill of `bytes` bytes of device memory with a kernel (a memset node does not replay reliably inside a
// captured graph); used for buffers that only some rows are written to
extern "C" int pyhip_moe_zero_fill(void* p, int64_t bytes, hipStream_t stream)
{
    PYHIP_REQUIRE(p && bytes >= 0 && ((uintptr_t)p % 16) == 0, "zero_fill: bad buffer");
    if(bytes == 0)
        return PYHIP_OK;
    size_t n16 = (size_t)bytes / 16;
    int ntail  = (int)(bytes - (int64_t)n16 * 16);
    int grid   = (int)((n16 + 255) / 256);
    grid       = grid < 1 ? 1 : (grid > 2048 ? 2048 : grid);
    hipLaunchKernelGGL(moe_zero_kernel, dim3(grid), dim3(256), 0, stream, (uint4*)p, n16, (unsigned char*)p + n16 * 16,
                       ntail);
    PYHIP_CHECK_LAUNCH("moe_zero_kernel");
    return PYHIP_OK;
}

// ---------------------------------------------------------------------------------------------
#define SMALL_PAIRS_MAX (SMALL_WAVES * SMALL_GROUPS * WAVE)
#define MAX_EXPERTS 2048

static int sort_groups(int64_t pairs)
{
    // workgroups of the large path: at least 1024 pairs each (4 groups of 64 per wave), at most 256 workgroups
    int64_t g = (pairs + 1023) / 1024;
    return (int)(g < 1 ? 1 : (g > 256 ? 256 : g));
}

extern "C" int64_t pyhip_moe_sorting_max_blocks(int64_t tokens, int topk, int experts, int block_size)
{
    return (tokens * topk + (int64_t)experts * (block_size - 1) + block_size - 1) / block_size;
}

extern "C" int64_t pyhip_moe_sorting_workspace_bytes(int64_t tokens, int topk, int experts)
{
    int64_t pairs = tokens * topk;
    if(pairs <= SMALL_PAIRS_MAX)
        return 256;
    return ((int64_t)sort_groups(pairs) + 1) * experts * 4 + 256;
}

extern "C" int64_t pyhip_moe_schedule_words(int experts) { return 2ll * experts + 1; }

// most tokens / experts the single-workgroup sort routes itself; beyond, the router gets a launch of its own
#define ROUTE_SORT_MAX_TOKENS 64
#define ROUTE_SORT_MAX_EXPERTS 512

static int launch_routing_sort(const SortArgs& a, const QuantArgs& qa, const RouteArgs& ra, unsigned qblocks, size_t lds,
                               hipStream_t stream)
{
    const dim3 grid(1 + qblocks), block(SMALL_THREADS);
#define ROUTE_SORT_CASE(N)                                                                                            \
    case N:                                                                                                           \
        if(ra.n_group > 0)                                                                                            \
            hipLaunchKernelGGL((moe_sort_small_kernel<N, true>), grid, block, lds, stream, a, qa, ra);                \
        else                                                                                                          \
            hipLaunchKernelGGL((moe_sort_small_kernel<N, false>), grid, block, lds, stream, a, qa, ra);               \
        break;
    switch(a.E / 64)
    {
        ROUTE_SORT_CASE(1) ROUTE_SORT_CASE(2) ROUTE_SORT_CASE(4) ROUTE_SORT_CASE(8)
    default: pyhip_set_error("moe_route_sorting: experts/64 = %d not in {1,2,4,8}", a.E / 64); return PYHIP_ERR_INVALID;
    }
#undef ROUTE_SORT_CASE
    PYHIP_CHECK_LAUNCH("moe_sort_small_kernel (routing)");
    return PYHIP_OK;
}

static int sorting_impl(const int32_t* topk_ids, const float* topk_weights, int tokens, int topk,
                        int experts, int block_size, const int32_t* expert_mask,
                        const int32_t* num_local_tokens, uint32_t* sorted_ids, float* sorted_weights,
                        uint32_t* sorted_expert_ids, uint32_t* num_valid_ids, uint32_t* schedule,
                        void* moe_out, int64_t moe_out_bytes, void* workspace, int64_t workspace_bytes,
                        QuantArgs qa, RouteArgs ra, hipStream_t stream)
{
    PYHIP_REQUIRE(topk_ids && topk_weights && sorted_ids && sorted_weights && sorted_expert_ids && num_valid_ids,
                  "moe_sorting: null pointer");
    PYHIP_REQUIRE(tokens >= 0 && tokens < (1 << 24), "moe_sorting: tokens=%d outside [0, 2^24)", tokens);
    PYHIP_REQUIRE(topk >= 1 && topk <= 255, "moe_sorting: topk=%d outside [1, 255]", topk);
    PYHIP_REQUIRE(experts >= 1 && experts <= MAX_EXPERTS, "moe_sorting: experts=%d outside [1, %d]", experts,
                  MAX_EXPERTS);
    PYHIP_REQUIRE(block_size >= 1, "moe_sorting: block_size=%d", block_size);
    int64_t pairs = (int64_t)tokens * topk;
    PYHIP_REQUIRE(pairs + (int64_t)experts * block_size < (1ll << 31), "moe_sorting: too many pairs");
    PYHIP_REQUIRE(workspace_bytes >= pyhip_moe_sorting_workspace_bytes(tokens, topk, experts) &&
                      (workspace || workspace_bytes == 0),
                  "moe_sorting: workspace too small");
    SortArgs a;
    a.topk_ids      = topk_ids;
    a.topk_w        = topk_weights;
    a.expert_mask   = expert_mask;
    a.num_local_tok = num_local_tokens;
    a.sorted_ids    = sorted_ids;
    a.sorted_w      = sorted_weights;
    a.sorted_e      = sorted_expert_ids;
    a.num_valid     = num_valid_ids;
    a.ws            = (u32*)workspace;
    a.sched         = schedule;
    a.T_all         = tokens;
    a.k             = topk;
    a.E             = experts;
    a.Bm            = block_size;
    a.n_blk         = (int)pyhip_moe_sorting_max_blocks(tokens, topk, experts, block_size);
    a.G             = 1;
    if(moe_out && moe_out_bytes > 0)
    {
        size_t n16 = (size_t)moe_out_bytes / 16;
        int ntail  = (int)(moe_out_bytes - (int64_t)n16 * 16);
        int grid   = (int)((n16 + 255) / 256);
        grid       = grid < 1 ? 1 : (grid > 2048 ? 2048 : grid);
        hipLaunchKernelGGL(moe_zero_kernel, dim3(grid), dim3(256), 0, stream, (uint4*)moe_out, n16,
                           (unsigned char*)moe_out + n16 * 16, ntail);
        PYHIP_CHECK_LAUNCH("moe_zero_kernel");
    }
    // workgroups that quantise, riding on the single-workgroup launch of either path
    const long long qwork = qa.rows * qa.SK;
    PYHIP_REQUIRE((qwork + SMALL_THREADS - 1) / SMALL_THREADS < (1ll << 31) - 1, "moe_sorting: too many rows to quantise");
    const unsigned qblocks = (unsigned)((qwork + SMALL_THREADS - 1) / SMALL_THREADS);
    if(pairs <= SMALL_PAIRS_MAX)
    {
        size_t lds = ((size_t)(SMALL_WAVES + 3) * experts + 2 * SMALL_WAVES + 2) * 4;
        if(lds > 64 * 1024)
        {
            PYHIP_REQUIRE(!ra.gating, "moe_sorting: the routing sort handles at most %d experts", ROUTE_SORT_MAX_EXPERTS);
            hipError_t e = hipFuncSetAttribute((const void*)moe_sort_small_kernel<0, false>,
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
            PYHIP_REQUIRE(e == hipSuccess, "moe_sorting: cannot reserve %zu B of LDS", lds);
        }
        if(ra.gating)
            return launch_routing_sort(a, qa, ra, qblocks, lds, stream);
        hipLaunchKernelGGL((moe_sort_small_kernel<0, false>), dim3(1 + qblocks), dim3(SMALL_THREADS), lds, stream, a, qa, ra);
        PYHIP_CHECK_LAUNCH("moe_sort_small_kernel");
        return PYHIP_OK;
    }
    a.G = sort_groups(pairs);
    hipLaunchKernelGGL(moe_sort_hist_kernel, dim3(a.G), dim3(SORT_THREADS), (size_t)experts * 4, stream, a);
    PYHIP_CHECK_LAUNCH("moe_sort_hist_kernel");
    hipLaunchKernelGGL(moe_sort_scan_kernel, dim3(1 + qblocks), dim3(SMALL_THREADS),
                       ((size_t)3 * experts + 2 * SMALL_WAVES + 2) * 4, stream, a, qa);
    PYHIP_CHECK_LAUNCH("moe_sort_scan_kernel");
    hipLaunchKernelGGL(moe_sort_scatter_kernel, dim3(a.G), dim3(SORT_THREADS), (size_t)SORT_WAVES * experts * 4,
                       stream, a);
    PYHIP_CHECK_LAUNCH("moe_sort_scatter_kernel");
    return PYHIP_OK;
}

extern "C" int pyhip_moe_sorting(const int32_t* topk_ids, const float* topk_weights, int tokens, int topk,
                                 int experts, int block_size, const int32_t* expert_mask,
                                 const int32_t* num_local_tokens, uint32_t* sorted_ids, float* sorted_weights,
                                 uint32_t* sorted_expert_ids, uint32_t* num_valid_ids, uint32_t* schedule,
                                 void* moe_out, int64_t moe_out_bytes, void* workspace, int64_t workspace_bytes,
                                 hipStream_t stream)
{
    QuantArgs qa = {};
    return sorting_impl(topk_ids, topk_weights, tokens, topk, experts, block_size, expert_mask, num_local_tokens,
                        sorted_ids, sorted_weights, sorted_expert_ids, num_valid_ids, schedule, moe_out, moe_out_bytes,
                        workspace, workspace_bytes, qa, RouteArgs{}, stream);
}

extern "C" int pyhip_moe_sorting_quant(const int32_t* topk_ids, const float* topk_weights, int tokens, int topk,
                                       int experts, int block_size, const int32_t* expert_mask,
                                       const int32_t* num_local_tokens, uint32_t* sorted_ids, float* sorted_weights,
                                       uint32_t* sorted_expert_ids, uint32_t* num_valid_ids, uint32_t* schedule,
                                       void* workspace, int64_t workspace_bytes, const void* x_bf16,
                                       int64_t row_stride_elems, int64_t rows, int K, uint8_t* q, uint8_t* scales,
                                       hipStream_t stream)
{
    QuantArgs qa;
    int rc = pyhip_make_quant_args("moe_sorting_quant", x_bf16, row_stride_elems, rows, K, q, scales, nullptr, &qa);
    if(rc)
        return rc;
    return sorting_impl(topk_ids, topk_weights, tokens, topk, experts, block_size, expert_mask, num_local_tokens,
                        sorted_ids, sorted_weights, sorted_expert_ids, num_valid_ids, schedule, nullptr, 0, workspace,
                        workspace_bytes, qa, RouteArgs{}, stream);
}

int pyhip_check_router(const char* name, const void* logits, const void* w, const void* ids, int tokens, int experts,
                       int topk);
extern "C" int pyhip_moe_topk_softmax(const float*, int, int, int, int, float*, int32_t*, hipStream_t);
extern "C" int pyhip_moe_topk_grouped_sigmoid(const float*, int, int, int, int, int, int, float*, int32_t*, hipStream_t);

// Router + sort (+ optional input quantisation).  Up to ROUTE_SORT_MAX_TOKENS tokens (and pairs that fit the
// single-workgroup sort) everything is ONE launch: the sort's workgroup routes the tokens itself.  Larger inputs take
// the router's own launch followed by the sort; the results are the same either way.
extern "C" int pyhip_moe_route_sorting(const float* gating, int tokens, int topk, int experts, int n_group,
                                       int topk_group, int renormalize, int block_size, const int32_t* expert_mask,
                                       const int32_t* num_local_tokens, float* topk_weight, int32_t* topk_ids,
                                       uint32_t* sorted_ids, float* sorted_weights, uint32_t* sorted_expert_ids,
                                       uint32_t* num_valid_ids, uint32_t* schedule, void* workspace,
                                       int64_t workspace_bytes, const void* x_bf16, int64_t row_stride_elems,
                                       int64_t rows, int K, uint8_t* q, uint8_t* scales, hipStream_t stream)
{
    int rc = pyhip_check_router("moe_route_sorting", gating, topk_weight, topk_ids, tokens, experts, topk);
    if(rc)
        return rc;
    PYHIP_REQUIRE(n_group >= 0 && (n_group == 0 || (n_group <= 64 && (n_group & (n_group - 1)) == 0 &&
                                                   experts % n_group == 0 && topk_group >= 1 && topk_group <= n_group &&
                                                   topk <= topk_group * (experts / n_group))),
                  "moe_route_sorting: n_group=%d topk_group=%d (0 groups = softmax router)", n_group, topk_group);
    QuantArgs qa = {};
    if(x_bf16)
    {
        rc = pyhip_make_quant_args("moe_route_sorting", x_bf16, row_stride_elems, rows, K, q, scales, nullptr, &qa);
        if(rc)
            return rc;
    }
    RouteArgs ra  = {};
    const int ne  = experts / 64;
    const bool fused = tokens > 0 && tokens <= ROUTE_SORT_MAX_TOKENS && (int64_t)tokens * topk <= SMALL_PAIRS_MAX &&
                       experts <= ROUTE_SORT_MAX_EXPERTS && (ne & (ne - 1)) == 0;
    if(fused)
    {
        ra.gating = gating; ra.topk_w = topk_weight; ra.topk_ids = topk_ids;
        ra.n_group = n_group; ra.topk_group = topk_group; ra.renorm = renormalize;
    }
    else
    {
        rc = n_group > 0 ? pyhip_moe_topk_grouped_sigmoid(gating, tokens, experts, topk, n_group, topk_group, renormalize,
                                                          topk_weight, topk_ids, stream)
                         : pyhip_moe_topk_softmax(gating, tokens, experts, topk, renormalize, topk_weight, topk_ids, stream);
        if(rc)
            return rc;
    }
    return sorting_impl(topk_ids, topk_weight, tokens, topk, experts, block_size, expert_mask, num_local_tokens,
                        sorted_ids, sorted_weights, sorted_expert_ids, num_valid_ids, schedule, nullptr, 0, workspace,
                        workspace_bytes, qa, ra, stream);
}
