// Measurement probe, not part of the layer: the inner loop of the 288-row MXFP4 GEMM reduced to its instruction and
// memory pattern, to measure on the machine at hand what that pattern can sustain.  One workgroup of four waves per CU,
// one wave per SIMD; an iteration is a K-group of the 288-row tile: 72 row groups of four
// v_mfma_scale_f32_16x16x128_f8f6f4 (288 MFMAs per wave), one ds_read_b128 operand read per row group, and, by
// variant, the 16 weight-tile loads (1 KB each, streamed from HBM through a buffer far larger than the caches, issued
// where the GEMM issues them and waited for one iteration later, as in the GEMM) and 29 LDS-DMA operations (from a
// cache-resident region, into LDS nobody reads).  No tiles, no epilogue, no barriers: what is left is the matrix pipeline
// against the memory stream.  bench.py --frontier times the variants and reports MFMA duty and TB/s for each.
//
//   variant 0  MFMAs only
//           1  + LDS operand reads
//           2  + the weight stream (16 KB per wave and iteration: the DeepSeek-V3 gate_up ratio of bytes per MFMA)
//           3  + the LDS-DMA operations
//           4  as 2, every second MFMA replaced by four VALU moves (the same issue time, half the matrix work)
//           5  as 2, every MFMA replaced: the load stream alone at the MFMA loop's pace
//           6  as 3, the weight tiles from a region that stays in the L2 (the compute-bound case: few experts, many rows)
//   and the same for the 128-row tile's pattern (two workgroups per CU, 128 MFMAs, 32 operand reads, 16 weight tiles
//   and 10 LDS-DMA operations per wave and K-group):
//           7  MFMAs + LDS operand reads          8  + LDS-DMA + weight tiles from the L2          9  + ... streamed from HBM
#include "gemm_device.h"

#define PROBE_LDS_BYTES(RG) ((RG) == 18 ? 96 * 1024 : 64 * 1024)     // one workgroup per CU, or two
#define PROBE_STREAM_MASK 0x3FFFFFFF            // the stream wraps inside the first GiB of the buffer
#define PROBE_MIN_BYTES ((1ll << 30) + (16ll << 20))

// V: what takes part (0..5 above); RG: row groups per K-step (18: the 288-row tile, 8: the 128-row tile); CACHED: the weight
// tiles come from 16 KB per wave that are read again and again (L2 hits) instead of a stream through the first GiB
template <int V, int RG, bool CACHED>
__global__ void __launch_bounds__(GEMM_THREADS, (RG == 18 ? 1 : 2)) probe_mfma_stream_kernel(int iters, const uint8_t* buf, int* sink)
{
#if defined(__HIP_DEVICE_COMPILE__)
    asm volatile("" ::: "a0", "a63");               // the 16 accumulator tiles the MFMAs below name
    __shared__ __attribute__((aligned(16))) uint8_t lds[PROBE_LDS_BYTES(RG)];
    const int tid = threadIdx.x, lane = tid % WAVE;
    const int wave = __builtin_amdgcn_readfirstlane(tid / WAVE);
    for(int i = tid; i < PROBE_LDS_BYTES(RG) / 4; i += GEMM_THREADS)
        ((u32*)lds)[i] = (u32)i * 2654435761u;
    __syncthreads();
    constexpr bool LDS_READS = V >= 1, STREAM = V >= 2, DMA = V == 3;
    static_assert(!CACHED || V == 3, "the cached source exists for the full pattern only");
    constexpr int MFMA_EVERY = V == 4 ? 2 : V == 5 ? 0 : 1;     // 1: every slot an MFMA; 2: every second; 0: none
    // stream: wave w of workgroup b reads 4 KB pieces at piece index (4 b + w) of consecutive 8 MiB chunks; the chunk
    // offset goes into the scalar offset (not range-checked: the mask keeps it inside the first GiB)
    const v4i rs      = make_rsrc(buf, 0x7FFFFFF0u);
    const int gw      = (int)((blockIdx.x * 4 + wave) & 2047);
    const int v_strm  = lane * 16 + gw * (CACHED ? 16384 : 4096);
    constexpr int NDMA = RG == 18 ? 29 : 10, DMA_RGS = RG == 18 ? 2 * RG : RG;   // LDS-DMA operations and the row groups they are spread over
    constexpr int WSTEP = RG / 4;                               // row groups between two weight tiles of a K-step
    const int v_dma   = lane * 16 + gw * 4096;                  // 4 KB per wave, read again every iteration: cache hits
    const u32 lds_dma = (u32)__builtin_amdgcn_readfirstlane((int)lds_addr_of(lds + 32768 + wave * 4096));
    const uint8_t* rd = lds + lane * 16;
    int sx            = 0;                                      // chunk offset of the stream
    v4i wf[16];
    v4i af[3];
    int t0 = lane, t1 = lane + 1, t2 = lane + 2, t3 = lane + 3;
#pragma unroll
    for(int i = 0; i < 16; i++)
    {
        const u32 h = (u32)(tid * 16 + i + 1) * 2654435761u;          // noise, as real e2m1 weights are
        wf[i]       = (v4i){(int)h, (int)(h * 3u), (int)(h * 5u), (int)(h * 7u)};
    }
    af[0] = af[1] = af[2] = wf[0];
    const int sc = 0x7f7f7f7f;                                  // scale bytes 127: 2^0
    gemm_zero_acc<4>();
    auto slot = [&](auto NN, auto JJ) __attribute__((always_inline)) {
        constexpr int n = decltype(NN)::value, j = decltype(JJ)::value, u = n / RG;
        constexpr int k = n * 4 + j;
        if constexpr(MFMA_EVERY == 1 || (MFMA_EVERY == 2 && k % 2 == 0))
            mfma_one<u, n % 4, 4, j>(wf[u * 4 + j], LDS_READS ? af[n % 3] : wf[0], sc, sc);
        else
        {
            int &x0 = t0, &x1 = t1, &x2 = t2, &x3 = t3;
            asm volatile("v_mov_b32 %0, %1\n\tv_mov_b32 %1, %2\n\tv_mov_b32 %2, %3\n\tv_mov_b32 %3, %0"
                         : "+v"(x0), "+v"(x1), "+v"(x2), "+v"(x3));
        }
    };
    auto stream_load = [&](auto II) __attribute__((always_inline)) {
        constexpr int i = decltype(II)::value;
        vm_load_b128<(i % 4) * 1024, false>(wf[i], v_strm, rs, sx);
        if constexpr(i % 4 == 3)
            sx = CACHED ? (sx + 4096) & 0x3FFF : (sx + 0x800000) & PROBE_STREAM_MASK;
    };
    if constexpr(LDS_READS)
    {
        af[0] = *(const v4i*)(rd);
        af[1] = *(const v4i*)(rd + 1024);
    }
    for(int it = 0; it < iters; it++)
    {
        static_for<4 * RG>([&](auto NN) __attribute__((always_inline)) {
            constexpr int n = decltype(NN)::value;
            __builtin_amdgcn_sched_barrier(0);
            static_for<4>([&](auto JJ) __attribute__((always_inline)) {
                constexpr int j = decltype(JJ)::value;
                slot(NN, JJ);
                __builtin_amdgcn_sched_barrier(0);
                if constexpr(LDS_READS && j == 0)
                    af[(n + 2) % 3] = *(const v4i*)(rd + ((n + 2) % 16) * 1024);
                // the LDS-DMA operations over the first two K-steps (288-row tile) or the first (128-row tile), as the GEMM
                // spreads them
                if constexpr(DMA && j >= 1 && n < DMA_RGS)
                {
                    constexpr int s = n * 3 + j - 1, NS = DMA_RGS * 3;  // slot 0 .. NS-1
                    if constexpr((s * NDMA) / NS != ((s + 1) * NDMA) / NS)
                        vm_dma_b128<((s * NDMA / NS) % 4) * 1024, 0>(v_dma, rs, 0, lds_dma);
                }
                // the weight tiles of K-step u go out during K-step u + 1 (u = 3: after the last row group)
                constexpr int m  = n >= RG ? n - RG : 0;               // row groups since the start of K-step 1
                constexpr int ti = (m / RG) * 4 + (m % RG) / WSTEP % 4;   // tile u * 4 + j goes out at row group RG (u + 1) + WSTEP j
                if constexpr(STREAM && j == 3 && n >= RG && m % RG % WSTEP == 0 && m % RG / WSTEP < 4)
                    stream_load(std::integral_constant<int, ti>{});
                __builtin_amdgcn_sched_barrier(0);
            });
        });
        if constexpr(STREAM)
        {
            static_for<4>([&](auto JJ) __attribute__((always_inline)) { stream_load(std::integral_constant<int, 12 + decltype(JJ)::value>{}); });
            // everything but this iteration's youngest 12 weight tiles has landed (the DMA operations, the tiles of
            // K-step 0, and all of the previous iteration's): the GEMM's wait at the end of a K-group
            if constexpr(RG == 18)
                asm volatile("s_waitcnt vmcnt(12)" ::: "memory");
            else
                asm volatile("s_waitcnt vmcnt(16)" ::: "memory");   // (128-row tile: all its weight tiles follow the LDS-DMA)
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_nop 15\n\ts_nop 15" ::: "memory");
    int r = (int)acc_fixed_read<0>() + t0 + t1 + t2 + t3;
#pragma unroll
    for(int i = 0; i < 16; i++)
        r += wf[i].x;
    if(r == 0x12345678)
        sink[blockIdx.x * GEMM_THREADS + tid] = r;
#endif
}

// Enqueues `launches` launches of variant `variant` with one workgroup per CU, `iters` iterations (K-groups) each.
// buf: device buffer of at least PROBE_MIN_BYTES bytes (read only), sink: at least 4 bytes (never written in practice).
// -> PYHIP_OK; *workgroups receives the number of workgroups per launch.  The caller times the launches.
extern "C" int pyhip_moe_probe_mfma_stream(int variant, int iters, const void* buf, int64_t buf_bytes, int32_t* sink,
                                       int launches, int* workgroups, hipStream_t stream)
{
    PYHIP_REQUIRE(variant >= 0 && variant <= 9, "probe_mfma_stream: variant=%d not in 0..9", variant);
    PYHIP_REQUIRE(iters > 0 && launches > 0, "probe_mfma_stream: bad counts");
    PYHIP_REQUIRE(buf && sink && buf_bytes >= PROBE_MIN_BYTES && ((uintptr_t)buf % 16) == 0,
                  "probe_mfma_stream: needs an aligned buffer of at least %lld bytes", (long long)PROBE_MIN_BYTES);
    const int cus = device_cu_count();
    const int wgs = variant >= 7 ? 2 * cus : cus;
    if(workgroups)
        *workgroups = wgs;
#define PROBE_LAUNCH(V, RG, C) \
    hipLaunchKernelGGL((probe_mfma_stream_kernel<V, RG, C>), dim3(wgs), dim3(GEMM_THREADS), 0, stream, iters, (const uint8_t*)buf, sink)
    for(int l = 0; l < launches; l++)
    {
        switch(variant)
        {
        case 0: PROBE_LAUNCH(0, 18, false); break;
        case 1: PROBE_LAUNCH(1, 18, false); break;
        case 2: PROBE_LAUNCH(2, 18, false); break;
        case 3: PROBE_LAUNCH(3, 18, false); break;
        case 4: PROBE_LAUNCH(4, 18, false); break;
        case 5: PROBE_LAUNCH(5, 18, false); break;
        case 6: PROBE_LAUNCH(3, 18, true); break;
        case 7: PROBE_LAUNCH(1, 8, false); break;
        case 8: PROBE_LAUNCH(3, 8, true); break;
        default: PROBE_LAUNCH(3, 8, false); break;
        }
    }
#undef PROBE_LAUNCH
    PYHIP_CHECK_LAUNCH("probe_mfma_stream_kernel");
    return PYHIP_OK;
}
