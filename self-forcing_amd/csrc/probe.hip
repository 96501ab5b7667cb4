// Measurement aid: what the matrix pipes of this device sustain on a stream of independent bf16 MFMAs.
// bench.py reports the dense kernel against this figure next to the nominal peak.

#include <hip/hip_runtime.h>

#include "sfm_attn.h"
#include "sfm_common.hpp"

// External linkage, so that the store in the kernel (and with it the MFMA chain) cannot be dropped as unobservable.
__device__ float sfm_probe_sink[1];

namespace sfm {
namespace {

__global__ __launch_bounds__(256) void mfma_probe_kernel(int iters) {
    f32x16 acc[4];
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[a][v] = 0.f;
    // operands: pseudo-random bf16 values of either sign with magnitudes in [0.125, 2), one set per chain (what the
    // pipes sustain depends on the data: all-small operands toggle few bits and clock higher)
    auto rnd16 = [](uint32_t h) {
        h *= 2654435761u;
        h ^= h >> 15;
        h *= 2246822519u;
        h ^= h >> 13;
        return (uint32_t)(((h & 1u) << 15) | ((0x7cu + ((h >> 1) & 3u)) << 7) | ((h >> 3) & 0x7fu));
    };
    auto rnd32 = [&](uint32_t h) { return rnd16(2 * h) | (rnd16(2 * h + 1) << 16); };
    u32x4 x[4], y;
#pragma unroll
    for (int a = 0; a < 4; ++a) {
        const uint32_t h = (threadIdx.x * 4 + a) * 4;
        x[a] = u32x4{rnd32(h), rnd32(h + 1), rnd32(h + 2), rnd32(h + 3)};
    }
    y = u32x4{rnd32(77777 + threadIdx.x * 4), rnd32(77778 + threadIdx.x * 4), rnd32(77779 + threadIdx.x * 4), rnd32(77780 + threadIdx.x * 4)};
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int r = 0; r < 4; ++r)
#pragma unroll
            for (int a = 0; a < 4; ++a) acc[a] = BF16::mfma32(x[a], y, acc[a]);
    }
    float s = 0.f;
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
        for (int v = 0; v < 16; ++v) s += acc[a][v];
    if (s == 12345.678f) sfm_probe_sink[0] = s;                 // keeps the accumulators alive; never true in practice
}

// Memory traffic of the Monarch forward's step 1 with nothing else: `tiles` work items in gridDim.x equal contiguous
// shares; item t reads 2 x rows_in rows of 16 x chunks bytes (contiguous, at t) and writes rows_out rows to each of two
// matrices, row r of item t at row index r * tiles + t (the scatter of the (a, j)-major scratch).
template <bool NT>
__global__ __launch_bounds__(320) void tile_traffic_kernel(const u32x4* in, u32x4* o0, u32x4* o1, int tiles, int rows_in, int rows_out, int chunks) {
    const int tid = threadIdx.x;
    const int t0 = (int)((int64_t)blockIdx.x * tiles / gridDim.x), t1 = (int)((int64_t)(blockIdx.x + 1) * tiles / gridDim.x);
    const int nin = 2 * rows_in * chunks, nout = rows_out * chunks;
    for (int t = t0; t < t1; ++t) {
        u32x4 acc = {0u, 0u, 0u, 0u};
        const u32x4* src = in + (size_t)t * nin;
        for (int c = tid; c < nin; c += 320) {
            const u32x4 v = src[c];
            acc.x ^= v.x; acc.y ^= v.y; acc.z ^= v.z; acc.w ^= v.w;
        }
        for (int c = tid; c < nout; c += 320) {
            const size_t at = ((size_t)(c / chunks) * tiles + t) * chunks + c % chunks;
            if (NT) {
                __builtin_nontemporal_store(acc, o0 + at);
                __builtin_nontemporal_store(acc, o1 + at);
            } else {
                o0[at] = acc;
                o1[at] = acc;
            }
        }
    }
}

// Memory traffic of the Monarch forward's step 2 with nothing else: wave w reads two blocks of `kb_per_block` KB (its
// Kbar rows and its Y rows), 16 bytes per lane and 8 KB of each block per batch, the next batch requested as soon as
// the current one has been consumed.
__global__ __launch_bounds__(256) void row_stream_kernel(const u32x4* in, int nwaves, int kb_per_block) {
    const int w = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
    if (w >= nwaves) return;
    const size_t block = (size_t)kb_per_block * 64;                      // 16-byte pieces per block
    const u32x4* k = in + (size_t)w * block;
    const u32x4* y = in + ((size_t)nwaves + w) * block;
    const int last = kb_per_block * 64 - 1;
    u32x4 buf[16];
    u32x4 acc = {0u, 0u, 0u, 0u};
    auto load = [&](int batch) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int idx = min(batch * 512 + i * 64 + lane, last);
            buf[i] = k[idx];
            buf[8 + i] = y[idx];
        }
    };
    const int nb = (kb_per_block + 7) / 8;
    load(0);
    for (int b = 0; b < nb; ++b) {
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            acc.x ^= buf[i].x; acc.y += buf[i].y; acc.z ^= buf[i].z; acc.w += buf[i].w;
        }
        load(min(b + 1, nb - 1));
    }
    if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x9e3779b9u) sfm_probe_sink[0] = (float)acc.x;    // keeps the loads alive
}

}  // namespace
}  // namespace sfm

extern "C" int sfm_probe_mfma_bf16(int32_t iters, void* stream, float* tflops) {
    using namespace sfm;
    if (iters < 1 || iters > (1 << 20) || tflops == nullptr) {
        set_error("sfm_probe_mfma_bf16: iters must be in [1, 2^20] and tflops non-null");
        return SFM_ERR_RANGE;
    }
    hipStream_t st = (hipStream_t)stream;
    const int wgs = 2 * cu_count();                          // two waves per SIMD
    hipEvent_t e0, e1;
    if (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess) {
        set_error("sfm_probe_mfma_bf16: hipEventCreate failed");
        return SFM_ERR_HIP;
    }
    hipLaunchKernelGGL(mfma_probe_kernel, dim3(wgs), dim3(256), 0, st, iters);          // warm-up
    (void)hipEventRecord(e0, st);
    hipLaunchKernelGGL(mfma_probe_kernel, dim3(wgs), dim3(256), 0, st, iters);
    (void)hipEventRecord(e1, st);
    hipError_t e = hipEventSynchronize(e1);
    float ms = 0.f;
    if (e == hipSuccess) e = hipEventElapsedTime(&ms, e0, e1);
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    if (e != hipSuccess || ms <= 0.f) {
        set_error("sfm_probe_mfma_bf16: %s", hipGetErrorString(e));
        return SFM_ERR_HIP;
    }
    const double flops = (double)wgs * 4 * (double)iters * 16 * (2.0 * 32 * 32 * 16);
    *tflops = (float)(flops / (ms * 1e-3) / 1e12);
    return SFM_OK;
}

extern "C" int sfm_probe_tile_traffic(int32_t tiles, int32_t rows_in, int32_t rows_out, int32_t row_bytes, int32_t nontemporal,
                                      void* workspace, size_t workspace_bytes, void* stream, float* us) {
    using namespace sfm;
    if (tiles < 1 || rows_in < 1 || rows_out < 1 || row_bytes < 16 || row_bytes % 16 || workspace == nullptr || us == nullptr) {
        set_error("sfm_probe_tile_traffic: tiles, rows_in, rows_out >= 1, row_bytes a multiple of 16, workspace and us non-null");
        return SFM_ERR_RANGE;
    }
    const size_t in_bytes = (size_t)tiles * 2 * rows_in * row_bytes, out_bytes = (size_t)tiles * rows_out * row_bytes;
    if (in_bytes + 2 * out_bytes > workspace_bytes || ((uintptr_t)workspace & 15)) {
        set_error("sfm_probe_tile_traffic: workspace of %zu bytes, 16-byte aligned, needed", in_bytes + 2 * out_bytes);
        return SFM_ERR_WORKSPACE;
    }
    hipStream_t st = (hipStream_t)stream;
    hipEvent_t e0, e1;
    if (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess) {
        set_error("sfm_probe_tile_traffic: hipEventCreate failed");
        return SFM_ERR_HIP;
    }
    u32x4* o0 = (u32x4*)((char*)workspace + in_bytes);
    u32x4* o1 = (u32x4*)((char*)workspace + in_bytes + out_bytes);
    // Consecutive passes read different copies of the input (as many as the workspace holds, at most 8): with a single
    // copy smaller than the memory-side cache the reads of every pass after the first are served from that cache and the
    // pass measures the writes only.
    int copies = (int)((workspace_bytes - 2 * out_bytes) / in_bytes);
    if (copies > 8) copies = 8;
    const int wgs = tiles < 2 * cu_count() ? tiles : 2 * cu_count();
    const int reps = 8;
    auto launch = [&](int i) {
        const int cp = i % copies;                           // copy 0 at the start, the others behind the two outputs
        const u32x4* in = (const u32x4*)((char*)workspace + (cp ? 2 * out_bytes + (size_t)cp * in_bytes : 0));
        if (nontemporal) hipLaunchKernelGGL(tile_traffic_kernel<true>, dim3(wgs), dim3(320), 0, st, in, o0, o1, tiles, rows_in, rows_out, row_bytes / 16);
        else hipLaunchKernelGGL(tile_traffic_kernel<false>, dim3(wgs), dim3(320), 0, st, in, o0, o1, tiles, rows_in, rows_out, row_bytes / 16);
    };
    launch(0);                                               // warm-up
    (void)hipEventRecord(e0, st);
    for (int i = 0; i < reps; ++i) launch(i + 1);
    (void)hipEventRecord(e1, st);
    hipError_t e = hipEventSynchronize(e1);
    float ms = 0.f;
    if (e == hipSuccess) e = hipEventElapsedTime(&ms, e0, e1);
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    if (e != hipSuccess || ms <= 0.f) {
        set_error("sfm_probe_tile_traffic: %s", hipGetErrorString(e));
        return SFM_ERR_HIP;
    }
    *us = ms * 1e3f / reps;
    return SFM_OK;
}

extern "C" int sfm_probe_row_stream(int32_t waves, int32_t kb_per_block, const void* workspace, size_t workspace_bytes, void* stream,
                                    float* us) {
    using namespace sfm;
    if (waves < 1 || kb_per_block < 1 || workspace == nullptr || us == nullptr) {
        set_error("sfm_probe_row_stream: waves, kb_per_block >= 1, workspace and us non-null");
        return SFM_ERR_RANGE;
    }
    const size_t need = (size_t)2 * waves * kb_per_block * 1024;
    if (need > workspace_bytes || ((uintptr_t)workspace & 15)) {
        set_error("sfm_probe_row_stream: workspace of %zu bytes, 16-byte aligned, needed", need);
        return SFM_ERR_WORKSPACE;
    }
    hipStream_t st = (hipStream_t)stream;
    hipEvent_t e0, e1;
    if (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess) {
        set_error("sfm_probe_row_stream: hipEventCreate failed");
        return SFM_ERR_HIP;
    }
    const int wgs = (waves + 3) / 4, reps = 5;
    auto launch = [&] { hipLaunchKernelGGL(row_stream_kernel, dim3(wgs), dim3(256), 0, st, (const u32x4*)workspace, waves, kb_per_block); };
    launch();                                                // warm-up
    (void)hipEventRecord(e0, st);
    for (int i = 0; i < reps; ++i) launch();
    (void)hipEventRecord(e1, st);
    hipError_t e = hipEventSynchronize(e1);
    float ms = 0.f;
    if (e == hipSuccess) e = hipEventElapsedTime(&ms, e0, e1);
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    if (e != hipSuccess || ms <= 0.f) {
        set_error("sfm_probe_row_stream: %s", hipGetErrorString(e));
        return SFM_ERR_HIP;
    }
    *us = ms * 1e3f / reps;
    return SFM_OK;
}


// ------------------------------------------------------------------------------------------------
// L2 -> compute unit read rate: every workgroup streams `stages` stages of 32 KB (64-byte pieces of 512 rows that are
// 4 KB apart, the next piece of every row per stage) of one 2 MB window that all workgroups share, i.e. that stays in
// every XCD's L2, straight into LDS (global_load_lds_dwordx4, three stages in flight).  What a tile-streaming kernel
// (one-kernel Monarch forward, block GEMM) can be fed at most when its tiles come from L2.
// ------------------------------------------------------------------------------------------------
namespace sfm {
namespace {
__device__ __forceinline__ void pr_load_lds16(const char* base, uint32_t off, uint32_t lds_addr) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_addr), "v"(off), "s"(base) : "memory", "m0");
}
__global__ __launch_bounds__(256) void l2_read_kernel(const char* src, int stages, float* sink) {
    extern __shared__ __attribute__((aligned(256))) char lds_pr[];
    const uint32_t lds0 = (uint32_t)(size_t)(__attribute__((address_space(3))) char*)lds_pr;
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    uint32_t off[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) off[j] = (uint32_t)((4 * j + wave) * 16 + (lane >> 2)) * 4096 + (lane & 3) * 16;
    const char* base = src;
    for (int s = 0; s < stages; ++s) {
        const uint32_t mb = lds0 + (uint32_t)(s & 3) * 32768 + wave * 1024;
#pragma unroll
        for (int j = 0; j < 8; ++j) pr_load_lds16(base, off[j], mb + j * 4096);
        base += 64;
        if (s >= 3) asm volatile("s_waitcnt vmcnt(24)" ::: "memory");
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    const u32x4 v = *(const u32x4*)(lds_pr + tid * 16);
    if (v.x == 0x12345678u && v.y == 0x9abcdef0u) sink[0] = 1.f;        // keeps the loads; practically never true
}
}  // namespace
}  // namespace sfm

extern "C" int sfm_probe_l2_read(int32_t workgroups, int32_t stages, void* workspace, size_t workspace_bytes, void* stream, float* us) {
    using namespace sfm;
    if (workgroups < 1 || stages < 4 || stages > 64 || workspace == nullptr || us == nullptr) {
        set_error("sfm_probe_l2_read: workgroups >= 1, 4 <= stages <= 64, workspace and us non-null");
        return SFM_ERR_RANGE;
    }
    const size_t need = (size_t)512 * 4096 + 256;
    if (need > workspace_bytes || ((uintptr_t)workspace & 255)) {
        set_error("sfm_probe_l2_read: workspace of %zu bytes, 256-byte aligned, needed", need);
        return SFM_ERR_WORKSPACE;
    }
    hipStream_t st = (hipStream_t)stream;
    if (hipFuncSetAttribute((const void*)l2_read_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 131072) != hipSuccess) {
        set_error("sfm_probe_l2_read: hipFuncSetAttribute failed");
        return SFM_ERR_HIP;
    }
    hipEvent_t e0, e1;
    if (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess) {
        set_error("sfm_probe_l2_read: hipEventCreate failed");
        return SFM_ERR_HIP;
    }
    const int reps = 10;
    float* sink = (float*)((char*)workspace + (size_t)512 * 4096);
    auto launch = [&] { hipLaunchKernelGGL(l2_read_kernel, dim3(workgroups), dim3(256), 131072, st, (const char*)workspace, stages, sink); };
    launch();                                                // warm-up: the window is in L2 afterwards
    (void)hipEventRecord(e0, st);
    for (int i = 0; i < reps; ++i) launch();
    (void)hipEventRecord(e1, st);
    hipError_t e = hipEventSynchronize(e1);
    float ms = 0.f;
    if (e == hipSuccess) e = hipEventElapsedTime(&ms, e0, e1);
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    if (e != hipSuccess || ms <= 0.f) {
        set_error("sfm_probe_l2_read: %s", hipGetErrorString(e));
        return SFM_ERR_HIP;
    }
    *us = ms * 1e3f / reps;
    return SFM_OK;
}
