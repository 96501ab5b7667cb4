// Monarch attention backward: the chain of its parts.  Each part runs as a fused MFMA kernel where the problem
// allows (monarch_bwd_left.hip, monarch_bwd_right.hip, step 1 of monarch_mfma.hip; make_parts() decides) and
// otherwise as batched library GEMMs plus small element-wise kernels, which is what this file holds.
//
// Every contraction of the backward (and of the forward it recomputes) is a plain matrix product once q, k, v
// are gathered into block-row-major copies: per (unit, block row k) the logits are [a*b2 x D] . [D x f*b2],
// per (unit, a, j) the left factor is [b1 x D] . [D x f*b1], and so on (13 products, listed in run()).
// They go to rocBLAS' strided batched GEMM (bf16 / fp16 / fp32 operands, fp32 accumulation); the scratch
// layouts are chosen so that every batch has one stride: intermediates of the right factor are kept per
// (unit, k, f) block, [a*b2 x D] or [a*b2 x b2] each, and the left factor orders its rows (k, f).  The
// softmaxes, the entropy term and their backward are row kernels in between.  Replaces _z_bwd_preprocess,
// _z_bwd, _al_cl_y_bwd and their orchestration (wan/modules/monarch_attn.py:852-886, 1034-1222, 403-596,
// 1326-1470, 1566-1693).  rocBLAS is resolved with dlopen on first use, so the library itself does not
// depend on it; without it the chain still runs where every part is fused, and the fp32 SIMT kernels of
// monarch_generic.hip otherwise.
//
// Formulas (s = sm_scale, per unit): S1 = s q.k, R = softmax_l S1, Kbar = R K, Y = R V, c = sum_l R ln R,
// S2 = s q.Kbar - c, L = softmax_(f,k) S2, O = L Y;
//   dLm = dO.Y   dS2 = L (dLm - sum L dLm)   dY = L^T dO   dKbar = s dS2^T q   dc = -sum_i dS2
//   dR = dKbar.K + dY.V + dc ln R            dS1 = R (dR - sum_l R dR)
//   dQ = s dS2 Kbar + s dS1 K                dK = R^T dKbar + s dS1^T q         dV = R^T dY

#include <cstdlib>

#include "sfm_common.hpp"

#include <dlfcn.h>
#include <mutex>
#include <rocblas/rocblas.h>

namespace sfm {

namespace {

// ---------------------------------------------------------------------------------------------
// rocBLAS, resolved at run time
// ---------------------------------------------------------------------------------------------
struct Blas {
    decltype(&rocblas_create_handle) create = nullptr;
    decltype(&rocblas_set_stream) set_stream = nullptr;
    decltype(&rocblas_gemm_strided_batched_ex) gemm = nullptr;
    bool tried = false, ok = false;
    rocblas_handle handle[16] = {};
};
Blas g_blas;
std::mutex g_blas_mutex;

bool blas_load() {
    std::lock_guard<std::mutex> lock(g_blas_mutex);
    if (g_blas.tried) return g_blas.ok;
    g_blas.tried = true;
    if (rocblas_disabled()) return false;                              // for tests: behave as where the library is absent
    void* lib = dlopen("librocblas.so.5", RTLD_NOW | RTLD_GLOBAL);
    if (!lib) lib = dlopen("/opt/rocm/lib/librocblas.so.5", RTLD_NOW | RTLD_GLOBAL);
    if (!lib) lib = dlopen("librocblas.so", RTLD_NOW | RTLD_GLOBAL);
    if (!lib) return false;
    g_blas.create = (decltype(g_blas.create))dlsym(lib, "rocblas_create_handle");
    g_blas.set_stream = (decltype(g_blas.set_stream))dlsym(lib, "rocblas_set_stream");
    g_blas.gemm = (decltype(g_blas.gemm))dlsym(lib, "rocblas_gemm_strided_batched_ex");
    g_blas.ok = g_blas.create && g_blas.set_stream && g_blas.gemm;
    return g_blas.ok;
}

// One handle per device, shared by the callers (rocBLAS serialises work on a handle by its stream; calls from
// several host threads on one device must not overlap).
rocblas_handle blas_handle(hipStream_t stream) {
    std::lock_guard<std::mutex> lock(g_blas_mutex);
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 16) return nullptr;
    if (!g_blas.handle[dev] && g_blas.create(&g_blas.handle[dev]) != rocblas_status_success) return nullptr;
    if (g_blas.set_stream(g_blas.handle[dev], stream) != rocblas_status_success) return nullptr;
    return g_blas.handle[dev];
}

// ---------------------------------------------------------------------------------------------
// element access
// ---------------------------------------------------------------------------------------------
template <typename E> struct El;
template <> struct El<float> {
    typedef float type;
    static constexpr rocblas_datatype kBlas = rocblas_datatype_f32_r;
    static __device__ __forceinline__ float get(const float* p, int64_t i) { return p[i]; }
    static __device__ __forceinline__ void put(float* p, int64_t i, float x) { p[i] = x; }
};
template <> struct El<BF16> {
    typedef uint16_t type;
    static constexpr rocblas_datatype kBlas = rocblas_datatype_bf16_r;
    static __device__ __forceinline__ float get(const uint16_t* p, int64_t i) { return BF16::to_float(p[i]); }
    static __device__ __forceinline__ void put(uint16_t* p, int64_t i, float x) { p[i] = BF16::from_float(x); }
};
template <> struct El<F16> {
    typedef uint16_t type;
    static constexpr rocblas_datatype kBlas = rocblas_datatype_f16_r;
    static __device__ __forceinline__ float get(const uint16_t* p, int64_t i) { return F16::to_float(p[i]); }
    static __device__ __forceinline__ void put(uint16_t* p, int64_t i, float x) { p[i] = F16::from_float(x); }
};

// ---------------------------------------------------------------------------------------------
// kernels.  Index names: u unit of the pass, k / i block row, a, f block-frames, j, l block columns,
// aj = a*b2 + j, AJ = na*b2, t = (u*b1 + k)*nf + f, r = k*nf + f (row of the left factor), RR = nf*b1.
// ---------------------------------------------------------------------------------------------
// Copies token-ordered rows into [u][i][bf][j][D] (col_major = 0) or [u][bf][j][i][D] (col_major = 1), in 8-byte
// pieces: the row of block coordinates (bf, i, j) is token map.row(bf, i) + j of unit unit0 + u.
template <typename E>
__global__ __launch_bounds__(256) void gather_rows(typename El<E>::type* dst, const void* src, int64_t s0, int64_t s1, int64_t s2,
                                                   TokMap map, int nbf, int H, int D, int unit0, int col_major, int64_t total) {
    const int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    constexpr int kPer = 8 / sizeof(typename El<E>::type);
    const int pieces = D / kPer;
    if (e >= total) return;
    const int pc = (int)(e % pieces);
    int64_t row = e / pieces;
    int i, j, bf;
    if (col_major) {
        i = (int)(row % map.b1);
        row /= map.b1;
        j = (int)(row % map.b2);
        row /= map.b2;
        bf = (int)(row % nbf);
        row /= nbf;
    } else {
        j = (int)(row % map.b2);
        row /= map.b2;
        bf = (int)(row % nbf);
        row /= nbf;
        i = (int)(row % map.b1);
        row /= map.b1;
    }
    const int unit = unit0 + (int)row;
    const int b = unit / H, h = unit % H;
    const int64_t tok = map.row(bf, i) + j;
    const typename El<E>::type* sp = (const typename El<E>::type*)src + b * s0 + tok * s1 + h * s2 + pc * kPer;
    *(uint64_t*)(dst + (e / pieces) * D + pc * kPer) = *(const uint64_t*)sp;
}

// Right factor: one wave per segment (u, k, aj, f) of b2 logits S1[(u,k)][aj][f][:], lane l holding logits
// l, l + 64, ... (one per lane when b2 <= 64).
// Rb[t][aj][:] = softmax(s * S1) rounded to the operand type; c[(u, aj)][r] = sum_l R ln R.
constexpr int kSegPerLane = 4;          // b2 <= 256

__device__ __forceinline__ float wave_max(float v) {
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o));
    return v;
}
__device__ __forceinline__ float wave_sum(float v) {
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
    return v;
}

template <typename E>
__global__ __launch_bounds__(256) void softmax_right(const float* S1, typename El<E>::type* Rb, float* c, int b1, int AJ, int nf, int b2,
                                                     float scale, int64_t nseg) {
    const int64_t seg = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (seg >= nseg) return;
    const int lane = threadIdx.x & 63;
    const int f = (int)(seg % nf);
    const int64_t row = seg / nf;                       // uk * AJ + aj
    const int aj = (int)(row % AJ);
    const int64_t uk = row / AJ;
    const int k = (int)(uk % b1);
    const int64_t u = uk / b1;
    const int64_t blk = (uk * nf + f) * AJ + aj;
    const float* z = S1 + seg * b2;
    float v[kSegPerLane];
    float mx = -INFINITY;
#pragma unroll
    for (int q = 0; q < kSegPerLane; ++q) {
        const int l = lane + 64 * q;
        v[q] = l < b2 ? z[l] * scale : -INFINITY;
        mx = fmaxf(mx, v[q]);
    }
    mx = wave_max(mx);
    float sum = 0.f;
#pragma unroll
    for (int q = 0; q < kSegPerLane; ++q) sum += __expf(v[q] - mx);
    sum = wave_sum(sum);
    const float lse = mx + __logf(sum);
    float ent = 0.f;
#pragma unroll
    for (int q = 0; q < kSegPerLane; ++q) {
        const int l = lane + 64 * q;
        if (l < b2) {
            const float lr = v[q] - lse;
            const float r = __expf(lr);
            El<E>::put(Rb, blk * b2 + l, r);
            ent += r * lr;
        }
    }
    ent = wave_sum(ent);
    if (lane == 0) c[(u * AJ + aj) * ((int64_t)nf * b1) + (int64_t)k * nf + f] = ent;
}

// Left factor: one workgroup per row (u, aj, i) of RR logits S2[(u,aj)][i][r], thread t holding logits
// t, t + 256, ... (RR <= 256 * kLeftPerThread).
// L = softmax(s * S2 - c) (masked block-frames give 0), dS2 = L (dLm - sum L dLm); both in the operand type.
constexpr int kLeftPerThread = 8;

template <typename E>
__global__ __launch_bounds__(256) void softmax_left(const float* S2, const float* dLm, const float* c, typename El<E>::type* L,
                                                    typename El<E>::type* dS2, int b1, int b2, int AJ, int nf, int causal, float scale) {
    __shared__ float red[8];
    const int RR = nf * b1;
    const int64_t row = blockIdx.x;                     // (u * AJ + aj) * b1 + i
    const int64_t uaj = row / b1;
    const int aj = (int)(uaj % AJ);
    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    const float* z = S2 + row * RR;
    const float* g = dLm + row * RR;
    const float* cc = c + uaj * RR;
    const int flim = causal ? min(nf, ((aj / b2) / causal + 1) * causal) : nf;      // visible kv block-frames
    auto block_max = [&](float v) {
        v = wave_max(v);
        __syncthreads();
        if (lane == 0) red[wv] = v;
        __syncthreads();
        return fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    };
    auto block_sum = [&](float v) {
        v = wave_sum(v);
        __syncthreads();
        if (lane == 0) red[wv] = v;
        __syncthreads();
        return red[0] + red[1] + red[2] + red[3];
    };
    float v[kLeftPerThread], gv[kLeftPerThread];
    float mx = -INFINITY;
#pragma unroll
    for (int q = 0; q < kLeftPerThread; ++q) {
        const int r = tid + 256 * q;
        const bool ok = r < RR && (r % nf) < flim;
        v[q] = ok ? z[r] * scale - cc[r] : -INFINITY;
        gv[q] = r < RR ? g[r] : 0.f;
        mx = fmaxf(mx, v[q]);
    }
    mx = block_max(mx);
    float sum = 0.f;
#pragma unroll
    for (int q = 0; q < kLeftPerThread; ++q) {
        v[q] = __expf(v[q] - mx);
        sum += v[q];
    }
    sum = block_sum(sum);
    const float inv = 1.f / sum;
    float dot = 0.f;
#pragma unroll
    for (int q = 0; q < kLeftPerThread; ++q) {
        v[q] *= inv;
        dot += v[q] * gv[q];
    }
    dot = block_sum(dot);
#pragma unroll
    for (int q = 0; q < kLeftPerThread; ++q) {
        const int r = tid + 256 * q;
        if (r < RR) {
            El<E>::put(L, row * RR + r, v[q]);
            El<E>::put(dS2, row * RR + r, v[q] * (gv[q] - dot));
        }
    }
}

// dc[(u, aj)][r] = - sum_i dS2[(u, aj)][i][r]
template <typename E>
__global__ __launch_bounds__(256) void reduce_dc(const typename El<E>::type* dS2, float* dc, int b1, int AJ, int RR, int64_t total) {
    const int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;      // (u * AJ + aj) * RR + r
    if (e >= total) return;
    const int64_t uaj = e / RR;
    const int r = (int)(e % RR);
    float s = 0.f;
    for (int i = 0; i < b1; ++i) s += El<E>::get(dS2, (uaj * b1 + i) * RR + r);
    dc[e] = -s;
}

// dS1[(u,k)][aj][f][:] = R (dR + dc ln R - sum_l R (dR + dc ln R)), same segments as softmax_right; R recomputed in float.
template <typename E>
__global__ __launch_bounds__(256) void softmax_right_bwd(const float* S1, const float* dRb, const float* dc, typename El<E>::type* dS1,
                                                         int b1, int AJ, int nf, int b2, float scale, int64_t nseg) {
    const int64_t seg = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (seg >= nseg) return;
    const int lane = threadIdx.x & 63;
    const int f = (int)(seg % nf);
    const int64_t row = seg / nf;
    const int aj = (int)(row % AJ);
    const int64_t uk = row / AJ;
    const int k = (int)(uk % b1);
    const int64_t u = uk / b1;
    const int64_t blk = (uk * nf + f) * AJ + aj;
    const float* z = S1 + seg * b2;
    const float* g = dRb + blk * b2;
    const float dcv = dc[(u * AJ + aj) * ((int64_t)nf * b1) + (int64_t)k * nf + f];
    float v[kSegPerLane], gv[kSegPerLane];
    float mx = -INFINITY;
#pragma unroll
    for (int q = 0; q < kSegPerLane; ++q) {
        const int l = lane + 64 * q;
        v[q] = l < b2 ? z[l] * scale : -INFINITY;
        gv[q] = l < b2 ? g[l] : 0.f;
        mx = fmaxf(mx, v[q]);
    }
    mx = wave_max(mx);
    float sum = 0.f;
#pragma unroll
    for (int q = 0; q < kSegPerLane; ++q) sum += __expf(v[q] - mx);
    sum = wave_sum(sum);
    const float lse = mx + __logf(sum);
    float dot = 0.f;
#pragma unroll
    for (int q = 0; q < kSegPerLane; ++q) {
        const int l = lane + 64 * q;
        if (l < b2) {
            const float lr = v[q] - lse;
            v[q] = __expf(lr);              // R
            gv[q] += dcv * lr;              // dR + dc ln R
            dot += v[q] * gv[q];
        }
    }
    dot = wave_sum(dot);
#pragma unroll
    for (int q = 0; q < kSegPerLane; ++q) {
        const int l = lane + 64 * q;
        if (l < b2) El<E>::put(dS1, seg * b2 + l, v[q] * (gv[q] - dot));
    }
}

// The same with R read back (16 bit, row pitch 64, rows [t][aj]) instead of recomputed from the logits.
template <typename E>
__global__ __launch_bounds__(256) void softmax_right_bwd_r(const typename El<E>::type* Rb, const float* dRb, const float* dc,
                                                           typename El<E>::type* dS1, int b1, int AJ, int nf, int b2, int64_t nseg) {
    const int64_t seg = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (seg >= nseg) return;
    const int lane = threadIdx.x & 63;
    const int f = (int)(seg % nf);
    const int64_t row = seg / nf;
    const int aj = (int)(row % AJ);
    const int64_t uk = row / AJ;
    const int k = (int)(uk % b1);
    const int64_t u = uk / b1;
    const int64_t blk = (uk * nf + f) * AJ + aj;
    const float dcv = dc[(u * AJ + aj) * ((int64_t)nf * b1) + (int64_t)k * nf + f];
    const bool in = lane < b2;                          // b2 <= 64 on this path
    const float r = in ? El<E>::get(Rb, blk * 64 + lane) : 0.f;
    float gv = in ? dRb[blk * b2 + lane] : 0.f;
    if (r > 0.f) gv += dcv * __logf(r);                 // dR + dc ln R
    const float dot = wave_sum(r * gv);
    if (in) El<E>::put(dS1, seg * b2 + lane, r * (gv - dot));
}

// dq[token row of (a, i, j)] = dQa[u][aj][i][:] (left factor) + dQk[u][i][aj][:] (right factor)
__global__ __launch_bounds__(256) void scatter_dq(const float* dQa, const float* dQk, float* dq, int64_t s0, int64_t s1, int64_t s2,
                                                  TokMap map, int na, int H, int D, int unit0, int64_t total) {
    const int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;      // float4 pieces of dQk
    const int pieces = D / 4;
    if (e >= total) return;
    const int pc = (int)(e % pieces);
    int64_t row = e / pieces;
    const int j = (int)(row % map.b2);
    row /= map.b2;
    const int a = (int)(row % na);
    row /= na;
    const int i = (int)(row % map.b1);
    const int64_t u = row / map.b1;
    const int unit = unit0 + (int)u;
    const int b = unit / H, h = unit % H;
    const int64_t tok = map.row(a, i) + j;
    const float4 x = *(const float4*)(dQk + (e / pieces) * D + pc * 4);
    const float4 y = *(const float4*)(dQa + (((u * na + a) * map.b2 + j) * map.b1 + i) * D + pc * 4);
    *(float4*)(dq + b * s0 + tok * s1 + h * s2 + pc * 4) = float4{x.x + y.x, x.y + y.y, x.z + y.z, x.w + y.w};
}

// dk / dv rows of kv block-frames [f0, f1) from the float accumulators dKk / dVk [u][k][f][l][D], 4 elements a thread
template <typename E>
__global__ __launch_bounds__(256) void scatter_dkv(const float* dKk, const float* dVk, typename El<E>::type* dk, typename El<E>::type* dv,
                                                   int64_t s0, int64_t s1, int64_t s2, TokMap map, int nf, int f0, int f1,
                                                   int64_t row0, int H, int D, int unit0, int64_t total) {
    const int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= total) return;
    const int pieces = D / 4;
    const int d = (int)(e % pieces) * 4;
    int64_t row = e / pieces;
    const int l = (int)(row % map.b2);
    row /= map.b2;
    const int ff = (int)(row % (f1 - f0));
    row /= (f1 - f0);
    const int k = (int)(row % map.b1);
    const int u = (int)(row / map.b1);
    const int f = f0 + ff;
    const int unit = unit0 + u;
    const int b = unit / H, h = unit % H;
    const int64_t src = ((((int64_t)u * map.b1 + k) * nf + f) * map.b2 + l) * D + d;
    const int64_t dst = b * s0 + (map.row(f, k) + l - row0) * s1 + h * s2 + d;
    const float4 x = *(const float4*)(dKk + src), y = *(const float4*)(dVk + src);
    El<E>::put(dk, dst, x.x); El<E>::put(dk, dst + 1, x.y); El<E>::put(dk, dst + 2, x.z); El<E>::put(dk, dst + 3, x.w);
    El<E>::put(dv, dst, y.x); El<E>::put(dv, dst + 1, y.y); El<E>::put(dv, dst + 2, y.z); El<E>::put(dv, dst + 3, y.w);
}

size_t align256(size_t x) { return (x + 255) & ~(size_t)255; }

// Scratch of a pass over n units, in bytes (all sub-buffers 256-byte aligned).
struct Layout {
    size_t Qk, Qa, dOa, Kk, Vk, S1f, dRb, Rb, dS1, Kbar, Y, dKbar, dY, c, dc, S2f, dLmf, L, dS2, dQa, dQk, dKk, dVk, total;
};

// dtype code of the fused kernels for operand type E, or -1 (fp32 operands stay on the GEMMs)
template <typename E> constexpr int left_dtype() { return -1; }
template <> constexpr int left_dtype<BF16>() { return SFM_BF16; }
template <> constexpr int left_dtype<F16>() { return SFM_F16; }

// Which parts of the chain run as fused kernels: decided by shapes, strides and (for measurements) the process-wide switches,
// so that the workspace query and the run agree.
struct Parts {
    bool left;     // 4-7: statistics and gradients of the left factor without the [i x r] matrices in memory
    bool fwd;      // 1-3: the forward's MFMA step 1 recomputes Kbar, Y, c and R straight into the scratch ([t][aj] rows)
    bool dqa;      // 8 and the scatter of dq: dQ of the left factor in its own kernel, which also adds the right factor's part
    bool right;    // 9, the right factor's softmax backward, 11-13 and the scatter of dk / dv in one kernel per tile t
    bool dqk;      // 10 in a kernel that reads K where the caller has it (with `right`: no gathered copy of K is needed)
};

Parts make_parts(const MonarchArgs& p, int dtype, const int64_t* dks) {
    Parts f;
    const unsigned sw = switches();
    const bool h16 = dtype == SFM_BF16 || dtype == SFM_F16;
    const bool q_rows_ok = (p.qs[0] | p.qs[1] | p.qs[2] | p.os[0] | p.os[1] | p.os[2]) % 8 == 0 &&       // 16-byte rows of q, dout, out
                           (int64_t)p.na * p.b1 * p.b2 * p.qs[1] * 2 < ((int64_t)1 << 32);
    f.left = h16 && q_rows_ok && monarch_bwd_left_supported(dtype, p.D, p.b1) && !(sw & SFM_SW_BWD_LEFT_GEMM);
    f.fwd = f.left && monarch_mfma_supported(dtype, p.D, p.b2) && p.b2 <= 64 && !(sw & SFM_SW_BWD_FWD_GEMM);   // R rows of 64 values
    f.dqa = f.left && !(sw & SFM_SW_BWD_DQA_GEMM);
    const bool direct_ok = (dks[0] | dks[1] | dks[2] | p.vs[0] | p.vs[1] | p.vs[2] | p.ks[0] | p.ks[1] | p.ks[2]) % 8 == 0 &&      // 16-byte rows of k, v, dk, dv
                           (int64_t)p.nf * p.b1 * p.b2 * p.ks[1] * 2 < ((int64_t)1 << 32);
    f.right = f.fwd && direct_ok && monarch_bwd_right_supported(dtype, p.D, p.b2, p.na * p.b2) &&
              !(sw & SFM_SW_BWD_RIGHT_GEMM);
    f.dqk = f.right && monarch_bwd_dqk_supported(dtype, p.D, p.b2, p.na * p.b2) && !(sw & SFM_SW_BWD_DQK_GEMM);
    return f;
}

Layout make_layout(const MonarchArgs& p, int n, size_t e, const Parts& f) {
    const size_t AJ = (size_t)p.na * p.b2, RR = (size_t)p.nf * p.b1, D = p.D;
    const size_t MQ = (size_t)p.b1 * AJ, MK = (size_t)p.b1 * p.nf * p.b2, NL = (size_t)p.nf * p.b2;
    Layout l;
    size_t o = 0;
    auto take = [&](bool used, size_t bytes) { size_t at = o; o += used ? align256(bytes) : 0; return at; };
    l.Qk = take(!f.fwd || !f.right, n * MQ * D * e);
    l.Qa = take(!f.left, n * MQ * D * e);
    l.dOa = take(!f.left, n * MQ * D * e);
    l.Kk = take(!f.dqk, n * MK * D * e);
    l.Vk = take(!f.right, n * MK * D * e);
    l.S1f = take(!f.fwd, n * p.b1 * AJ * NL * 4);
    l.dRb = take(!f.right, n * p.b1 * AJ * NL * 4);
    l.Rb = take(true, n * p.b1 * AJ * p.nf * (size_t)(p.b2 > 64 ? p.b2 : 64) * e);      // row pitch 64 when step 1 of the forward writes it
    l.dS1 = take(true, n * p.b1 * AJ * NL * e);
    l.Kbar = take(true, n * AJ * RR * D * e);
    l.Y = take(true, n * AJ * RR * D * e);
    const size_t nz = f.left ? (size_t)(p.b1 + 31) / 32 : 1;      // the fused left factor writes one partial slab per 32 query rows
    l.dKbar = take(true, nz * n * AJ * RR * D * e);
    l.dY = take(true, nz * n * AJ * RR * D * e);
    l.c = take(true, n * AJ * RR * 4);
    l.dc = take(true, nz * n * AJ * RR * 4);
    l.S2f = take(!f.left, n * AJ * p.b1 * RR * 4);
    l.dLmf = take(!f.left, n * AJ * p.b1 * RR * 4);
    l.L = take(!f.left, n * AJ * p.b1 * RR * e);
    l.dS2 = take(true, n * AJ * p.b1 * ((RR + 7) / 8 * 8) * e);                         // rows padded to 8 for the fused kernels
    l.dQa = take(!f.dqa, n * MQ * D * 4);
    l.dQk = take(true, n * MQ * D * 4);
    l.dKk = take(!f.right, n * MK * D * 4);
    l.dVk = take(!f.right, n * MK * D * 4);
    l.total = o;
    return l;
}

struct Ctx {
    rocblas_handle h;
    char* ws;
    int status;
    hipStream_t stream;
};

// one operand of a batched product: byte offset of batch 0 in the scratch, leading dimension and batch stride in elements
struct Op {
    size_t off;
    int64_t ld, stride;
};

// row-major C[M,N] = alpha op(A) op(B) + beta C for `batch` problems.
void gemm(Ctx& cx, bool ta, bool tb, int M, int N, int K, float alpha, float beta, const Op& A, const Op& B, const Op& C,
          rocblas_datatype tab, rocblas_datatype tc, int batch) {
    if (cx.status) return;
    if (!cx.h && (!blas_load() || !(cx.h = blas_handle(cx.stream)))) {
        set_error("rocBLAS is needed for this shape and could not be loaded (or its handle not created)");
        cx.status = SFM_ERR_UNSUPPORTED;
        return;
    }
    // column-major view: C^T[N,M] = op(B)^T op(A)^T
    void* c = cx.ws + C.off;
    rocblas_status st = g_blas.gemm(cx.h, tb ? rocblas_operation_transpose : rocblas_operation_none,
                                    ta ? rocblas_operation_transpose : rocblas_operation_none, N, M, K, &alpha, cx.ws + B.off, tab,
                                    (rocblas_int)B.ld, B.stride, cx.ws + A.off, tab, (rocblas_int)A.ld, A.stride, &beta, c, tc,
                                    (rocblas_int)C.ld, C.stride, c, tc, (rocblas_int)C.ld, C.stride, batch, rocblas_datatype_f32_r,
                                    rocblas_gemm_algo_standard, 0, 0);
    if (st != rocblas_status_success) {
        set_error("rocblas_gemm_strided_batched_ex failed with status %d (M=%d N=%d K=%d batch=%d)", (int)st, M, N, K, batch);
        cx.status = SFM_ERR_HIP;
    }
}

template <typename E>
int run(const MonarchBwdArgs& g, int n, void* workspace, hipStream_t stream) {
    typedef typename El<E>::type T;
    const MonarchArgs& p = g.p;
    const size_t e = sizeof(T);
    const Parts parts = make_parts(p, left_dtype<E>() >= 0 ? left_dtype<E>() : SFM_F32, g.dks);
    const Layout lay = make_layout(p, n, e, parts);
    char* ws = (char*)workspace;
    Ctx cx{nullptr, ws, 0, stream};                      // the rocBLAS handle is made by the first product that needs it
    const int b1 = p.b1, b2 = p.b2, nf = p.nf, na = p.na, D = p.D, H = p.H;
    const int AJ = na * b2, RR = nf * b1, NL = nf * b2;
    const int64_t MQ = (int64_t)b1 * AJ, MK = (int64_t)b1 * NL;
    const float s = p.scale;
    const rocblas_datatype tE = El<E>::kBlas, tF = rocblas_datatype_f32_r;

    const int64_t nseg = (int64_t)n * b1 * AJ * nf;
    const bool fused_left = parts.left, fused_fwd = parts.fwd, fused_dqa = parts.dqa, fused_right = parts.right;
    const int ds2_ld = fused_left ? (RR + 7) / 8 * 8 : RR;
    const int rb_ld = fused_fwd ? 64 : b2;
    if (fused_right && ((uintptr_t)g.dk | (uintptr_t)g.dv | (uintptr_t)p.v) % 16) {
        set_error("Monarch backward: v, dk and dv must be 16-byte aligned");
        return SFM_ERR_ALIGN;
    }
    // the forward's output and row statistics, when the caller kept them, save the left factor's first pass
    const bool saved = fused_left && g.fout != nullptr && g.fstats != nullptr;
    // gather q, dout (query map; both row orders) and k, v (key map)
    {
        constexpr int kPer = 8 / sizeof(T);
        const int64_t tq = (int64_t)n * MQ * (D / kPer), tk = (int64_t)n * MK * (D / kPer);
        const unsigned gq = (unsigned)((tq + 255) / 256), gk = (unsigned)((tk + 255) / 256);
        // the fused kernels read q, dout (and out) rows where the callers' tensors have them
        if (!fused_fwd || !fused_right)
            hipLaunchKernelGGL((gather_rows<E>), dim3(gq), dim3(256), 0, stream, (T*)(ws + lay.Qk), p.q, p.qs[0], p.qs[1], p.qs[2], p.qmap,
                               na, H, D, p.unit0, 0, tq);
        if (!fused_left) {
            hipLaunchKernelGGL((gather_rows<E>), dim3(gq), dim3(256), 0, stream, (T*)(ws + lay.Qa), p.q, p.qs[0], p.qs[1], p.qs[2], p.qmap,
                               na, H, D, p.unit0, 1, tq);
            hipLaunchKernelGGL((gather_rows<E>), dim3(gq), dim3(256), 0, stream, (T*)(ws + lay.dOa), g.dout, g.dos[0], g.dos[1], g.dos[2],
                               p.qmap, na, H, D, p.unit0, 1, tq);
        }
        if (!parts.dqk)
            hipLaunchKernelGGL((gather_rows<E>), dim3(gk), dim3(256), 0, stream, (T*)(ws + lay.Kk), p.k, p.ks[0], p.ks[1], p.ks[2], p.kmap,
                               nf, H, D, p.unit0, 0, tk);
        if (!fused_right)                               // the fused right-factor kernel reads v where it is
            hipLaunchKernelGGL((gather_rows<E>), dim3(gk), dim3(256), 0, stream, (T*)(ws + lay.Vk), p.v, p.vs[0], p.vs[1], p.vs[2], p.kmap,
                           nf, H, D, p.unit0, 0, tk);
    }
    const int nuk = n * b1, nt = n * b1 * nf;
    // operands per (u, k): whole [AJ x D] / [NL x D] / [AJ x NL] matrices
    const Op Qk_uk{lay.Qk, D, (int64_t)AJ * D}, Kk_uk{lay.Kk, D, (int64_t)NL * D};
    const Op S1_uk{lay.S1f, NL, (int64_t)AJ * NL}, dS1_uk{lay.dS1, NL, (int64_t)AJ * NL};
    const Op dQk_uk{lay.dQk, D, (int64_t)AJ * D}, dKk_uk{lay.dKk, D, (int64_t)NL * D};
    // operands per t = (u, k, f): [b2 x D] blocks of K, V, dK, dV; [AJ x b2] blocks of R, dR; [AJ x D] blocks of Kbar, Y, dKbar, dY
    const Op Kk_t{lay.Kk, D, (int64_t)b2 * D}, Vk_t{lay.Vk, D, (int64_t)b2 * D};
    const Op dKk_t{lay.dKk, D, (int64_t)b2 * D}, dVk_t{lay.dVk, D, (int64_t)b2 * D};
    const Op dRb_t{lay.dRb, b2, (int64_t)AJ * b2};
    const Op Kbar_t{lay.Kbar, D, (int64_t)AJ * D}, Y_t{lay.Y, D, (int64_t)AJ * D};
    const Op dKbar_t{lay.dKbar, D, (int64_t)AJ * D}, dY_t{lay.dY, D, (int64_t)AJ * D};

    const Op Rb_t{lay.Rb, rb_ld, (int64_t)AJ * rb_ld};
    if (fused_fwd) {
        MonarchArgs f1 = p;
        f1.kbar = ws + lay.Kbar;
        f1.y = ws + lay.Y;
        f1.cl = (float*)(ws + lay.c);
        f1.rb = ws + lay.Rb;
        f1.ws_unit = (uint32_t)((int64_t)RR * AJ);
        f1.ws_aj = 1;
        f1.ws_row = (uint32_t)(nf * AJ);
        f1.ws_f = (uint32_t)AJ;
        f1.cl_unit = f1.ws_unit;         // c sits where its scratch row does: [row][(a, j)]
        f1.cl_aj = 1;
        f1.cl_row = 1;
        if (!cx.status) cx.status = launch_monarch_step1(f1, left_dtype<E>(), n, stream);
    } else {
        // 1. S1 = Qk Kk^T per (u, k)
        gemm(cx, false, true, AJ, NL, D, 1.f, 0.f, Qk_uk, Kk_uk, S1_uk, tE, tF, nuk);
        hipLaunchKernelGGL((softmax_right<E>), dim3((unsigned)((nseg + 3) / 4)), dim3(256), 0, stream, (const float*)(ws + lay.S1f),
                           (T*)(ws + lay.Rb), (float*)(ws + lay.c), b1, AJ, nf, b2, s, nseg);
        // 2, 3. Kbar, Y blocks = R block . K / V block per t
        gemm(cx, false, false, AJ, D, b2, 1.f, 0.f, Rb_t, Kk_t, Kbar_t, tE, tE, nt);
        gemm(cx, false, false, AJ, D, b2, 1.f, 0.f, Rb_t, Vk_t, Y_t, tE, tE, nt);
    }
    if (fused_left) {
        // 4-7 in one kernel: statistics and gradients of the left factor without the [i x r] matrices in memory
        if (!cx.status)
            cx.status = launch_monarch_bwd_left(left_dtype<E>(), D, n, b1, b2, AJ, nf, p.causal, s, p.q, p.qs, g.dout, saved ? g.fout : nullptr,
                                                g.dos, p.qmap, H, p.unit0, ws + lay.Kbar, ws + lay.Y, (const float*)(ws + lay.c),
                                                fused_fwd ? 1 : 0, ws + lay.dKbar, ws + lay.dY, (float*)(ws + lay.dc), ws + lay.dS2, ds2_ld,
                                                saved ? g.fstats : nullptr, (b1 + 31) / 32 * 32, stream);
    } else {
        // 4, 5. per unit and (a, j): S2 = q_i . Kbar_r, dLm = dO_i . Y_r; the [RR x D] matrix of column aj is every AJ-th row
        for (int u = 0; u < n && !cx.status; ++u) {
            const Op Qa_u{lay.Qa + (size_t)u * MQ * D * e, D, (int64_t)b1 * D}, dOa_u{lay.dOa + (size_t)u * MQ * D * e, D, (int64_t)b1 * D};
            const Op Kbar_u{lay.Kbar + (size_t)u * AJ * RR * D * e, (int64_t)AJ * D, D}, Y_u{lay.Y + (size_t)u * AJ * RR * D * e, (int64_t)AJ * D, D};
            const Op S2_u{lay.S2f + (size_t)u * AJ * b1 * RR * 4, RR, (int64_t)b1 * RR}, dLm_u{lay.dLmf + (size_t)u * AJ * b1 * RR * 4, RR, (int64_t)b1 * RR};
            gemm(cx, false, true, b1, RR, D, 1.f, 0.f, Qa_u, Kbar_u, S2_u, tE, tF, AJ);
            gemm(cx, false, true, b1, RR, D, 1.f, 0.f, dOa_u, Y_u, dLm_u, tE, tF, AJ);
        }
        hipLaunchKernelGGL((softmax_left<E>), dim3((unsigned)((int64_t)n * AJ * b1)), dim3(256), 0, stream, (const float*)(ws + lay.S2f),
                           (const float*)(ws + lay.dLmf), (const float*)(ws + lay.c), (T*)(ws + lay.L), (T*)(ws + lay.dS2), b1, b2, AJ, nf,
                           p.causal, s);
        {
            const int64_t tot = (int64_t)n * AJ * RR;
            hipLaunchKernelGGL((reduce_dc<E>), dim3((unsigned)((tot + 255) / 256)), dim3(256), 0, stream, (const T*)(ws + lay.dS2),
                               (float*)(ws + lay.dc), b1, AJ, RR, tot);
        }
        // 6, 7, 8. per unit and (a, j): dY = L^T dO, dKbar = s dS2^T q, dQ (left factor) = s dS2 Kbar
        for (int u = 0; u < n && !cx.status; ++u) {
            const Op Qa_u{lay.Qa + (size_t)u * MQ * D * e, D, (int64_t)b1 * D}, dOa_u{lay.dOa + (size_t)u * MQ * D * e, D, (int64_t)b1 * D};
            const Op Kbar_u{lay.Kbar + (size_t)u * AJ * RR * D * e, (int64_t)AJ * D, D};
            const Op dKbar_u{lay.dKbar + (size_t)u * AJ * RR * D * e, (int64_t)AJ * D, D}, dY_u{lay.dY + (size_t)u * AJ * RR * D * e, (int64_t)AJ * D, D};
            const Op L_u{lay.L + (size_t)u * AJ * b1 * RR * e, RR, (int64_t)b1 * RR}, dS2_u{lay.dS2 + (size_t)u * AJ * b1 * RR * e, RR, (int64_t)b1 * RR};
            const Op dQa_u{lay.dQa + (size_t)u * MQ * D * 4, D, (int64_t)b1 * D};
            gemm(cx, true, false, RR, D, b1, 1.f, 0.f, L_u, dOa_u, dY_u, tE, tE, AJ);
            gemm(cx, true, false, RR, D, b1, s, 0.f, dS2_u, Qa_u, dKbar_u, tE, tE, AJ);
        }
    }
    // 8. per unit and (a, j): dQ (left factor) = s dS2 Kbar
    for (int u = 0; u < n && !cx.status && !fused_dqa; ++u) {
        const Op Kbar_u{lay.Kbar + (size_t)u * AJ * RR * D * e, (int64_t)AJ * D, D};
        const Op dS2_u{lay.dS2 + (size_t)u * AJ * b1 * ds2_ld * e, ds2_ld, (int64_t)b1 * ds2_ld};
        const Op dQa_u{lay.dQa + (size_t)u * MQ * D * 4, D, (int64_t)b1 * D};
        gemm(cx, false, false, b1, D, RR, s, 0.f, dS2_u, Kbar_u, dQa_u, tE, tF, AJ);
    }
    if (fused_right) {
        if (!cx.status)
            cx.status = launch_monarch_bwd_right(left_dtype<E>(), D, nt, b1, b2, AJ, nf, s, p.k, p.ks, p.v, p.vs, ws + lay.Rb,
                                                 ws + lay.dKbar, ws + lay.dY, (const float*)(ws + lay.dc), p.q, p.qs, p.qmap, ws + lay.dS1, g.dk,
                                                 g.dv, g.dks, g.dk_row0, p.kmap, H, p.unit0, g.kv_f0, g.kv_f1, stream);
    } else {
        // 9. dR block = dKbar block . K block^T + dY block . V block^T per t
        gemm(cx, false, true, AJ, b2, D, 1.f, 0.f, dKbar_t, Kk_t, dRb_t, tE, tF, nt);
        gemm(cx, false, true, AJ, b2, D, 1.f, 1.f, dY_t, Vk_t, dRb_t, tE, tF, nt);
    }
    if (fused_right) {
        // dS1 is already written
    } else if (fused_fwd)
        hipLaunchKernelGGL((softmax_right_bwd_r<E>), dim3((unsigned)((nseg + 3) / 4)), dim3(256), 0, stream, (const T*)(ws + lay.Rb),
                           (const float*)(ws + lay.dRb), (const float*)(ws + lay.dc), (T*)(ws + lay.dS1), b1, AJ, nf, b2, nseg);
    else
        hipLaunchKernelGGL((softmax_right_bwd<E>), dim3((unsigned)((nseg + 3) / 4)), dim3(256), 0, stream, (const float*)(ws + lay.S1f),
                           (const float*)(ws + lay.dRb), (const float*)(ws + lay.dc), (T*)(ws + lay.dS1), b1, AJ, nf, b2, s, nseg);
    // 10. dQ (right factor) = s dS1 K per (u, k)
    if (parts.dqk) {
        if (!cx.status)
            cx.status = launch_monarch_bwd_dqk(left_dtype<E>(), D, nuk, b1, b2, AJ, nf, s, p.k, p.ks, p.kmap, ws + lay.dS1,
                                               (float*)(ws + lay.dQk), H, p.unit0, stream);
    } else {
        gemm(cx, false, false, AJ, D, NL, s, 0.f, dS1_uk, Kk_uk, dQk_uk, tE, tF, nuk);
    }
    if (!fused_right) {
        // 11. dK = s dS1^T q per (u, k)
        gemm(cx, true, false, NL, D, AJ, s, 0.f, dS1_uk, Qk_uk, dKk_uk, tE, tF, nuk);
        // 12. dK block += R block^T dKbar block;  13. dV block = R block^T dY block per t
        gemm(cx, true, false, b2, D, AJ, 1.f, 1.f, Rb_t, dKbar_t, dKk_t, tE, tF, nt);
        gemm(cx, true, false, b2, D, AJ, 1.f, 0.f, Rb_t, dY_t, dVk_t, tE, tF, nt);
    }
    if (cx.status) return cx.status;
    // scatter the gradients back to the callers' layouts
    {
        const int64_t tq = (int64_t)n * MQ * (D / 4);
        if (fused_dqa)
            cx.status = launch_monarch_bwd_dqa(left_dtype<E>(), D, n, b1, b2, AJ, nf, s, ws + lay.Kbar, ws + lay.dS2, ds2_ld,
                                               (const float*)(ws + lay.dQk), g.dq, g.dqs, p.qmap, H, p.unit0, stream);
        else
            hipLaunchKernelGGL(scatter_dq, dim3((unsigned)((tq + 255) / 256)), dim3(256), 0, stream, (const float*)(ws + lay.dQa),
                               (const float*)(ws + lay.dQk), g.dq, g.dqs[0], g.dqs[1], g.dqs[2], p.qmap, na, H, D, p.unit0, tq);
        const int64_t tk = (int64_t)n * b1 * (g.kv_f1 - g.kv_f0) * b2 * (D / 4);
        if (!fused_right && tk > 0)
            hipLaunchKernelGGL((scatter_dkv<E>), dim3((unsigned)((tk + 255) / 256)), dim3(256), 0, stream, (const float*)(ws + lay.dKk),
                               (const float*)(ws + lay.dVk), (T*)g.dk, (T*)g.dv, g.dks[0], g.dks[1], g.dks[2], p.kmap, nf, g.kv_f0,
                               g.kv_f1, g.dk_row0, H, D, p.unit0, tk);
        if (cx.status) return cx.status;
    }
    hipError_t err = hipGetLastError();
    if (err != hipSuccess) {
        set_error("hip launch failed: %s", hipGetErrorString(err));
        return SFM_ERR_HIP;
    }
    return SFM_OK;
}

}  // namespace

bool monarch_bwd_gemm_available() { return blas_load(); }

bool monarch_bwd_all_fused(const MonarchArgs& p, int dtype, const int64_t* dkv_stride) {
    const Parts f = make_parts(p, dtype, dkv_stride);
    return f.left && f.fwd && f.dqa && f.right && f.dqk;
}

size_t monarch_bwd_gemm_bytes(const MonarchArgs& p, int dtype, int nunits, const int64_t* dkv_stride) {
    return make_layout(p, nunits, dtype == SFM_F32 ? 4 : 2, make_parts(p, dtype, dkv_stride)).total;
}

int launch_monarch_bwd_gemm(const MonarchBwdArgs& g, int dtype, int nunits, void* workspace, hipStream_t stream) {
    if (!monarch_bwd_all_fused(g.p, dtype, g.dks) && !blas_load()) {
        set_error("rocBLAS could not be loaded");
        return SFM_ERR_UNSUPPORTED;
    }
    if (g.p.b2 > 64 * kSegPerLane || g.p.nf * g.p.b1 > 256 * kLeftPerThread) {
        set_error("Monarch backward: b2=%d or rows=%d beyond the row kernels' limits (%d, %d)", g.p.b2, g.p.nf * g.p.b1,
                  64 * kSegPerLane, 256 * kLeftPerThread);
        return SFM_ERR_UNSUPPORTED;
    }
    if (dtype == SFM_F32) return run<float>(g, nunits, workspace, stream);
    if (dtype == SFM_BF16) return run<BF16>(g, nunits, workspace, stream);
    return run<F16>(g, nunits, workspace, stream);
}

}  // namespace sfm
