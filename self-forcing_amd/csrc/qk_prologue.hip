// Fused q/k prologue: RMSNorm over the full model dim + 3-D RoPE, writing roped K and V straight
// into the KV cache (Monarch block order) and roped Q to its own tensor.
//
// Replaces, per layer and per pass, the eager chain
//   WanRMSNorm           wan/modules/model.py:462-478   (fp32 normalise, cast back, times weight)
//   causal_rope_apply    wan/modules/causal_model.py:687-715   (complex128 rotation of interleaved pairs)
//   rearrange + slice-assign into the cache   wan/modules/monarch_attn.py:1783-1785, 1230-1231
// HBM-bound: one workgroup per token reads 3 rows of C elements and writes 3.
//
// Rounding points follow the reference: the normalised value is rounded to the tensor dtype, the
// product with the weight is rounded again, the rotation is done in float64 from the float64
// angle table and rounded once.

#include "sfm_common.hpp"

namespace sfm {

template <typename T> struct Row8;   // 8 consecutive elements <-> 8 floats

template <> struct Row8<float> {
    static constexpr int kBytes = 32;
    static __device__ __forceinline__ void load(const void* p, int64_t e, float* x) {
        const f32x4* s = (const f32x4*)((const float*)p + e);
        f32x4 a = s[0], b = s[1];
        x[0] = a.x; x[1] = a.y; x[2] = a.z; x[3] = a.w; x[4] = b.x; x[5] = b.y; x[6] = b.z; x[7] = b.w;
    }
    static __device__ __forceinline__ void store(void* p, int64_t e, const float* x) {
        f32x4* d = (f32x4*)((float*)p + e);
        f32x4 a = {x[0], x[1], x[2], x[3]}, b = {x[4], x[5], x[6], x[7]};
        d[0] = a; d[1] = b;
    }
    static __device__ __forceinline__ float rnd(float x) { return x; }
    struct Raw { f32x4 a, b; };
    static __device__ __forceinline__ Raw load_raw(const void* p, int64_t e) {
        const f32x4* s = (const f32x4*)((const float*)p + e);
        return {s[0], s[1]};
    }
    static __device__ __forceinline__ void store_raw(void* p, int64_t e, const Raw& r) {
        f32x4* d = (f32x4*)((float*)p + e);
        d[0] = r.a; d[1] = r.b;
    }
};

template <class E> struct Row8_16 {
    static constexpr int kBytes = 16;
    static __device__ __forceinline__ void load(const void* p, int64_t e, float* x) {
        u32x4 w = *(const u32x4*)((const uint16_t*)p + e);
        uint32_t ww[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            x[2 * i] = E::to_float((uint16_t)(ww[i] & 0xffffu));
            x[2 * i + 1] = E::to_float((uint16_t)(ww[i] >> 16));
        }
    }
    static __device__ __forceinline__ void store(void* p, int64_t e, const float* x) {
        u32x4 w;
        w.x = pack2<E>(x[0], x[1]); w.y = pack2<E>(x[2], x[3]); w.z = pack2<E>(x[4], x[5]); w.w = pack2<E>(x[6], x[7]);
        // written once and read by a later kernel: streaming stores keep the rows out of the way of the loads
        __builtin_nontemporal_store(w, (u32x4*)((uint16_t*)p + e));
    }
    static __device__ __forceinline__ float rnd(float x) { return E::to_float(E::from_float(x)); }
    using Raw = u32x4;
    static __device__ __forceinline__ Raw load_raw(const void* p, int64_t e) { return *(const u32x4*)((const uint16_t*)p + e); }
    static __device__ __forceinline__ void store_raw(void* p, int64_t e, const Raw& r) {
        __builtin_nontemporal_store(r, (u32x4*)((uint16_t*)p + e));
    }
};
template <> struct Row8<BF16> : Row8_16<BF16> {};
template <> struct Row8<F16> : Row8_16<F16> {};

constexpr int kMaxThreads = 512;

// One workgroup per token, CPT chunks of 8 elements per thread.  Rows of up to 1536 elements are one wave's work (64
// lanes x 3 chunks: no second wave to wait for, and every token of a 4680-token chunk is resident at once); longer rows
// take the chunk count divided by CPT, rounded up to whole waves (320 threads x 2 chunks at model dim 5120), so that no
// lane idles.  A thread's q, k, v chunks (and, with fewer than three chunks, its four rotation pairs) are requested before
// the row's sum of squares is reduced; the norm weights (cache hits) are fetched after it, which keeps the kernel at
// 5-8 waves per SIMD.  The sums
// of squares are accumulated in float64 (per thread over its chunks, then a butterfly over the wave, then the waves in
// order).
template <typename T, int CPT>
__global__ __launch_bounds__(kMaxThreads) __attribute__((amdgpu_waves_per_eu(5))) void qk_prologue_kernel(sfm_prologue_desc p, TokMap map, const void* xq,
                                                                  const void* xk, const void* xv, const void* wq,
                                                                  const void* wk, const double* __restrict__ rope,
                                                                  void* q_out, void* kc, void* vc) {
    using R8 = Row8<T>;
    __shared__ double red[2][kMaxThreads / 64];
    const int tid = threadIdx.x, nt = blockDim.x;
    const int b = blockIdx.y, s = blockIdx.x;
    const int D = p.D, C = p.H * p.D;
    const int nchunk = C / 8;

    // the row's loads go out first; the token's coordinates are worked out while they are in flight
    const int64_t xoff = (int64_t)b * p.x_stride[0] + (int64_t)s * p.x_stride[1];
    float q[CPT][8], k[CPT][8];
    typename R8::Raw v[CPT];
#pragma unroll
    for (int t = 0; t < CPT; ++t) {
        const int ch = tid + t * nt;
        if (ch < nchunk) {
            R8::load(xq, xoff + ch * 8, q[t]);
            R8::load(xk, xoff + ch * 8, k[t]);
            v[t] = R8::load_raw(xv, xoff + ch * 8);
        }
    }

    // token coordinates and its row in the cache (block order within the new chunk)
    const int frame = s / (p.h * p.w);
    const int rem = s - frame * p.h * p.w;
    const int row = rem / p.w, col = rem - row * p.w;
    const int A = frame / map.f_tied, ft = frame - A * map.f_tied;
    const int c = row / map.hh, ii = row - c * map.hh;
    const int e = col / map.ww, j = col - e * map.ww;
    const int bf = (A * map.h_reduce + c) * map.w_reduce + e;
    const int64_t crow = p.start_idx + ((int64_t)bf * map.b1 + (ft * map.hh + ii)) * map.b2 + j;
    const int64_t cbase = (int64_t)b * p.cache_stride[0] + crow * p.cache_stride[1];

    double sq = 0.0, sk = 0.0;
#pragma unroll
    for (int t = 0; t < CPT; ++t) {
        const int ch = tid + t * nt;
        if (ch < nchunk) {
            // V is copied as is
            const int hd = (ch * 8) / D, d0 = (ch * 8) % D;
            R8::store_raw(vc, cbase + (int64_t)hd * p.cache_stride[2] + d0, v[t]);
        }
    }
    // the rotation pairs of a thread's chunks: the same for every chunk when the block's stride is a multiple of the
    // head dim (always so for power-of-two head dims up to 512), fetched per chunk otherwise
    const int half = D / 2;
    const int n0 = half - 2 * (half / 3), n1 = half / 3;
    const int pos0 = frame + p.start_frame;
    const bool same_pairs = (nt * 8) % D == 0;
    double cs[4], sn[4];
    auto load_pairs = [&](int d0) {
#pragma unroll
        for (int pr = 0; pr < 4; ++pr) {
            const int mpair = d0 / 2 + pr;
            const int pos = mpair < n0 ? pos0 : (mpair < n0 + n1 ? row : col);
            const double2 v = *(const double2*)(rope + ((int64_t)pos * half + mpair) * 2);
            cs[pr] = v.x;
            sn[pr] = v.y;
        }
    };
    constexpr bool kEarlyPairs = CPT < 3;       // three chunks of q and k fill the registers of a 5-wave kernel
    if (same_pairs && kEarlyPairs) load_pairs((tid * 8) % D);

#pragma unroll
    for (int t = 0; t < CPT; ++t) {
        if (tid + t * nt < nchunk) {
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                sq += (double)q[t][i] * q[t][i];
                sk += (double)k[t][i] * k[t][i];
            }
        }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        sq += __shfl_xor(sq, o);
        sk += __shfl_xor(sk, o);
    }
    if ((tid & 63) == 0) {
        red[0][tid >> 6] = sq;
        red[1][tid >> 6] = sk;
    }
    __syncthreads();
    sq = sk = 0.0;
    for (int w = 0; w < nt / 64; ++w) {
        sq += red[0][w];
        sk += red[1][w];
    }
    const float rq = 1.0f / sqrtf((float)(sq / C) + p.eps);
    const float rk = 1.0f / sqrtf((float)(sk / C) + p.eps);
    if (same_pairs && !kEarlyPairs) load_pairs((tid * 8) % D);

#pragma unroll
    for (int t = 0; t < CPT; ++t) {
        const int ch = tid + t * nt;
        if (ch < nchunk) {
            const int hd = (ch * 8) / D, d0 = (ch * 8) % D;
            if (!same_pairs) load_pairs(d0);
            float wqv[8], wkv[8], oq[8], ok[8];
            R8::load(wq, ch * 8, wqv);
            R8::load(wk, ch * 8, wkv);
#pragma unroll
            for (int pr = 0; pr < 4; ++pr) {
                const double q0 = R8::rnd(R8::rnd(q[t][2 * pr] * rq) * wqv[2 * pr]);
                const double q1 = R8::rnd(R8::rnd(q[t][2 * pr + 1] * rq) * wqv[2 * pr + 1]);
                const double k0 = R8::rnd(R8::rnd(k[t][2 * pr] * rk) * wkv[2 * pr]);
                const double k1 = R8::rnd(R8::rnd(k[t][2 * pr + 1] * rk) * wkv[2 * pr + 1]);
                oq[2 * pr] = (float)(q0 * cs[pr] - q1 * sn[pr]);
                oq[2 * pr + 1] = (float)(q0 * sn[pr] + q1 * cs[pr]);
                ok[2 * pr] = (float)(k0 * cs[pr] - k1 * sn[pr]);
                ok[2 * pr + 1] = (float)(k0 * sn[pr] + k1 * cs[pr]);
            }
            R8::store(q_out, (int64_t)b * p.q_stride[0] + (int64_t)s * p.q_stride[1] + (int64_t)hd * p.q_stride[2] + d0, oq);
            R8::store(kc, cbase + (int64_t)hd * p.cache_stride[2] + d0, ok);
        }
    }
}

template <typename T>
static void launch_t(int cpt, dim3 grid, dim3 block, hipStream_t stream, const sfm_prologue_desc& d, const TokMap& map,
                     const void* xq, const void* xk, const void* xv, const void* wq, const void* wk, const double* rope,
                     void* q_out, void* kc, void* vc) {
    if (cpt == 1)
        hipLaunchKernelGGL((qk_prologue_kernel<T, 1>), grid, block, 0, stream, d, map, xq, xk, xv, wq, wk, rope, q_out, kc, vc);
    else if (cpt == 3)
        hipLaunchKernelGGL((qk_prologue_kernel<T, 3>), grid, block, 0, stream, d, map, xq, xk, xv, wq, wk, rope, q_out, kc, vc);
    else
        hipLaunchKernelGGL((qk_prologue_kernel<T, 2>), grid, block, 0, stream, d, map, xq, xk, xv, wq, wk, rope, q_out, kc, vc);
}

// Model dims up to kMaxThreads x 2 chunks x 8 elements = 8192 (the entry point checks it).
int launch_prologue(const sfm_prologue_desc& d, const TokMap& map, const void* xq, const void* xk, const void* xv,
                    const void* wq, const void* wk, const double* rope, void* q_out, void* kc, void* vc,
                    hipStream_t stream) {
    const int nchunk = d.H * d.D / 8;
    const int cpt = nchunk <= 192 ? (nchunk + 63) / 64 : (nchunk > kMaxThreads ? 2 : 1);
    const int nt = (((nchunk + cpt - 1) / cpt) + 63) / 64 * 64;
    dim3 grid((unsigned)d.S, (unsigned)d.B), block(nt);
    if (d.dtype == SFM_BF16)
        launch_t<BF16>(cpt, grid, block, stream, d, map, xq, xk, xv, wq, wk, rope, q_out, kc, vc);
    else if (d.dtype == SFM_F16)
        launch_t<F16>(cpt, grid, block, stream, d, map, xq, xk, xv, wq, wk, rope, q_out, kc, vc);
    else
        launch_t<float>(cpt, grid, block, stream, d, map, xq, xk, xv, wq, wk, rope, q_out, kc, vc);
    hipError_t err = hipGetLastError();
    if (err != hipSuccess) {
        set_error("hip launch failed: %s", hipGetErrorString(err));
        return SFM_ERR_HIP;
    }
    return SFM_OK;
}

}  // namespace sfm
