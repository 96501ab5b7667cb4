// Fused element-wise kernels of the causal Wan block around the attention op (HBM-bound, one pass each):
//
//   ln_modulate     y = LayerNorm(x) * (1 + scale[frame]) + shift[frame]         (norm1 / norm2 + adaLN,
//                   wan/modules/causal_model.py:1179-1183, 1198-1201), or with an affine weight/bias
//                   and no modulation (norm3, causal_model.py:1194)
//   gate_residual   x += y * gate[frame]                                          (causal_model.py:1189, 1203-1204)
//   rms_norm        y = (x * rsqrt(mean(x^2) + eps)).type_as(x) * w               (WanRMSNorm, model.py:462-478)
//   gate_residual_ln  gate_residual followed by ln_modulate of the updated row, one pass over it
//
// One wave per token row for the normalisations (C <= 8192; the row stays in registers, sums by lane shuffles,
// no barrier), one workgroup per row for the residual.  Statistics in fp32; the reference's rounding points are kept:
// every eager op of the reference rounds to the tensor dtype, so the kernels round after the same steps
// (LayerNorm output, 1 + scale, the product, the sum; y * gate, x + ...).

#include "sfm_common.hpp"

namespace sfm {

template <typename T> struct V8;   // 8 consecutive elements <-> 8 floats
template <> struct V8<float> {
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
};
template <class E> struct V8_16 {
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
        *(u32x4*)((uint16_t*)p + e) = w;
    }
    static __device__ __forceinline__ float rnd(float x) { return E::to_float(E::from_float(x)); }
};
template <> struct V8<BF16> : V8_16<BF16> {};
template <> struct V8<F16> : V8_16<F16> {};

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
    return v;
}

// x [rows, C] (row stride xs), scale/shift [B, F, C] addressed through (row -> frame) = row / rows_per_frame,
// with element strides ms (between frames); weight/bias [C] or nullptr.  NT = 8-element chunks per lane.
template <typename T, int NT>
__global__ __launch_bounds__(256) void ln_modulate_kernel(const void* x, int64_t xs, void* y, int64_t ys, int C, float eps,
                                                          const void* scale, const void* shift, int64_t ms,
                                                          int rows_per_frame, const void* weight, const void* bias, int64_t rows) {
    using V = V8<T>;
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;
    const int lane = threadIdx.x & 63, nch = C / 8;
    float v[NT][8];
    float sum = 0.f;
#pragma unroll
    for (int t = 0; t < NT; ++t) {
        const int ch = lane + t * 64;
        if (ch < nch) {
            V::load(x, row * xs + ch * 8, v[t]);
#pragma unroll
            for (int i = 0; i < 8; ++i) sum += v[t][i];
        }
    }
    const float mean = wave_sum(sum) / C;
    float sq = 0.f;
#pragma unroll
    for (int t = 0; t < NT; ++t) {
        const int ch = lane + t * 64;
        if (ch < nch) {
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                float d = v[t][i] - mean;
                sq += d * d;
            }
        }
    }
    const float rstd = 1.0f / sqrtf(wave_sum(sq) / C + eps);
    const int64_t moff = (row / rows_per_frame) * ms;
#pragma unroll
    for (int t = 0; t < NT; ++t) {
        const int ch = lane + t * 64;
        if (ch < nch) {
            float o[8];
            if (weight != nullptr) {
                float w[8], b[8];
                V::load(weight, ch * 8, w);
                V::load(bias, ch * 8, b);
#pragma unroll
                for (int i = 0; i < 8; ++i) o[i] = (v[t][i] - mean) * rstd * w[i] + b[i];
            } else {
                float sc[8], sh[8];
                V::load(scale, moff + ch * 8, sc);
                V::load(shift, moff + ch * 8, sh);
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    float n = V::rnd((v[t][i] - mean) * rstd);
                    float g = V::rnd(1.0f + sc[i]);
                    o[i] = V::rnd(n * g) + sh[i];
                }
            }
            V::store(y, row * ys + ch * 8, o);
        }
    }
}

// x += y * gate (gate = nullptr: x += y), written back, then out = the LayerNorm variant of ln_modulate_kernel
// applied to the updated (rounded) row, which never leaves the registers in between.
template <typename T, int NT>
__global__ __launch_bounds__(256) void gate_residual_ln_kernel(void* x, int64_t xs, const void* yv, int64_t ys, const void* gate,
                                                               int64_t gms, int g_rows_per_frame, void* out, int64_t os, int C,
                                                               float eps, const void* scale, const void* shift, int64_t ms,
                                                               int rows_per_frame, const void* weight, const void* bias, int64_t rows) {
    using V = V8<T>;
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;
    const int lane = threadIdx.x & 63, nch = C / 8;
    const int64_t goff = gate != nullptr ? (row / g_rows_per_frame) * gms : 0;
    float v[NT][8];
    float sum = 0.f;
#pragma unroll
    for (int t = 0; t < NT; ++t) {
        const int ch = lane + t * 64;
        if (ch < nch) {
            float b[8], g[8];
            V::load(x, row * xs + ch * 8, v[t]);
            V::load(yv, row * ys + ch * 8, b);
            if (gate != nullptr) {
                V::load(gate, goff + ch * 8, g);
#pragma unroll
                for (int i = 0; i < 8; ++i) {
#pragma clang fp contract(off)      // two eager ops in the reference: no fma
                    float prod = b[i] * g[i];
                    v[t][i] = V::rnd(v[t][i] + V::rnd(prod));
                }
            } else {
#pragma unroll
                for (int i = 0; i < 8; ++i) v[t][i] = V::rnd(v[t][i] + b[i]);
            }
            V::store(x, row * xs + ch * 8, v[t]);
#pragma unroll
            for (int i = 0; i < 8; ++i) sum += v[t][i];
        }
    }
    const float mean = wave_sum(sum) / C;
    float sq = 0.f;
#pragma unroll
    for (int t = 0; t < NT; ++t) {
        const int ch = lane + t * 64;
        if (ch < nch) {
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                float d = v[t][i] - mean;
                sq += d * d;
            }
        }
    }
    const float rstd = 1.0f / sqrtf(wave_sum(sq) / C + eps);
    const int64_t moff = (row / rows_per_frame) * ms;
#pragma unroll
    for (int t = 0; t < NT; ++t) {
        const int ch = lane + t * 64;
        if (ch < nch) {
            float o[8];
            if (weight != nullptr) {
                float w[8], b[8];
                V::load(weight, ch * 8, w);
                V::load(bias, ch * 8, b);
#pragma unroll
                for (int i = 0; i < 8; ++i) o[i] = (v[t][i] - mean) * rstd * w[i] + b[i];
            } else {
                float sc[8], sh[8];
                V::load(scale, moff + ch * 8, sc);
                V::load(shift, moff + ch * 8, sh);
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    float n = V::rnd((v[t][i] - mean) * rstd);
                    float g = V::rnd(1.0f + sc[i]);
                    o[i] = V::rnd(n * g) + sh[i];
                }
            }
            V::store(out, row * os + ch * 8, o);
        }
    }
}

template <typename T>
__global__ __launch_bounds__(256) void gate_residual_kernel(void* x, int64_t xs, const void* y, int64_t ys, int C,
                                                            const void* gate, int64_t ms, int rows_per_frame) {
    using V = V8<T>;
    const int row = blockIdx.x, nch = C / 8;
    const int64_t moff = (int64_t)(row / rows_per_frame) * ms;
    for (int ch = threadIdx.x; ch < nch; ch += 256) {
        float a[8], b[8], g[8];
        V::load(x, (int64_t)row * xs + ch * 8, a);
        V::load(y, (int64_t)row * ys + ch * 8, b);
        if (gate != nullptr) {
            V::load(gate, moff + ch * 8, g);
#pragma unroll
            for (int i = 0; i < 8; ++i) {
#pragma clang fp contract(off)      // two eager ops in the reference: no fma
                float prod = b[i] * g[i];
                a[i] = a[i] + V::rnd(prod);
            }
        } else {
#pragma unroll
            for (int i = 0; i < 8; ++i) a[i] += b[i];
        }
        V::store(x, (int64_t)row * xs + ch * 8, a);
    }
}

template <typename T, int NT>
__global__ __launch_bounds__(256) void rms_norm_kernel(const void* x, int64_t xs, void* y, int64_t ys, int C, float eps,
                                                       const void* weight, int64_t rows) {
    using V = V8<T>;
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;
    const int lane = threadIdx.x & 63, nch = C / 8;
    float v[NT][8];
    float sq = 0.f;
#pragma unroll
    for (int t = 0; t < NT; ++t) {
        const int ch = lane + t * 64;
        if (ch < nch) {
            V::load(x, row * xs + ch * 8, v[t]);
#pragma unroll
            for (int i = 0; i < 8; ++i) sq += v[t][i] * v[t][i];
        }
    }
    const float r = 1.0f / sqrtf(wave_sum(sq) / C + eps);
#pragma unroll
    for (int t = 0; t < NT; ++t) {
        const int ch = lane + t * 64;
        if (ch < nch) {
            float w[8], o[8];
            V::load(weight, ch * 8, w);
#pragma unroll
            for (int i = 0; i < 8; ++i) o[i] = V::rnd(v[t][i] * r) * w[i];
            V::store(y, row * ys + ch * 8, o);
        }
    }
}

#define SFM_DISPATCH(dtype, KERNEL, grid, stream, ...)                                                         \
    do {                                                                                                         \
        if ((dtype) == SFM_BF16) hipLaunchKernelGGL((KERNEL<BF16>), grid, dim3(256), 0, stream, __VA_ARGS__);    \
        else if ((dtype) == SFM_F16) hipLaunchKernelGGL((KERNEL<F16>), grid, dim3(256), 0, stream, __VA_ARGS__); \
        else hipLaunchKernelGGL((KERNEL<float>), grid, dim3(256), 0, stream, __VA_ARGS__);                       \
    } while (0)

static int finish() {
    hipError_t err = hipGetLastError();
    if (err != hipSuccess) {
        set_error("hip launch failed: %s", hipGetErrorString(err));
        return SFM_ERR_HIP;
    }
    return SFM_OK;
}

// wave-per-row kernels: 4 rows per workgroup, NT = chunks of 8 elements per lane (3 covers C <= 1536, 10 C <= 5120)
#define SFM_DISPATCH_ROWS(dtype, KERNEL, C, rows, stream, ...)                                                      \
    do {                                                                                                            \
        const dim3 grid((unsigned)(((rows) + 3) / 4));                                                              \
        const int nt_ = ((C) / 8 + 63) / 64;                                                                        \
        if (nt_ <= 3) SFM_DISPATCH_NT(dtype, KERNEL, 3, grid, stream, __VA_ARGS__);                                 \
        else if (nt_ <= 10) SFM_DISPATCH_NT(dtype, KERNEL, 10, grid, stream, __VA_ARGS__);                          \
        else SFM_DISPATCH_NT(dtype, KERNEL, 16, grid, stream, __VA_ARGS__);                                         \
    } while (0)
#define SFM_DISPATCH_NT(dtype, KERNEL, NT, grid, stream, ...)                                                       \
    do {                                                                                                            \
        if ((dtype) == SFM_BF16) hipLaunchKernelGGL((KERNEL<BF16, NT>), grid, dim3(256), 0, stream, __VA_ARGS__);   \
        else if ((dtype) == SFM_F16) hipLaunchKernelGGL((KERNEL<F16, NT>), grid, dim3(256), 0, stream, __VA_ARGS__); \
        else hipLaunchKernelGGL((KERNEL<float, NT>), grid, dim3(256), 0, stream, __VA_ARGS__);                      \
    } while (0)

int launch_ln_modulate(int dtype, int64_t rows, int C, float eps, const void* x, int64_t xs, void* y, int64_t ys,
                       const void* scale, const void* shift, int64_t ms, int rows_per_frame, const void* weight,
                       const void* bias, hipStream_t stream) {
    SFM_DISPATCH_ROWS(dtype, ln_modulate_kernel, C, rows, stream, x, xs, y, ys, C, eps, scale, shift, ms, rows_per_frame,
                      weight, bias, rows);
    return finish();
}

int launch_gate_residual_ln(int dtype, int64_t rows, int C, float eps, void* x, int64_t xs, const void* y, int64_t ys,
                            const void* gate, int64_t gms, int g_rows_per_frame, void* out, int64_t os, const void* scale,
                            const void* shift, int64_t ms, int rows_per_frame, const void* weight, const void* bias,
                            hipStream_t stream) {
    SFM_DISPATCH_ROWS(dtype, gate_residual_ln_kernel, C, rows, stream, x, xs, y, ys, gate, gms, g_rows_per_frame, out, os, C, eps,
                      scale, shift, ms, rows_per_frame, weight, bias, rows);
    return finish();
}

int launch_gate_residual(int dtype, int64_t rows, int C, void* x, int64_t xs, const void* y, int64_t ys,
                         const void* gate, int64_t ms, int rows_per_frame, hipStream_t stream) {
    SFM_DISPATCH(dtype, gate_residual_kernel, dim3((unsigned)rows), stream, x, xs, y, ys, C, gate, ms, rows_per_frame);
    return finish();
}

int launch_rms_norm(int dtype, int64_t rows, int C, float eps, const void* x, int64_t xs, void* y, int64_t ys,
                    const void* weight, hipStream_t stream) {
    SFM_DISPATCH_ROWS(dtype, rms_norm_kernel, C, rows, stream, x, xs, y, ys, C, eps, weight, rows);
    return finish();
}

}  // namespace sfm
