// Monarch attention forward, shape-generic fp32 path (any dtype in {bf16, fp16, fp32}, any head_dim
// and block shape that fits LDS).  Same two steps and the same workspace layout as the MFMA path,
// with Kbar / Y kept in float.  This is the path fp32 tensors take, and the one block shapes
// outside the MFMA kernels' limits fall back to; it computes exactly
//   wan/modules/monarch_attn.py:1801-1830 (monarch_attn_ref_op)
// with all arithmetic in fp32.

#include "sfm_common.hpp"

namespace sfm {

template <typename T> struct Ld;
template <> struct Ld<float> {
    static __device__ __forceinline__ float get(const void* p, int64_t i) { return ((const float*)p)[i]; }
    static __device__ __forceinline__ void put(void* p, int64_t i, float x) { ((float*)p)[i] = x; }
};
template <> struct Ld<BF16> {
    static __device__ __forceinline__ float get(const void* p, int64_t i) { return BF16::to_float(((const uint16_t*)p)[i]); }
    static __device__ __forceinline__ void put(void* p, int64_t i, float x) { ((uint16_t*)p)[i] = BF16::from_float(x); }
};
template <> struct Ld<F16> {
    static __device__ __forceinline__ float get(const void* p, int64_t i) { return F16::to_float(((const uint16_t*)p)[i]); }
    static __device__ __forceinline__ void put(void* p, int64_t i, float x) { ((uint16_t*)p)[i] = F16::from_float(x); }
};

// workgroup = (block row k, kv block-frame f, unit x query block-frame a); 256 threads
template <typename T>
__global__ __launch_bounds__(256) void monarch_generic_step1(MonarchArgs p) {
    extern __shared__ float sm[];
    const int D = p.D, b2 = p.b2, DP = D + 1;
    float* Ks = sm;                    // [b2][D+1]
    float* Vs = Ks + b2 * DP;          // [b2][D+1]
    float* qs = Vs + b2 * DP;          // [D]
    float* zs = qs + D;                // [b2]

    const int k = blockIdx.x, f = blockIdx.y;
    const int ul = blockIdx.z / p.na, a = blockIdx.z % p.na;
    if (p.causal && (a / p.causal) < (f / p.causal)) return;
    const int unit = p.unit0 + ul;
    const int b = unit / p.H, h = unit % p.H;
    const int tid = threadIdx.x, nt = blockDim.x;

    const int64_t krow0 = p.kmap.row(f, k);
    for (int e = tid; e < b2 * D; e += nt) {
        int l = e / D, d = e % D;
        Ks[l * DP + d] = Ld<T>::get(p.k, (int64_t)b * p.ks[0] + (krow0 + l) * p.ks[1] + (int64_t)h * p.ks[2] + d);
        Vs[l * DP + d] = Ld<T>::get(p.v, (int64_t)b * p.vs[0] + (krow0 + l) * p.vs[1] + (int64_t)h * p.vs[2] + d);
    }
    const int64_t qrow0 = p.qmap.row(a, k);
    const float sc2 = p.scale * kLog2e;
    float* kbar = (float*)p.kbar;
    float* yw = (float*)p.y;

    for (int j = 0; j < b2; ++j) {
        __syncthreads();
        for (int d = tid; d < D; d += nt)
            qs[d] = Ld<T>::get(p.q, (int64_t)b * p.qs[0] + (qrow0 + j) * p.qs[1] + (int64_t)h * p.qs[2] + d);
        __syncthreads();
        for (int l = tid; l < b2; l += nt) {
            float acc = 0.f;
            for (int d = 0; d < D; ++d) acc += qs[d] * Ks[l * DP + d];
            zs[l] = acc * sc2;
        }
        __syncthreads();
        float mx = -INFINITY;
        for (int l = 0; l < b2; ++l) mx = fmaxf(mx, zs[l]);
        float sum = 0.f, ent = 0.f;
        for (int l = 0; l < b2; ++l) {
            float e = exp2f(zs[l] - mx);
            sum += e;
            ent += e * zs[l];
        }
        const float inv = 1.f / sum;
        const int64_t blk = (int64_t)ul * p.ws_unit + (int64_t)(a * b2 + j) * p.ws_aj + (int64_t)(f * p.b1 + k) * p.ws_row;
        if (tid == 0) p.cl[blk] = ent * inv - (mx + log2f(sum));
        for (int d = tid; d < D; d += nt) {
            float ak = 0.f, av = 0.f;
            for (int l = 0; l < b2; ++l) {
                float r = exp2f(zs[l] - mx) * inv;
                ak += r * Ks[l * DP + d];
                av += r * Vs[l * DP + d];
            }
            kbar[blk * D + d] = ak;
            yw[blk * D + d] = av;
        }
    }
}

// workgroup = (unit, a, j); loops over the block rows i; 256 threads
template <typename T>
__global__ __launch_bounds__(256) void monarch_generic_step2(MonarchArgs p) {
    extern __shared__ float sm[];
    const int D = p.D, b2 = p.b2;
    const int a = blockIdx.x / b2, j = blockIdx.x % b2;
    const int ul = blockIdx.y;
    const int unit = p.unit0 + ul;
    const int b = unit / p.H, h = unit % p.H;
    const int tid = threadIdx.x, nt = blockDim.x;
    const int f_lim = p.causal ? min(p.nf, (a / p.causal + 1) * p.causal) : p.nf;
    const int R = f_lim * p.b1;

    float* qs = sm;            // [D]
    float* zs = qs + D;        // [R]
    float* red = zs + R;       // [nt]

    const int64_t blk = (int64_t)ul * p.ws_unit + (int64_t)(a * b2 + j) * p.ws_aj;
    const int64_t rs = p.ws_row;
    const float* kbar = (const float*)p.kbar + blk * D;
    const float* yw = (const float*)p.y + blk * D;
    const float* cl = p.cl + blk;
    const float sc2 = p.scale * kLog2e;

    for (int i = 0; i < p.b1; ++i) {
        const int64_t tok = p.qmap.row(a, i) + j;
        __syncthreads();
        for (int d = tid; d < D; d += nt)
            qs[d] = Ld<T>::get(p.q, (int64_t)b * p.qs[0] + tok * p.qs[1] + (int64_t)h * p.qs[2] + d);
        __syncthreads();
        float mx = -INFINITY;
        for (int r = tid; r < R; r += nt) {
            float acc = 0.f;
            const float* row = kbar + (int64_t)r * rs * D;
            for (int d = 0; d < D; ++d) acc += qs[d] * row[d];
            float z = acc * sc2 - cl[r * rs];
            zs[r] = z;
            mx = fmaxf(mx, z);
        }
        red[tid] = mx;
        __syncthreads();
        for (int s = nt / 2; s > 0; s >>= 1) {
            if (tid < s) red[tid] = fmaxf(red[tid], red[tid + s]);
            __syncthreads();
        }
        mx = red[0];
        __syncthreads();
        float sum = 0.f;
        for (int r = tid; r < R; r += nt) {
            float e = exp2f(zs[r] - mx);
            zs[r] = e;
            sum += e;
        }
        red[tid] = sum;
        __syncthreads();
        for (int s = nt / 2; s > 0; s >>= 1) {
            if (tid < s) red[tid] += red[tid + s];
            __syncthreads();
        }
        const float inv = 1.f / red[0];
        for (int d = tid; d < D; d += nt) {
            float acc = 0.f;
            for (int r = 0; r < R; ++r) acc += zs[r] * yw[(int64_t)r * rs * D + d];
            Ld<T>::put(p.out, (int64_t)b * p.os[0] + tok * p.os[1] + (int64_t)h * p.os[2] + d, acc * inv);
        }
    }
}

static size_t generic_lds1_bytes(const MonarchArgs& a) { return sizeof(float) * ((size_t)2 * a.b2 * (a.D + 1) + a.D + a.b2); }

// ------------------------------------------------------------------------------------------------
// Iterated refinement (num_iters > 1): wan/modules/monarch_attn.py:1705-1751 (monarch_attn_slow), which the
// reference runs as pure-torch einsums.  Each pass recomputes the right factor from per-block query
// representatives rep[a,f,k,j,:] = sum_i L[a,i,j,(f,k)] Q s^1/2 with weight w = sum_i L (first pass:
// rep = Q[a,k,j] s^1/2, w = 1) using logits <rep, K s^1/2> * min(1/(w + 1e-6), 1e4), then the left factor.
// fp32 throughout; Kbar here is R (K s^1/2), cl = sum_l R ln R (natural log), rep / w live in the scratch.
// ------------------------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void monarch_iter_step1(MonarchArgs p, int first, int last) {
    extern __shared__ float sm[];
    const int D = p.D, b2 = p.b2, DP = D + 1;
    float* Ks = sm;                    // [b2][D+1]  K * sqrt(s)
    float* Vs = Ks + b2 * DP;          // [b2][D+1]
    float* qs = Vs + b2 * DP;          // [D]        representative
    float* zs = qs + D;                // [b2]
    const int k = blockIdx.x, f = blockIdx.y;
    const int ul = blockIdx.z / p.na, a = blockIdx.z % p.na;
    const int unit = p.unit0 + ul;
    const int b = unit / p.H, h = unit % p.H;
    const int tid = threadIdx.x, nt = blockDim.x;
    const float rs = sqrtf(p.scale);

    const int64_t krow0 = p.kmap.row(f, k);
    for (int e = tid; e < b2 * D; e += nt) {
        int l = e / D, d = e % D;
        Ks[l * DP + d] = rs * Ld<T>::get(p.k, (int64_t)b * p.ks[0] + (krow0 + l) * p.ks[1] + (int64_t)h * p.ks[2] + d);
        Vs[l * DP + d] = last ? Ld<T>::get(p.v, (int64_t)b * p.vs[0] + (krow0 + l) * p.vs[1] + (int64_t)h * p.vs[2] + d) : 0.f;
    }
    const int64_t qrow0 = p.qmap.row(a, k);
    float* kbar = (float*)p.kbar;
    float* yw = (float*)p.y;
    const float* rep = (const float*)p.rep;

    for (int j = 0; j < b2; ++j) {
        const int64_t blk = (int64_t)ul * p.ws_unit + (int64_t)(a * b2 + j) * p.ws_aj + (int64_t)(f * p.b1 + k) * p.ws_row;
        __syncthreads();
        for (int d = tid; d < D; d += nt)
            qs[d] = first ? rs * Ld<T>::get(p.q, (int64_t)b * p.qs[0] + (qrow0 + j) * p.qs[1] + (int64_t)h * p.qs[2] + d)
                          : rep[blk * D + d];
        const float wsc = first ? 1.0f / (1.0f + 1e-6f) : fminf(1.0f / (p.wgt[blk] + 1e-6f), 1e4f);
        __syncthreads();
        for (int l = tid; l < b2; l += nt) {
            float acc = 0.f;
            for (int d = 0; d < D; ++d) acc += qs[d] * Ks[l * DP + d];
            zs[l] = acc * wsc;
        }
        __syncthreads();
        float mx = -INFINITY;
        for (int l = 0; l < b2; ++l) mx = fmaxf(mx, zs[l]);
        float sum = 0.f, ent = 0.f;
        for (int l = 0; l < b2; ++l) {
            float e = expf(zs[l] - mx);
            sum += e;
            ent += e * zs[l];
        }
        const float inv = 1.f / sum;
        if (tid == 0) p.cl[blk] = ent * inv - (mx + logf(sum));
        for (int d = tid; d < D; d += nt) {
            float ak = 0.f, av = 0.f;
            for (int l = 0; l < b2; ++l) {
                float r = expf(zs[l] - mx) * inv;
                ak += r * Ks[l * DP + d];
                av += r * Vs[l * DP + d];
            }
            kbar[blk * D + d] = ak;
            if (last) yw[blk * D + d] = av;
        }
    }
}

constexpr int kIterRows = 32;   // query rows of one (a, j) column held in registers / LDS at a time

// workgroup = (unit, a, j): left factor L[i, r] over all rows r = (f, k); then either the new representatives
// (rep[r,:] = sum_i L[i,r] q_i, w[r] = sum_i L[i,r]) or, in the last pass, the output rows sum_r L[i,r] Y[r,:].
// Query rows are taken `ic` at a time (rows of L are independent; rep and w accumulate over the chunks).
template <typename T>
__global__ __launch_bounds__(256) void monarch_iter_step2(MonarchArgs p, int last, int ic) {
    extern __shared__ float sm[];
    const int D = p.D, b2 = p.b2, b1 = p.b1, DP = D + 1;
    const int a = blockIdx.x / b2, j = blockIdx.x % b2;
    const int ul = blockIdx.y;
    const int unit = p.unit0 + ul;
    const int b = unit / p.H, h = unit % p.H;
    const int tid = threadIdx.x, nt = blockDim.x;
    const int R = p.nf * b1;
    const float rs = sqrtf(p.scale);
    float* qs = sm;                    // [ic][D+1]   Q[a, i, j, :] * sqrt(s)
    float* S = qs + ic * DP;           // [ic][R]     logits, then L
    float* red = S + (size_t)ic * R;   // [2 * ic]    row max, 1 / row sum

    const int64_t blk = (int64_t)ul * p.ws_unit + (int64_t)(a * b2 + j) * p.ws_aj;
    const int64_t rsd = p.ws_row;
    const float* kbar = (const float*)p.kbar + blk * D;
    const float* yw = (const float*)p.y + blk * D;
    const float* cl = p.cl + blk;
    float* rep = (float*)p.rep + blk * D;
    float* wgt = p.wgt + blk;

    for (int i0 = 0; i0 < b1; i0 += ic) {
        const int ni = b1 - i0 < ic ? b1 - i0 : ic;
        __syncthreads();
        for (int e = tid; e < ni * D; e += nt) {
            int i = e / D, d = e % D;
            qs[i * DP + d] =
                rs * Ld<T>::get(p.q, (int64_t)b * p.qs[0] + (p.qmap.row(a, i0 + i) + j) * p.qs[1] + (int64_t)h * p.qs[2] + d);
        }
        __syncthreads();
        for (int r = tid; r < R; r += nt) {            // logits of row r against the chunk's query rows
            float acc[kIterRows];
#pragma unroll
            for (int i = 0; i < kIterRows; ++i) acc[i] = 0.f;
            const float* row = kbar + (int64_t)r * rsd * D;
            for (int d = 0; d < D; ++d) {
                const float kv = row[d];
#pragma unroll
                for (int i = 0; i < kIterRows; ++i)
                    if (i < ni) acc[i] += qs[i * DP + d] * kv;
            }
            const float c = cl[r * rsd];
#pragma unroll
            for (int i = 0; i < kIterRows; ++i)
                if (i < ni) S[(size_t)i * R + r] = acc[i] - c;
        }
        __syncthreads();
        for (int i = tid >> 6; i < ni; i += nt >> 6) {  // one wave per query row: max and sum over r
            float mx = -INFINITY;
            for (int r = tid & 63; r < R; r += 64) mx = fmaxf(mx, S[(size_t)i * R + r]);
            for (int o = 32; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o));
            float sum = 0.f;
            for (int r = tid & 63; r < R; r += 64) sum += expf(S[(size_t)i * R + r] - mx);
            for (int o = 32; o > 0; o >>= 1) sum += __shfl_xor(sum, o);
            if ((tid & 63) == 0) {
                red[2 * i] = mx;
                red[2 * i + 1] = 1.f / sum;
            }
        }
        __syncthreads();
        for (int e = tid; e < ni * R; e += nt) {
            int i = e / R;
            S[e] = expf(S[e] - red[2 * i]) * red[2 * i + 1];
        }
        __syncthreads();
        if (!last) {
            for (int r = tid; r < R; r += nt) {
                float w = i0 ? wgt[r * rsd] : 0.f;
                for (int i = 0; i < ni; ++i) w += S[(size_t)i * R + r];
                wgt[r * rsd] = w;
                float* dst = rep + (int64_t)r * rsd * D;
                for (int d = 0; d < D; ++d) {
                    float acc = i0 ? dst[d] : 0.f;
                    for (int i = 0; i < ni; ++i) acc += S[(size_t)i * R + r] * qs[i * DP + d];
                    dst[d] = acc;
                }
            }
        } else {
            for (int d = tid; d < D; d += nt) {
                float acc[kIterRows];
#pragma unroll
                for (int i = 0; i < kIterRows; ++i) acc[i] = 0.f;
                for (int r = 0; r < R; ++r) {
                    const float yv = yw[(int64_t)r * rsd * D + d];
#pragma unroll
                    for (int i = 0; i < kIterRows; ++i)
                        if (i < ni) acc[i] += S[(size_t)i * R + r] * yv;
                }
#pragma unroll
                for (int i = 0; i < kIterRows; ++i)
                    if (i < ni)
                        Ld<T>::put(p.out,
                                   (int64_t)b * p.os[0] + (p.qmap.row(a, i0 + i) + j) * p.os[1] + (int64_t)h * p.os[2] + d,
                                   acc[i]);
            }
        }
    }
}

// query rows per chunk: as many as fit 128 KB of LDS next to the chunk's logits, at most kIterRows
static int iter_rows(const MonarchArgs& a) {
    const size_t per_row = sizeof(float) * ((size_t)(a.D + 1) + (size_t)a.nf * a.b1 + 2);
    size_t ic = (128 * 1024) / per_row;
    if (ic > (size_t)kIterRows) ic = kIterRows;
    if (ic > (size_t)a.b1) ic = a.b1;
    return (int)ic;
}

static size_t iter_lds2(const MonarchArgs& a) {
    return sizeof(float) * (size_t)iter_rows(a) * ((size_t)(a.D + 1) + (size_t)a.nf * a.b1 + 2);
}

bool monarch_iter_supported(const MonarchArgs& a) { return iter_rows(a) >= 1 && generic_lds1_bytes(a) <= 160 * 1024; }

template <typename T>
static int launch_iter_t(const MonarchArgs& a, int nunits, int num_iters, hipStream_t stream) {
    const size_t l1 = generic_lds1_bytes(a), l2 = iter_lds2(a);
    hipError_t err = hipSuccess;
    if (l1 > 64 * 1024)
        err = hipFuncSetAttribute((const void*)monarch_iter_step1<T>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)l1);
    if (err == hipSuccess && l2 > 64 * 1024)
        err = hipFuncSetAttribute((const void*)monarch_iter_step2<T>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)l2);
    if (err != hipSuccess) {
        set_error("hipFuncSetAttribute failed: %s", hipGetErrorString(err));
        return SFM_ERR_HIP;
    }
    for (int it = 0; it < num_iters; ++it) {
        const int last = it + 1 == num_iters;
        hipLaunchKernelGGL((monarch_iter_step1<T>), dim3(a.b1, a.nf, nunits * a.na), dim3(256), l1, stream, a, it == 0, last);
        hipLaunchKernelGGL((monarch_iter_step2<T>), dim3(a.na * a.b2, nunits), dim3(256), l2, stream, a, last, iter_rows(a));
    }
    err = hipGetLastError();
    if (err != hipSuccess) {
        set_error("hip launch failed: %s", hipGetErrorString(err));
        return SFM_ERR_HIP;
    }
    return SFM_OK;
}

int launch_monarch_iter(const MonarchArgs& a, int dtype, int nunits, int num_iters, hipStream_t stream) {
    if (!monarch_iter_supported(a)) {
        set_error("iterated Monarch: block shape b1=%d, b2=%d, rows=%d, D=%d exceeds the limits of this path", a.b1, a.b2,
                  a.nf * a.b1, a.D);
        return SFM_ERR_UNSUPPORTED;
    }
    if (dtype == SFM_F32) return launch_iter_t<float>(a, nunits, num_iters, stream);
    if (dtype == SFM_BF16) return launch_iter_t<BF16>(a, nunits, num_iters, stream);
    return launch_iter_t<F16>(a, nunits, num_iters, stream);
}

// ------------------------------------------------------------------------------------------------
// Backward of the one-iteration forward (replaces _z_bwd_preprocess, _z_bwd, _al_cl_y_bwd,
// wan/modules/monarch_attn.py:852-886, 1034-1222, 403-596, and the orchestration :1326-1470, 1566-1693), fp32.
// With S1 = s q.k, R = softmax_l S1, Kbar = R K, Y = R V, c = sum_l R ln R, S2 = s q.Kbar - c, L = softmax_(f,k) S2,
// O = L Y and a given dO:
//   dLm[i,r] = dO_i . Y_r            dS2 = L (dLm - sum_r L dLm)
//   dY_r = sum_i L[i,r] dO_i         dKbar_r = s sum_i dS2[i,r] q_i       dc_r = - sum_i dS2[i,r]
//   dQ(a,i,j) = s sum_r dS2[i,r] Kbar_r                                              (left factor)
//   dR_l = dKbar . K_l + dY . V_l + dc (ln R_l + 1)        dS1 = R (dR - sum_l R dR)
//   dQ(a,k,j) += s sum_f sum_l dS1_l K_l     dK_l += R_l dKbar + s dS1_l q     dV_l += R_l dY   (right factor)
// Three launches per pass: the forward's step 1 (Kbar, Y, c into the scratch), the left-factor kernel
// (workgroup = (unit, a, j); writes dKbar, dY, dc to the scratch and its part of dQ), the right-factor
// kernel (workgroup = (unit, k), which owns the rows dQ[a, k, :] and the tiles dK/dV[f, k, :], so that
// nothing needs an atomic).  The "+ 1" drops out of the softmax backward.
// ------------------------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void monarch_bwd_left(MonarchBwdArgs g, int ic) {
    extern __shared__ float sm[];
    const MonarchArgs& p = g.p;
    const int D = p.D, b2 = p.b2, b1 = p.b1, DP = D + 1;
    const int a = blockIdx.x / b2, j = blockIdx.x % b2;
    const int ul = blockIdx.y;
    const int unit = p.unit0 + ul;
    const int b = unit / p.H, h = unit % p.H;
    const int tid = threadIdx.x, nt = blockDim.x;
    const int f_lim = p.causal ? min(p.nf, (a / p.causal + 1) * p.causal) : p.nf;
    const int R = f_lim * b1;
    const int RP = p.nf * b1;          // row pitch of the LDS arrays
    const float sc2 = p.scale * kLog2e;
    float* qs = sm;                    // [ic][D+1]   q_i
    float* dos = qs + ic * DP;         // [ic][D+1]   dO_i
    float* S = dos + ic * DP;          // [ic][RP]    logits (log2 units), then L
    float* G = S + (size_t)ic * RP;    // [ic][RP]    dLm, then dS2

    const int64_t blk = (int64_t)ul * p.ws_unit + (int64_t)(a * b2 + j) * p.ws_aj;
    const int64_t rsd = p.ws_row;
    const float* kbar = (const float*)p.kbar + blk * D;
    const float* yw = (const float*)p.y + blk * D;
    const float* cl = p.cl + blk;
    float* dkbar = g.dkbar + blk * D;
    float* dy = g.dy + blk * D;
    float* dcl = g.dcl + blk;

    for (int i0 = 0; i0 < b1; i0 += ic) {
        const int ni = b1 - i0 < ic ? b1 - i0 : ic;
        __syncthreads();
        for (int e = tid; e < ni * D; e += nt) {
            const int i = e / D, d = e % D;
            const int64_t tok = p.qmap.row(a, i0 + i) + j;
            qs[i * DP + d] = Ld<T>::get(p.q, (int64_t)b * p.qs[0] + tok * p.qs[1] + (int64_t)h * p.qs[2] + d);
            dos[i * DP + d] = Ld<T>::get(g.dout, (int64_t)b * g.dos[0] + tok * g.dos[1] + (int64_t)h * g.dos[2] + d);
        }
        __syncthreads();
        for (int r = tid; r < R; r += nt) {
            float as[kIterRows], al[kIterRows];
#pragma unroll
            for (int i = 0; i < kIterRows; ++i) as[i] = al[i] = 0.f;
            const float* krow = kbar + (int64_t)r * rsd * D;
            const float* yrow = yw + (int64_t)r * rsd * D;
            for (int d = 0; d < D; ++d) {
                const float kv = krow[d], yv = yrow[d];
#pragma unroll
                for (int i = 0; i < kIterRows; ++i)
                    if (i < ni) {
                        as[i] += qs[i * DP + d] * kv;
                        al[i] += dos[i * DP + d] * yv;
                    }
            }
            const float c = cl[r * rsd];
#pragma unroll
            for (int i = 0; i < kIterRows; ++i)
                if (i < ni) {
                    S[(size_t)i * RP + r] = as[i] * sc2 - c;
                    G[(size_t)i * RP + r] = al[i];
                }
        }
        __syncthreads();
        for (int i = tid >> 6; i < ni; i += nt >> 6) {      // one wave per query row
            float* Si = S + (size_t)i * RP;
            float* Gi = G + (size_t)i * RP;
            float mx = -INFINITY;
            for (int r = tid & 63; r < R; r += 64) mx = fmaxf(mx, Si[r]);
            for (int o = 32; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o));
            float sum = 0.f;
            for (int r = tid & 63; r < R; r += 64) sum += exp2f(Si[r] - mx);
            for (int o = 32; o > 0; o >>= 1) sum += __shfl_xor(sum, o);
            const float inv = 1.f / sum;
            float dot = 0.f;
            for (int r = tid & 63; r < R; r += 64) {
                const float l = exp2f(Si[r] - mx) * inv;
                Si[r] = l;
                dot += l * Gi[r];
            }
            for (int o = 32; o > 0; o >>= 1) dot += __shfl_xor(dot, o);
            for (int r = tid & 63; r < R; r += 64) Gi[r] = Si[r] * (Gi[r] - dot);
        }
        __syncthreads();
        for (int e = tid; e < R * D; e += nt) {
            const int r = e / D, d = e % D;
            float ay = 0.f, ak = 0.f;
            for (int i = 0; i < ni; ++i) {
                ay += S[(size_t)i * RP + r] * dos[i * DP + d];
                ak += G[(size_t)i * RP + r] * qs[i * DP + d];
            }
            const int64_t o = (int64_t)r * rsd * D + d;
            if (i0 == 0) {
                dy[o] = ay;
                dkbar[o] = ak * p.scale;
            } else {
                dy[o] += ay;
                dkbar[o] += ak * p.scale;
            }
        }
        for (int r = tid; r < R; r += nt) {
            float sds = 0.f;
            for (int i = 0; i < ni; ++i) sds += G[(size_t)i * RP + r];
            if (i0 == 0) dcl[r * rsd] = -sds;
            else dcl[r * rsd] -= sds;
        }
        for (int e = tid; e < ni * D; e += nt) {
            const int i = e / D, d = e % D;
            float acc = 0.f;
            for (int r = 0; r < R; ++r) acc += G[(size_t)i * RP + r] * kbar[(int64_t)r * rsd * D + d];
            const int64_t tok = p.qmap.row(a, i0 + i) + j;
            g.dq[(int64_t)b * g.dqs[0] + tok * g.dqs[1] + (int64_t)h * g.dqs[2] + d] = acc * p.scale;
        }
    }
}

template <typename T>
__global__ __launch_bounds__(256) void monarch_bwd_right(MonarchBwdArgs g) {
    extern __shared__ float sm[];
    const MonarchArgs& p = g.p;
    const int D = p.D, b2 = p.b2, DP = D + 1;
    float* Ks = sm;                    // [b2][D+1]
    float* Vs = Ks + b2 * DP;          // [b2][D+1]
    float* dKs = Vs + b2 * DP;         // [b2][D+1]
    float* dVs = dKs + b2 * DP;        // [b2][D+1]
    float* qs = dVs + b2 * DP;         // [D]
    float* dkb = qs + D;               // [D]
    float* dyv = dkb + D;              // [D]
    float* zs = dyv + D;               // [b2]
    float* Rr = zs + b2;               // [b2]
    float* dR = Rr + b2;               // [b2]

    const int k = blockIdx.x, ul = blockIdx.y;
    const int unit = p.unit0 + ul;
    const int b = unit / p.H, h = unit % p.H;
    const int tid = threadIdx.x, nt = blockDim.x;
    const float sc2 = p.scale * kLog2e;
    constexpr float kLn2 = 0.6931471805599453f;

    for (int f = 0; f < p.nf; ++f) {
        const int64_t krow0 = p.kmap.row(f, k);
        __syncthreads();
        for (int e = tid; e < b2 * D; e += nt) {
            const int l = e / D, d = e % D;
            Ks[l * DP + d] = Ld<T>::get(p.k, (int64_t)b * p.ks[0] + (krow0 + l) * p.ks[1] + (int64_t)h * p.ks[2] + d);
            Vs[l * DP + d] = Ld<T>::get(p.v, (int64_t)b * p.vs[0] + (krow0 + l) * p.vs[1] + (int64_t)h * p.vs[2] + d);
            dKs[l * DP + d] = 0.f;
            dVs[l * DP + d] = 0.f;
        }
        for (int a = 0; a < p.na; ++a) {
            if (p.causal && (a / p.causal) < (f / p.causal)) continue;
            const int64_t qrow0 = p.qmap.row(a, k);
            for (int j = 0; j < b2; ++j) {
                const int64_t blk = (int64_t)ul * p.ws_unit + (int64_t)(a * b2 + j) * p.ws_aj + (int64_t)(f * p.b1 + k) * p.ws_row;
                __syncthreads();
                for (int d = tid; d < D; d += nt) {
                    qs[d] = Ld<T>::get(p.q, (int64_t)b * p.qs[0] + (qrow0 + j) * p.qs[1] + (int64_t)h * p.qs[2] + d);
                    dkb[d] = g.dkbar[blk * D + d];
                    dyv[d] = g.dy[blk * D + d];
                }
                __syncthreads();
                for (int l = tid; l < b2; l += nt) {
                    float acc = 0.f;
                    for (int d = 0; d < D; ++d) acc += qs[d] * Ks[l * DP + d];
                    zs[l] = acc * sc2;
                }
                __syncthreads();
                float mx = -INFINITY;
                for (int l = 0; l < b2; ++l) mx = fmaxf(mx, zs[l]);
                float sum = 0.f;
                for (int l = 0; l < b2; ++l) sum += exp2f(zs[l] - mx);
                const float lse2 = mx + log2f(sum);
                const float dc = g.dcl[blk];
                for (int l = tid; l < b2; l += nt) {
                    const float lr2 = zs[l] - lse2;              // log2 R_l
                    float acc = 0.f;
                    for (int d = 0; d < D; ++d) acc += dkb[d] * Ks[l * DP + d] + dyv[d] * Vs[l * DP + d];
                    Rr[l] = exp2f(lr2);
                    dR[l] = acc + dc * (lr2 * kLn2);
                }
                __syncthreads();
                float dot = 0.f;
                for (int l = 0; l < b2; ++l) dot += Rr[l] * dR[l];
                __syncthreads();
                for (int l = tid; l < b2; l += nt) dR[l] = Rr[l] * (dR[l] - dot);      // dS1
                __syncthreads();
                for (int e = tid; e < b2 * D; e += nt) {
                    const int l = e / D, d = e % D;
                    dKs[l * DP + d] += Rr[l] * dkb[d] + p.scale * dR[l] * qs[d];
                    dVs[l * DP + d] += Rr[l] * dyv[d];
                }
                for (int d = tid; d < D; d += nt) {
                    float acc = 0.f;
                    for (int l = 0; l < b2; ++l) acc += dR[l] * Ks[l * DP + d];
                    g.dq[(int64_t)b * g.dqs[0] + (qrow0 + j) * g.dqs[1] + (int64_t)h * g.dqs[2] + d] += acc * p.scale;
                }
            }
        }
        __syncthreads();
        if (f >= g.kv_f0 && f < g.kv_f1) {
            for (int e = tid; e < b2 * D; e += nt) {
                const int l = e / D, d = e % D;
                const int64_t o = (int64_t)b * g.dks[0] + (krow0 + l - g.dk_row0) * g.dks[1] + (int64_t)h * g.dks[2] + d;
                Ld<T>::put(g.dk, o, dKs[l * DP + d]);
                Ld<T>::put(g.dv, o, dVs[l * DP + d]);
            }
        }
    }
}

static int bwd_rows(const MonarchArgs& a) {
    const size_t per_row = sizeof(float) * (2 * (size_t)(a.D + 1) + 2 * (size_t)a.nf * a.b1);
    size_t ic = (128 * 1024) / per_row;
    if (ic > (size_t)kIterRows) ic = kIterRows;
    if (ic > (size_t)a.b1) ic = a.b1;
    return (int)ic;
}
static size_t bwd_lds_left(const MonarchArgs& a) {
    return sizeof(float) * (size_t)bwd_rows(a) * (2 * (size_t)(a.D + 1) + 2 * (size_t)a.nf * a.b1);
}
static size_t bwd_lds_right(const MonarchArgs& a) {
    return sizeof(float) * (4 * (size_t)a.b2 * (a.D + 1) + 3 * (size_t)a.D + 3 * (size_t)a.b2);
}

template <typename T>
static int launch_bwd_t(const MonarchBwdArgs& g, int nunits, hipStream_t stream) {
    const MonarchArgs& a = g.p;
    const size_t l1 = generic_lds1_bytes(a), ll = bwd_lds_left(a), lr = bwd_lds_right(a);
    hipError_t err = hipSuccess;
    if (l1 > 64 * 1024)
        err = hipFuncSetAttribute((const void*)monarch_generic_step1<T>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)l1);
    if (err == hipSuccess && ll > 64 * 1024)
        err = hipFuncSetAttribute((const void*)monarch_bwd_left<T>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)ll);
    if (err == hipSuccess && lr > 64 * 1024)
        err = hipFuncSetAttribute((const void*)monarch_bwd_right<T>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lr);
    if (err != hipSuccess) {
        set_error("hipFuncSetAttribute failed: %s", hipGetErrorString(err));
        return SFM_ERR_HIP;
    }
    hipLaunchKernelGGL((monarch_generic_step1<T>), dim3(a.b1, a.nf, nunits * a.na), dim3(256), l1, stream, a);
    hipLaunchKernelGGL((monarch_bwd_left<T>), dim3(a.na * a.b2, nunits), dim3(256), ll, stream, g, bwd_rows(a));
    hipLaunchKernelGGL((monarch_bwd_right<T>), dim3(a.b1, nunits), dim3(256), lr, stream, g);
    err = hipGetLastError();
    if (err != hipSuccess) {
        set_error("hip launch failed: %s", hipGetErrorString(err));
        return SFM_ERR_HIP;
    }
    return SFM_OK;
}

int launch_monarch_bwd(const MonarchBwdArgs& g, int dtype, int nunits, hipStream_t stream) {
    const MonarchArgs& a = g.p;
    if (bwd_rows(a) < 1 || generic_lds1_bytes(a) > 160 * 1024 || bwd_lds_right(a) > 160 * 1024) {
        set_error("Monarch backward: block shape b1=%d, b2=%d, rows=%d, D=%d exceeds the LDS budget of this path", a.b1, a.b2,
                  a.nf * a.b1, a.D);
        return SFM_ERR_UNSUPPORTED;
    }
    if (dtype == SFM_F32) return launch_bwd_t<float>(g, nunits, stream);
    if (dtype == SFM_BF16) return launch_bwd_t<BF16>(g, nunits, stream);
    return launch_bwd_t<F16>(g, nunits, stream);
}

static size_t generic_lds2(const MonarchArgs& a) { return sizeof(float) * ((size_t)a.D + (size_t)a.nf * a.b1 + 256); }

bool monarch_generic_supported(const MonarchArgs& a) {
    return generic_lds1_bytes(a) <= 160 * 1024 && generic_lds2(a) <= 160 * 1024;
}

template <typename T>
static int launch_generic_t(const MonarchArgs& a, int nunits, hipStream_t stream, const StepEvents* ev) {
    const size_t l1 = generic_lds1_bytes(a), l2 = generic_lds2(a);
    hipError_t err = hipSuccess;
    if (l1 > 64 * 1024)
        err = hipFuncSetAttribute((const void*)monarch_generic_step1<T>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)l1);
    if (err == hipSuccess && l2 > 64 * 1024)
        err = hipFuncSetAttribute((const void*)monarch_generic_step2<T>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)l2);
    if (err != hipSuccess) {
        set_error("hipFuncSetAttribute failed: %s", hipGetErrorString(err));
        return SFM_ERR_HIP;
    }
    if (ev) (void)hipEventRecord(ev->ev[0], stream);
    hipLaunchKernelGGL((monarch_generic_step1<T>), dim3(a.b1, a.nf, nunits * a.na), dim3(256), l1, stream, a);
    if (ev) (void)hipEventRecord(ev->ev[1], stream);
    hipLaunchKernelGGL((monarch_generic_step2<T>), dim3(a.na * a.b2, nunits), dim3(256), l2, stream, a);
    if (ev) (void)hipEventRecord(ev->ev[2], stream);
    err = hipGetLastError();
    if (err != hipSuccess) {
        set_error("hip launch failed: %s", hipGetErrorString(err));
        return SFM_ERR_HIP;
    }
    return SFM_OK;
}

int launch_monarch_generic(const MonarchArgs& a, int dtype, int nunits, hipStream_t stream, const StepEvents* ev) {
    if (!monarch_generic_supported(a)) {
        set_error("block shape b2=%d, rows=%d, D=%d exceeds the LDS budget of the generic path", a.b2, a.nf * a.b1, a.D);
        return SFM_ERR_UNSUPPORTED;
    }
    if (dtype == SFM_F32) return launch_generic_t<float>(a, nunits, stream, ev);
    if (dtype == SFM_BF16) return launch_generic_t<BF16>(a, nunits, stream, ev);
    return launch_generic_t<F16>(a, nunits, stream, ev);
}

}  // namespace sfm
