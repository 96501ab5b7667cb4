// Dense (non-causal) softmax attention of a query chunk against a KV-cache prefix, and the cache
// row copy used by the *_with_kv_cache entry points.
//
// Replaces attention() (wan/modules/attention.py:141-187, SDPA branch) and the Triton _attn_fwd
// (wan/modules/attn_patch.py:20-110).
//
// MFMA kernel (bf16 / fp16, head_dim 64 or 128): workgroup = 128 queries of one (batch, head),
// wave = 32 queries.  Per 64-key tile (K row-major and V^T staged once in LDS):
//     S^T[l, q] = K[l,:] . Q[q,:]          online softmax per query column (lane)
//     O^T[d, q] += V^T[d, l] P^T[l, q]     P^T is fed from the accumulator layout (perm_row)
// The next tile's K/V rows are prefetched into registers while the current one is consumed.

#include "sfm_common.hpp"

namespace sfm {

template <int D>
struct DnLds {
    static constexpr int kRowPitch = D + 8;
    static constexpr int kTPitch = 72;
    static constexpr int kKrow = 0;
    static constexpr int kVT = 64 * kRowPitch;
    static constexpr int kTiles = kVT + D * kTPitch;
    static constexpr int kStage = 4 * 32 * kRowPitch;
    static constexpr int kTotal = kTiles > kStage ? kTiles : kStage;
    static constexpr size_t bytes() { return 2 * (size_t)kTotal; }
};

template <class E, int D>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void dense_fwd_kernel(sfm_dense_desc p, const uint16_t* __restrict__ q,
                                                        const uint16_t* __restrict__ kp,
                                                        const uint16_t* __restrict__ vp, uint16_t* __restrict__ out,
                                                        float* __restrict__ lse) {
    using L = DnLds<D>;
    constexpr int DS = D / 16, DT = D / 32, DP = D / 2;
    __shared__ __attribute__((aligned(16))) uint16_t lds[L::kTotal];

    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, m = lane & 31, hf = lane >> 5;
    const int b = blockIdx.y / p.H, h = blockIdx.y % p.H;
    const int q0 = blockIdx.x * 128 + wave * 32;
    const int nq = p.q_tokens, nk = p.kv_tokens;

    const uint16_t* kg = kp + (int64_t)b * p.k_stride[0] + (int64_t)h * p.k_stride[2];
    const uint16_t* vg = vp + (int64_t)b * p.v_stride[0] + (int64_t)h * p.v_stride[2];

    // query operand (B of the logits MFMA): lane (m, hf) holds Q[q0 + m][16 ds + 8 hf + 0..7]
    u32x4 qb[DS];
    {
        const int qi = min(q0 + m, nq - 1);
        const uint16_t* qrow = q + (int64_t)b * p.q_stride[0] + (int64_t)qi * p.q_stride[1] + (int64_t)h * p.q_stride[2] + 8 * hf;
#pragma unroll
        for (int ds = 0; ds < DS; ++ds) qb[ds] = *(const u32x4*)(qrow + 16 * ds);
    }

    constexpr int kTasks = 8 * DP;                 // (sh, dword column) staging tasks per matrix
    constexpr int kPer = (kTasks + 255) / 256;     // 2 for D=128, 1 for D=64
    uint32_t pk[kPer][8], pv[kPer][8];
    auto prefetch = [&](int l0) {
#pragma unroll
        for (int t = 0; t < kPer; ++t) {
            int task = tid + t * 256;
            if (task < kTasks) {
                int pc = task % DP, sh = task / DP;
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    int l = l0 + perm_row(sh >> 1, sh & 1, e);
                    uint32_t kk = 0, vv = 0;
                    if (l < nk) {
                        kk = *(const uint32_t*)(kg + (int64_t)l * p.k_stride[1] + 2 * pc);
                        vv = *(const uint32_t*)(vg + (int64_t)l * p.v_stride[1] + 2 * pc);
                    }
                    pk[t][e] = kk;
                    pv[t][e] = vv;
                }
            }
        }
    };
    auto commit = [&]() {
#pragma unroll
        for (int t = 0; t < kPer; ++t) {
            int task = tid + t * 256;
            if (task < kTasks) {
                int pc = task % DP, sh = task / DP;
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    int l = perm_row(sh >> 1, sh & 1, e);
                    *(uint32_t*)(lds + L::kKrow + l * L::kRowPitch + 2 * pc) = pk[t][e];
                }
                u32x4 lo, hi;
                lo.x = lo16x2(pv[t][0], pv[t][1]); lo.y = lo16x2(pv[t][2], pv[t][3]);
                lo.z = lo16x2(pv[t][4], pv[t][5]); lo.w = lo16x2(pv[t][6], pv[t][7]);
                hi.x = hi16x2(pv[t][0], pv[t][1]); hi.y = hi16x2(pv[t][2], pv[t][3]);
                hi.z = hi16x2(pv[t][4], pv[t][5]); hi.w = hi16x2(pv[t][6], pv[t][7]);
                *(u32x4*)(lds + L::kVT + (2 * pc) * L::kTPitch + sh * 8) = lo;
                *(u32x4*)(lds + L::kVT + (2 * pc + 1) * L::kTPitch + sh * 8) = hi;
            }
        }
    };

    f32x16 oacc[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int v = 0; v < 16; ++v) oacc[dt][v] = 0.f;
    float mrun = -INFINITY, lrun = 0.f;            // running max (scaled, base-2 units) and sum
    const float sc2 = p.sm_scale * kLog2e;
    const int ntile = (nk + 63) / 64;

    prefetch(0);
    for (int tile = 0; tile < ntile; ++tile) {
        lds_barrier();                   // everyone is done reading the previous tile
        commit();
        if (tile + 1 < ntile) prefetch(64 * (tile + 1));
        lds_barrier();                   // tile visible; the prefetch stays in flight

        f32x16 s[2];
#pragma unroll
        for (int t = 0; t < 2; ++t) {
#pragma unroll
            for (int v = 0; v < 16; ++v) s[t][v] = 0.f;
            const uint16_t* arow = lds + L::kKrow + (32 * t + m) * L::kRowPitch + 8 * hf;
#pragma unroll
            for (int ds = 0; ds < DS; ++ds) {
                u32x4 a = *(const u32x4*)(arow + 16 * ds);
                s[t] = E::mfma32(a, qb[ds], s[t]);
            }
        }
        // online softmax in base 2; the scale is folded into the exponent argument (one fma per logit)
        const int lrem = nk - 64 * tile;           // valid keys in this tile (>= 1)
        if (lrem < 64) {                           // ragged last tile only (wave-uniform)
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    int l = 32 * t + 8 * (v >> 2) + 4 * hf + (v & 3);
                    s[t][v] = l < lrem ? s[t][v] : kMaskLogit;
                }
        }
        float mx = s[0][0];
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int v = 0; v < 16; ++v) mx = fmaxf(mx, s[t][v]);
        mx = xhalf_max(mx) * sc2;
        const float mnew = fmaxf(mrun, mx);
        float psum = 0.f;
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                float e = fast_exp2(fmaf(s[t][v], sc2, -mnew));
                psum += e;
                s[t][v] = e;
            }
        u32x4 pb[4];
#pragma unroll
        for (int st = 0; st < 4; ++st) {
            const int t = st >> 1, v0 = 8 * (st & 1);
            pb[st].x = pack2<E>(s[t][v0 + 0], s[t][v0 + 1]);
            pb[st].y = pack2<E>(s[t][v0 + 2], s[t][v0 + 3]);
            pb[st].z = pack2<E>(s[t][v0 + 4], s[t][v0 + 5]);
            pb[st].w = pack2<E>(s[t][v0 + 6], s[t][v0 + 7]);
        }
        // rescale the running output only when some query of the wave raised its maximum
        if (__builtin_amdgcn_ballot_w64(mnew > mrun) != 0) {
            const float alpha = fast_exp2(mrun - mnew);
            lrun *= alpha;
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                for (int v = 0; v < 16; ++v) oacc[dt][v] *= alpha;
            mrun = mnew;
        }
        lrun += psum;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
            const uint16_t* arow = lds + L::kVT + (32 * dt + m) * L::kTPitch + 8 * hf;
#pragma unroll
            for (int st = 0; st < 4; ++st) {
                u32x4 a = *(const u32x4*)(arow + 16 * st);
                oacc[dt] = E::mfma32(a, pb[st], oacc[dt]);
            }
        }
    }

    const float ltot = xhalf_sum(lrun);
    const float inv = 1.f / ltot;
    if (lse != nullptr && hf == 0 && q0 + m < nq)
        lse[((int64_t)b * p.H + h) * nq + q0 + m] = (mrun + log2f(ltot)) * kLn2;

    __syncthreads();                                   // tiles are dead; reuse LDS as output stage
    uint16_t* stage = lds + wave * 32 * L::kRowPitch;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            u32x2 w;
            w.x = pack2<E>(oacc[dt][4 * g + 0] * inv, oacc[dt][4 * g + 1] * inv);
            w.y = pack2<E>(oacc[dt][4 * g + 2] * inv, oacc[dt][4 * g + 3] * inv);
            *(u32x2*)(stage + m * L::kRowPitch + 32 * dt + 8 * g + 4 * hf) = w;
        }
    __syncthreads();
    {
        uint16_t* og = out + (int64_t)b * p.o_stride[0] + (int64_t)h * p.o_stride[2];
        constexpr int CH = D / 8;
        for (int c = lane; c < 32 * CH; c += 64) {
            int r = c / CH, ch = c % CH;
            if (q0 + r < nq) {
                u32x4 w = *(const u32x4*)(stage + r * L::kRowPitch + ch * 8);
                *(u32x4*)(og + (int64_t)(q0 + r) * p.o_stride[1] + ch * 8) = w;
            }
        }
    }
}

// ------------------------------------------------------------------------------------------------
// shape-generic fp32 path: workgroup = one query of one (batch, head); keys in chunks of 256
// ------------------------------------------------------------------------------------------------
template <typename T> struct DLd;
template <> struct DLd<float> {
    static __device__ __forceinline__ float get(const void* p, int64_t i) { return ((const float*)p)[i]; }
    static __device__ __forceinline__ void put(void* p, int64_t i, float x) { ((float*)p)[i] = x; }
};
template <> struct DLd<BF16> {
    static __device__ __forceinline__ float get(const void* p, int64_t i) { return BF16::to_float(((const uint16_t*)p)[i]); }
    static __device__ __forceinline__ void put(void* p, int64_t i, float x) { ((uint16_t*)p)[i] = BF16::from_float(x); }
};
template <> struct DLd<F16> {
    static __device__ __forceinline__ float get(const void* p, int64_t i) { return F16::to_float(((const uint16_t*)p)[i]); }
    static __device__ __forceinline__ void put(void* p, int64_t i, float x) { ((uint16_t*)p)[i] = F16::from_float(x); }
};

template <typename T>
__global__ __launch_bounds__(256) void dense_generic_kernel(sfm_dense_desc p, const void* q, const void* kp,
                                                            const void* vp, void* out, float* lse) {
    __shared__ float qs[256];
    __shared__ float zs[256];
    __shared__ float red[256];
    const int tid = threadIdx.x;
    const int qi = blockIdx.x;
    const int b = blockIdx.y / p.H, h = blockIdx.y % p.H;
    const int D = p.D;
    const int64_t qoff = (int64_t)b * p.q_stride[0] + (int64_t)qi * p.q_stride[1] + (int64_t)h * p.q_stride[2];
    const int64_t koff = (int64_t)b * p.k_stride[0] + (int64_t)h * p.k_stride[2];
    const int64_t voff = (int64_t)b * p.v_stride[0] + (int64_t)h * p.v_stride[2];
    if (tid < D) qs[tid] = DLd<T>::get(q, qoff + tid);
    __syncthreads();
    const float sc2 = p.sm_scale * kLog2e;
    float mrun = -INFINITY, lrun = 0.f, acc = 0.f;      // acc: output element d = tid
    for (int l0 = 0; l0 < p.kv_tokens; l0 += 256) {
        const int l = l0 + tid;
        float z = -INFINITY;
        if (l < p.kv_tokens) {
            float s = 0.f;
            for (int d = 0; d < D; ++d) s += qs[d] * DLd<T>::get(kp, koff + (int64_t)l * p.k_stride[1] + d);
            z = s * sc2;
        }
        red[tid] = z;
        __syncthreads();
        for (int s = 128; s > 0; s >>= 1) {
            if (tid < s) red[tid] = fmaxf(red[tid], red[tid + s]);
            __syncthreads();
        }
        const float mnew = fmaxf(mrun, red[0]);
        __syncthreads();
        const float e = exp2f(z - mnew);
        zs[tid] = e;
        red[tid] = e;
        __syncthreads();
        for (int s = 128; s > 0; s >>= 1) {
            if (tid < s) red[tid] += red[tid + s];
            __syncthreads();
        }
        const float alpha = exp2f(mrun - mnew);
        lrun = lrun * alpha + red[0];
        mrun = mnew;
        if (tid < D) {
            acc *= alpha;
            const int cnt = min(256, p.kv_tokens - l0);
            for (int r = 0; r < cnt; ++r) acc += zs[r] * DLd<T>::get(vp, voff + (int64_t)(l0 + r) * p.v_stride[1] + tid);
        }
        __syncthreads();
    }
    if (tid < D)
        DLd<T>::put(out, (int64_t)b * p.o_stride[0] + (int64_t)qi * p.o_stride[1] + (int64_t)h * p.o_stride[2] + tid, acc / lrun);
    if (lse != nullptr && tid == 0) lse[((int64_t)b * p.H + h) * p.q_tokens + qi] = (mrun + log2f(lrun)) * kLn2;
}

int launch_dense(const sfm_dense_desc& d, const void* q, const void* k, const void* v, void* out, float* lse,
                 hipStream_t stream) {
    const bool mfma = (d.dtype == SFM_BF16 || d.dtype == SFM_F16) && (d.D == 64 || d.D == 128);
    if (mfma) {
        dim3 grid((d.q_tokens + 127) / 128, d.B * d.H);
        const uint16_t* qq = (const uint16_t*)q;
        const uint16_t* kk = (const uint16_t*)k;
        const uint16_t* vv = (const uint16_t*)v;
        uint16_t* oo = (uint16_t*)out;
        if (d.dtype == SFM_BF16) {
            if (d.D == 128) hipLaunchKernelGGL((dense_fwd_kernel<BF16, 128>), grid, dim3(256), 0, stream, d, qq, kk, vv, oo, lse);
            else hipLaunchKernelGGL((dense_fwd_kernel<BF16, 64>), grid, dim3(256), 0, stream, d, qq, kk, vv, oo, lse);
        } else {
            if (d.D == 128) hipLaunchKernelGGL((dense_fwd_kernel<F16, 128>), grid, dim3(256), 0, stream, d, qq, kk, vv, oo, lse);
            else hipLaunchKernelGGL((dense_fwd_kernel<F16, 64>), grid, dim3(256), 0, stream, d, qq, kk, vv, oo, lse);
        }
    } else {
        dim3 grid(d.q_tokens, d.B * d.H);
        if (d.dtype == SFM_F32) hipLaunchKernelGGL((dense_generic_kernel<float>), grid, dim3(256), 0, stream, d, q, k, v, out, lse);
        else if (d.dtype == SFM_BF16) hipLaunchKernelGGL((dense_generic_kernel<BF16>), grid, dim3(256), 0, stream, d, q, k, v, out, lse);
        else hipLaunchKernelGGL((dense_generic_kernel<F16>), grid, dim3(256), 0, stream, d, q, k, v, out, lse);
    }
    hipError_t err = hipGetLastError();
    if (err != hipSuccess) {
        set_error("hip launch failed: %s", hipGetErrorString(err));
        return SFM_ERR_HIP;
    }
    return SFM_OK;
}

// ------------------------------------------------------------------------------------------------
// cache row copy: new rows (token order) -> cache[start + block-order index]
// ------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void kv_cache_write_kernel(int B, int H, int chunks_per_head, TokMap map, int nbf,
                                                             const u32x4* __restrict__ nk, const u32x4* __restrict__ nv,
                                                             int64_t ns0, int64_t ns1, int64_t ns2, u32x4* __restrict__ kc,
                                                             u32x4* __restrict__ vc, int64_t cs0, int64_t cs1, int64_t cs2,
                                                             int64_t start) {
    // strides are in 16-byte units here
    const int64_t per_tok = (int64_t)H * chunks_per_head;
    const int64_t ntok = (int64_t)nbf * map.b1 * map.b2;
    const int64_t total = (int64_t)B * ntok * per_tok;
    for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (int64_t)gridDim.x * blockDim.x) {
        int64_t c = idx % chunks_per_head;
        int64_t t = idx / chunks_per_head;
        int hd = (int)(t % H);
        t /= H;
        int64_t blk_tok = t % ntok;       // position in block order
        int b = (int)(t / ntok);
        int j = (int)(blk_tok % map.b2);
        int64_t r = blk_tok / map.b2;
        int i = (int)(r % map.b1);
        int bf = (int)(r / map.b1);
        int64_t src_tok = map.row(bf, i) + j;
        int64_t so = b * ns0 + src_tok * ns1 + hd * ns2 + c;
        int64_t dst = b * cs0 + (start + blk_tok) * cs1 + hd * cs2 + c;
        kc[dst] = nk[so];
        vc[dst] = nv[so];
    }
}

int launch_kv_cache_write(int esz, int B, int H, int D, const TokMap& map, int nbf, const void* nk, const void* nv,
                          const int64_t ns[3], void* kc, void* vc, const int64_t cs[3], int64_t start,
                          hipStream_t stream) {
    const int per16 = 16 / esz;
    const int cph = D / per16;
    const int64_t total = (int64_t)B * nbf * map.b1 * map.b2 * H * cph;
    int64_t blocks = (total + 255) / 256;
    if (blocks > 65536) blocks = 65536;
    hipLaunchKernelGGL(kv_cache_write_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, B, H, cph, map, nbf,
                       (const u32x4*)nk, (const u32x4*)nv, ns[0] / per16, ns[1] / per16, ns[2] / per16, (u32x4*)kc,
                       (u32x4*)vc, cs[0] / per16, cs[1] / per16, cs[2] / per16, start);
    hipError_t err = hipGetLastError();
    if (err != hipSuccess) {
        set_error("hip launch failed: %s", hipGetErrorString(err));
        return SFM_ERR_HIP;
    }
    return SFM_OK;
}

}  // namespace sfm
