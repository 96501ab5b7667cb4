// Right-factor part of the Monarch backward on gfx950 MFMA (bf16 / fp16, head_dim 64 or 128, b2 <= 64 a multiple of 4,
// at most 160 (a, j) columns).
//
// Replaces, per tile t = (unit, k, f), the small batched products and the row kernel of the GEMM chain
//     dR[aj, l]  = dKbar[aj,:] . K[l,:] + dY[aj,:] . V[l,:]
//     dS1[aj, l] = R (dR + dc ln R - sum_l R (dR + dc ln R))
//     dK[l, :]   = sum_aj R[aj, l] dKbar[aj,:]          (the s dS1^T q term is added by the library GEMM that follows)
//     dV[l, :]   = sum_aj R[aj, l] dY[aj,:]
// (wan/modules/monarch_attn.py:403-596 `_al_cl_y_bwd`).  One workgroup per tile: the K and V blocks, the tile's rows of
// R, dKbar and dY (all contiguous in the backward's scratch) go straight into LDS (global_load_lds_dwordx4, 16-byte
// chunks XOR-swizzled per row as in the dense attention kernel), rows past the end are zeroed.
//   phase 1: wave = 32 columns aj.  dR^T[l, aj] with A = K / V rows, B = dKbar / dY rows, so that a lane owns one
//            column and the softmax backward is in-lane plus one cross-half add; dS1 leaves as 8-byte pieces.
//   phase 2: wave = (dK or dV, 32 head-dim rows).  C^T[d, l] with both operands from transposing LDS reads
//            (ds_read_tr16_b64): A = dKbar^T / dY^T, B = R^T, contraction over the columns aj.

#include <hip/hip_runtime.h>

#include <type_traits>

#include "sfm_attn.h"
#include "sfm_common.hpp"

namespace sfm {
namespace {

constexpr int kMaxAJ = 160;

struct RightArgs {
    const char* kk;          // [t][b2][D]
    const char* vk;
    const char* rb;          // [t][AJ][64]
    const char* dkbar;       // [t][AJ][D]
    const char* dy;
    const float* dc;         // [u][AJ][RR]
    uint16_t* ds1;           // [(u, k)][AJ][nf * b2]
    float* dkk;              // [t][b2][D]
    float* dvk;
    int b1, b2, AJ, nf;
};

typedef short br_s16x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ u32x2 br_read_tr(const char* lds, uint32_t off) {
    br_s16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((br_s16x4 __attribute__((address_space(3)))*)(lds + off));
    return __builtin_bit_cast(u32x2, v);
}
__device__ __forceinline__ void br_load_lds16(const char* base, uint32_t off, uint32_t lds_addr) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_addr), "v"(off), "s"(base) : "memory", "m0");
}

// chunk c (16 bytes) of row r sits at chunk position c ^ swz(r); rows of CPR chunks (16: 256-byte rows, 8: 128-byte rows)
template <int CPR>
__device__ __forceinline__ int br_swz(int r) {
    return CPR >= 16 ? (((r & 3) << 2) | ((r >> 2) & 3)) : ((((r >> 1) & 1) << 2) | ((r >> 2) & 3));
}

template <class E, int D>
__global__ __launch_bounds__(320) void monarch_bwd_right_kernel(RightArgs p) {
    constexpr int DS = D / 16, DT = D / 32;
    constexpr int CPR = D / 8;                            // chunks per row of the D-wide tiles
    constexpr int kPitch = 2 * D;
    constexpr int kKV = 64 * kPitch;                      // K or V tile, 64 rows
    constexpr int kG = kMaxAJ * kPitch;                   // dKbar or dY tile, 160 rows
    constexpr int kR = kMaxAJ * 128;                      // R tile, 160 rows of 64
    constexpr int oK = 0, oV = kKV, oG = 2 * kKV, oH = 2 * kKV + kG, oR = 2 * kKV + 2 * kG;
    extern __shared__ __attribute__((aligned(256))) char lds[];
    const uint32_t lds0 = (uint32_t)(size_t)(__attribute__((address_space(3))) char*)lds;

    const int tid = threadIdx.x, lane = tid & 63, m = lane & 31, hf = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int64_t t = blockIdx.x;
    const int b2 = p.b2, AJ = p.AJ, nf = p.nf;
    const int f = (int)(t % nf);
    const int64_t uk = t / nf;
    const int k = (int)(uk % p.b1);
    const int64_t u = uk / p.b1;

    // ---- stage the five tiles: LDS position P (16-byte units) of a tile holds chunk (P % CPR) ^ swz(row) of row P / CPR
    auto stage = [&](const char* src, int nchunks, uint32_t dst, auto cpr_c) {
        constexpr int C = decltype(cpr_c)::value;
        for (int g = wave; g * 64 < nchunks; g += 5) {
            const int P = min(g * 64 + lane, nchunks - 1);             // lanes past the end repeat the last chunk (into a pad row, zeroed below)
            const int r = P / C, c = (P % C) ^ br_swz<C>(r);
            br_load_lds16(src, (uint32_t)((r * C + c) * 16), lds0 + dst + (uint32_t)g * 1024);
        }
    };
    using c_d = std::integral_constant<int, CPR>;
    using c_r = std::integral_constant<int, 8>;
    stage(p.kk + t * b2 * kPitch, b2 * CPR, oK, c_d{});
    stage(p.vk + t * b2 * kPitch, b2 * CPR, oV, c_d{});
    stage(p.dkbar + t * AJ * kPitch, AJ * CPR, oG, c_d{});
    stage(p.dy + t * AJ * kPitch, AJ * CPR, oH, c_d{});
    stage(p.rb + t * AJ * 128, AJ * 8, oR, c_r{});
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    // rows past the end of a tile are zero, so that they add nothing to any contraction
    {
        const u32x4 z = {0u, 0u, 0u, 0u};
        for (int i = tid; i < (64 - b2) * CPR; i += 320) {
            *(u32x4*)(lds + oK + b2 * kPitch + i * 16) = z;
            *(u32x4*)(lds + oV + b2 * kPitch + i * 16) = z;
        }
        for (int i = tid; i < (kMaxAJ - AJ) * CPR; i += 320) {
            *(u32x4*)(lds + oG + AJ * kPitch + i * 16) = z;
            *(u32x4*)(lds + oH + AJ * kPitch + i * 16) = z;
        }
        for (int i = tid; i < (kMaxAJ - AJ) * 8; i += 320) *(u32x4*)(lds + oR + AJ * 128 + i * 16) = z;
    }
    __syncthreads();

    // ---- phase 1: dS1 for the wave's 32 columns
    {
        const int col = 32 * wave + m;                                   // < 160
        const bool col_ok = col < AJ;
        const uint32_t a_off = (uint32_t)m * kPitch + (uint32_t)((hf ^ br_swz<CPR>(m)) << 4);          // rows l = 32 tl + m (swz depends on r mod 16)
        const uint32_t b_off = (uint32_t)col * kPitch + (uint32_t)((hf ^ br_swz<CPR>(col)) << 4);
        f32x16 dr[2];
#pragma unroll
        for (int tl = 0; tl < 2; ++tl)
#pragma unroll
            for (int v = 0; v < 16; ++v) dr[tl][v] = 0.f;
#pragma unroll
        for (int ds = 0; ds < DS; ++ds) {
            const u32x4 bg = *(const u32x4*)(lds + oG + (b_off ^ (uint32_t)(ds << 5)));
            const u32x4 bh = *(const u32x4*)(lds + oH + (b_off ^ (uint32_t)(ds << 5)));
#pragma unroll
            for (int tl = 0; tl < 2; ++tl) {
                const u32x4 ak = *(const u32x4*)(lds + oK + tl * 32 * kPitch + (a_off ^ (uint32_t)(ds << 5)));
                const u32x4 av = *(const u32x4*)(lds + oV + tl * 32 * kPitch + (a_off ^ (uint32_t)(ds << 5)));
                dr[tl] = E::mfma32(ak, bg, dr[tl]);
                dr[tl] = E::mfma32(av, bh, dr[tl]);
            }
        }
        // R[col][l] for the l this lane holds: l = 32 tl + 8 g + 4 hf + 0..3, i.e. 8 bytes of chunk 4 tl + g
        const float dcv = col_ok ? p.dc[(u * AJ + col) * ((int64_t)nf * p.b1) + (int64_t)k * nf + f] : 0.f;
        float rv[2][16];
        float dot = 0.f;
#pragma unroll
        for (int tl = 0; tl < 2; ++tl)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int c = 4 * tl + g;
                const u32x2 w = *(const u32x2*)(lds + oR + col * 128 + ((c ^ br_swz<8>(col)) << 4) + 8 * hf);
                const float r0 = E::to_float((uint16_t)(w.x & 0xffffu)), r1 = E::to_float((uint16_t)(w.x >> 16));
                const float r2 = E::to_float((uint16_t)(w.y & 0xffffu)), r3 = E::to_float((uint16_t)(w.y >> 16));
                const bool live = 32 * tl + 8 * g + 4 * hf < b2;        // b2 is a multiple of 4: whole pieces
                const float rr[4] = {live ? r0 : 0.f, live ? r1 : 0.f, live ? r2 : 0.f, live ? r3 : 0.f};
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int v = 4 * g + e;
                    float gv = dr[tl][v];
                    if (rr[e] > 0.f) gv += dcv * __logf(rr[e]);          // dR + dc ln R
                    else gv = 0.f;
                    rv[tl][v] = rr[e];
                    dr[tl][v] = gv;
                    dot += rr[e] * gv;
                }
            }
        dot = xhalf_sum(dot);
        uint16_t* out = p.ds1 + (uk * AJ + col) * ((int64_t)nf * b2) + (int64_t)f * b2;
#pragma unroll
        for (int tl = 0; tl < 2; ++tl)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int l0 = 32 * tl + 8 * g + 4 * hf;
                u32x2 w;
                w.x = pack2<E>(rv[tl][4 * g + 0] * (dr[tl][4 * g + 0] - dot), rv[tl][4 * g + 1] * (dr[tl][4 * g + 1] - dot));
                w.y = pack2<E>(rv[tl][4 * g + 2] * (dr[tl][4 * g + 2] - dot), rv[tl][4 * g + 3] * (dr[tl][4 * g + 3] - dot));
                if (col_ok && l0 < b2) *(u32x2*)(out + l0) = w;
            }
    }

    // ---- phase 2: dK^T[d, l] = sum_aj dKbar^T[d, aj] R[aj, l] and the same with dY for dV; work items (product, 32 head-dim rows)
    {
        const int s16 = lane & 15, g16 = lane >> 4;
        const int rl = 4 * hf + (s16 >> 2);
        const int cl = 2 * (g16 & 1) + ((s16 & 3) >> 1);
        const uint32_t sub = (uint32_t)(s16 & 1) * 8;
        for (int item = wave; item < 2 * DT; item += 5) {
            const int which = item / DT, dt = item % DT;
            const uint32_t oA = which == 0 ? oG : oH;
            f32x16 acc[2];
#pragma unroll
            for (int lb = 0; lb < 2; ++lb)
#pragma unroll
                for (int v = 0; v < 16; ++v) acc[lb][v] = 0.f;
#pragma unroll
            for (int ks = 0; ks < kMaxAJ / 16; ++ks) {
                const int r0 = 16 * ks + rl, r1 = r0 + 8;                 // rows aj of the two halves of the operand
                const int ca = 4 * dt + cl;
                const u32x2 alo = br_read_tr(lds, oA + (uint32_t)r0 * kPitch + (uint32_t)((ca ^ br_swz<CPR>(r0)) << 4) + sub);
                const u32x2 ahi = br_read_tr(lds, oA + (uint32_t)r1 * kPitch + (uint32_t)((ca ^ br_swz<CPR>(r1)) << 4) + sub);
                const u32x4 aop = {alo.x, alo.y, ahi.x, ahi.y};
#pragma unroll
                for (int lb = 0; lb < 2; ++lb) {
                    const int cb = 4 * lb + cl;
                    const u32x2 blo = br_read_tr(lds, oR + (uint32_t)r0 * 128 + (uint32_t)((cb ^ br_swz<8>(r0)) << 4) + sub);
                    const u32x2 bhi = br_read_tr(lds, oR + (uint32_t)r1 * 128 + (uint32_t)((cb ^ br_swz<8>(r1)) << 4) + sub);
                    const u32x4 bop = {blo.x, blo.y, bhi.x, bhi.y};
                    acc[lb] = E::mfma32(aop, bop, acc[lb]);
                }
            }
            float* dst = which == 0 ? p.dkk : p.dvk;
#pragma unroll
            for (int lb = 0; lb < 2; ++lb) {
                const int l = 32 * lb + m;
                if (l < b2) {
                    float* row = dst + (t * b2 + l) * D + 32 * dt + 4 * hf;
#pragma unroll
                    for (int g = 0; g < 4; ++g) {
                        const f32x4 w = {acc[lb][4 * g + 0], acc[lb][4 * g + 1], acc[lb][4 * g + 2], acc[lb][4 * g + 3]};
                        *(f32x4*)(row + 8 * g) = w;
                    }
                }
            }
        }
    }
}

}  // namespace

bool monarch_bwd_right_supported(int dtype, int D, int b2, int AJ) {
    return (dtype == SFM_BF16 || dtype == SFM_F16) && (D == 64 || D == 128) && b2 >= 4 && b2 <= 64 && b2 % 4 == 0 && AJ <= kMaxAJ;
}

int launch_monarch_bwd_right(int dtype, int D, int64_t ntiles, int b1, int b2, int AJ, int nf, const void* kk, const void* vk,
                             const void* rb, const void* dkbar, const void* dy, const float* dc, void* ds1, float* dkk, float* dvk,
                             hipStream_t stream) {
    RightArgs a;
    a.kk = (const char*)kk; a.vk = (const char*)vk; a.rb = (const char*)rb;
    a.dkbar = (const char*)dkbar; a.dy = (const char*)dy;
    a.dc = dc;
    a.ds1 = (uint16_t*)ds1;
    a.dkk = dkk; a.dvk = dvk;
    a.b1 = b1; a.b2 = b2; a.AJ = AJ; a.nf = nf;
    const size_t ldsb = (size_t)2 * 64 * 2 * D + (size_t)2 * kMaxAJ * 2 * D + (size_t)kMaxAJ * 128;
    const void* fn = nullptr;
    if (dtype == SFM_BF16) fn = D == 128 ? (const void*)monarch_bwd_right_kernel<BF16, 128> : (const void*)monarch_bwd_right_kernel<BF16, 64>;
    else fn = D == 128 ? (const void*)monarch_bwd_right_kernel<F16, 128> : (const void*)monarch_bwd_right_kernel<F16, 64>;
    if (ldsb > 64 * 1024) {
        hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)ldsb);
        if (e != hipSuccess) {
            set_error("monarch backward (right factor): cannot reserve %zu bytes of LDS: %s", ldsb, hipGetErrorString(e));
            return SFM_ERR_HIP;
        }
    }
    const dim3 grid((unsigned)ntiles);
    if (dtype == SFM_BF16) {
        if (D == 128) hipLaunchKernelGGL((monarch_bwd_right_kernel<BF16, 128>), grid, dim3(320), ldsb, stream, a);
        else hipLaunchKernelGGL((monarch_bwd_right_kernel<BF16, 64>), grid, dim3(320), ldsb, stream, a);
    } else {
        if (D == 128) hipLaunchKernelGGL((monarch_bwd_right_kernel<F16, 128>), grid, dim3(320), ldsb, stream, a);
        else hipLaunchKernelGGL((monarch_bwd_right_kernel<F16, 64>), grid, dim3(320), ldsb, stream, a);
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        set_error("monarch backward (right factor): launch failed: %s", hipGetErrorString(e));
        return SFM_ERR_HIP;
    }
    return SFM_OK;
}

}  // namespace sfm
