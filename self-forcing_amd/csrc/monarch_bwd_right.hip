// Right-factor part of the Monarch backward on gfx950 MFMA (bf16 / fp16, head_dim 64 or 128, b2 <= 64 a multiple of 4;
// at most 480 (a, j) columns, taken 160 at a time).
//
// Replaces, per tile t = (unit, k, f), the small batched products and the row kernel of the GEMM chain
//     dR[aj, l]  = dKbar[aj,:] . K[l,:] + dY[aj,:] . V[l,:]
//     dS1[aj, l] = R (dR + dc ln R - sum_l R (dR + dc ln R))
//     dK[l, :]   = sum_aj R[aj, l] dKbar[aj,:] + s sum_aj dS1[aj, l] q[aj,:]
//     dV[l, :]   = sum_aj R[aj, l] dY[aj,:]
// (wan/modules/monarch_attn.py:403-596 `_al_cl_y_bwd`).  One workgroup per tile: the K and V blocks (52 rows each, read
// where the callers' tensors have them), and the tile's rows of R, dKbar and dY (contiguous in the backward's scratch)
// go straight into LDS (global_load_lds_dwordx4, 16-byte chunks XOR-swizzled per row as in the dense attention
// kernel); rows past the end are zeroed.  A tile with more than 160 columns is taken in passes of 160, the K and V
// blocks and the accumulators of dK and dV staying where they are.
// Sixteen waves per workgroup (one workgroup fills the LDS of a compute unit, so the waves have to come from it).
//   phase 1: wave = 32 columns aj x 32 key rows l (ten waves busy).  dR^T[l, aj] with A = K / V rows, B = dKbar / dY
//            rows, so that a lane owns one column and the softmax backward is in-lane plus one cross-half add and one
//            exchange between the two waves of a column through LDS.
//   phase 2: wave = 32 head-dim rows x 32 key rows of dV or of dK.  C^T[d, l] with both operands from transposing LDS
//            reads (ds_read_tr16_b64): A = dY^T / dKbar^T / q^T, B = R or dS1 (kept in LDS, 16 bit; with a single pass
//            over the K / V tiles once phase 1 is done with them), contraction over the columns aj.  The products
//            with R run right after the logits of phase 1; the query rows of (unit, k) then load over the dY tile
//            while the softmax backward runs.  dK and dV leave in the tensor dtype, straight to the caller's rows;
//            tiles whose kv block-frame is outside the wanted range skip phase 2.
// dS1 is also written to memory (16 bit) for dQ = s dS1 K, which contracts over f across tiles (monarch_bwd_dqk_kernel
// below).

#include <hip/hip_runtime.h>

#include <type_traits>

#include "sfm_attn.h"
#include "sfm_common.hpp"

namespace sfm {
namespace {

constexpr int kMaxAJ = 160;

struct RightArgs {
    const char* kk;          // callers' tensors: row kmap.row(f, k) + l, strides (batch, row, head) in elements
    const char* v;
    int64_t ks0, ks1, ks2, vs0, vs1, vs2;
    const char* rb;          // [t][AJ][64]
    const char* dkbar;       // [t][AJ][D]
    const char* dy;
    const float* dc;         // [u][AJ][RR]
    const char* q;           // caller's tensor: row (a, j) of (unit, k) is token qmap.row(a, k) + j, strides qs0, qs1, qs2
    int64_t qs0, qs1, qs2;
    TokMap qmap;
    uint16_t* ds1;           // [(u, k)][AJ][nf * b2]
    uint16_t* dk;            // caller's tensors: row kmap.row(f, k) + l - row0, strides s0 (batch), s1 (row), s2 (head)
    uint16_t* dv;
    int64_t s0, s1, s2, row0;
    TokMap kmap;
    int b1, b2, AJ, nf, H, unit0, f0, f1;
    float scale;
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

constexpr int kWaves = 16, kThreads = 64 * kWaves;

// NP: passes over the tile, 160 columns each (with more than one the dS1 tile has LDS of its own).  The passes are
// written out one after the other: as a loop, the invariant LDS addresses of all the transposing reads get hoisted
// out of it and spill.
template <class E, int D, int NP>
__global__ __launch_bounds__(kThreads) void monarch_bwd_right_kernel(RightArgs p) {
    constexpr int DS = D / 16, DT = D / 32;
    constexpr int CPR = D / 8;                            // chunks per row of the D-wide tiles
    constexpr int kPitch = 2 * D;
    constexpr int kKV = 64 * kPitch;                      // K or V tile, 64 rows
    constexpr int kG = kMaxAJ * kPitch;                   // dKbar or dY tile, 160 rows
    constexpr int kR = kMaxAJ * 128;                      // R tile, 160 rows of 64
    constexpr int oK = 0, oV = kKV, oG = 2 * kKV, oH = 2 * kKV + kG, oR = 2 * kKV + 2 * kG;
    // dS1 tile (like R): over the K / V tiles after phase 1 where it fits there and they are not needed again (head_dim
    // 128, all columns in one pass), else behind the R tile
    constexpr bool MULTI = NP > 1;
    constexpr bool s_over_kv = kR <= 2 * kKV && !MULTI;
    constexpr uint32_t oS = s_over_kv ? 0 : oR + kR;
    constexpr uint32_t oDot = oR + kR + (s_over_kv ? 0 : kR);             // float [2][160]: per-column partial sums of the two l halves
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
    auto stage = [&](const char* src, uint32_t row_bytes, int nchunks, uint32_t dst, auto cpr_c) {
        constexpr int C = decltype(cpr_c)::value;
        for (int g = wave; g * 64 < nchunks; g += kWaves) {
            const int P = min(g * 64 + lane, nchunks - 1);             // lanes past the end repeat the last chunk (into a pad row, zeroed below)
            const int r = P / C, c = (P % C) ^ br_swz<C>(r);
            br_load_lds16(src, (uint32_t)r * row_bytes + (uint32_t)(c * 16), lds0 + dst + (uint32_t)g * 1024);
        }
    };
    using c_d = std::integral_constant<int, CPR>;
    using c_r = std::integral_constant<int, 8>;
    const int unit = p.unit0 + (int)u;
    stage(p.kk + ((int64_t)(unit / p.H) * p.ks0 + (int64_t)(unit % p.H) * p.ks2 + p.kmap.row(f, k) * p.ks1) * 2, (uint32_t)(p.ks1 * 2),
          b2 * CPR, oK, c_d{});
    stage(p.v + ((int64_t)(unit / p.H) * p.vs0 + (int64_t)(unit % p.H) * p.vs2 + p.kmap.row(f, k) * p.vs1) * 2, (uint32_t)(p.vs1 * 2),
          b2 * CPR, oV, c_d{});
    const bool want = f >= p.f0 && f < p.f1;                             // uniform: dK / dV of this kv block-frame are asked for

    // phase 2 operands: C^T[d, l] = sum_aj A^T[d, aj] B[aj, l]; a wave owns 32 head-dim rows x 32 key rows of dV (waves
    // 0 .. 2 DT - 1) or of dK (the next 2 DT waves)
    const int s16 = lane & 15, g16 = lane >> 4;
    const int rl = 4 * hf + (s16 >> 2);
    const int cl = 2 * (g16 & 1) + ((s16 & 3) >> 1);
    const uint32_t sub = (uint32_t)(s16 & 1) * 8;
    const int dt = wave % DT, lb = (wave / DT) & 1, which = wave / (2 * DT);      // which: 0 dV, 1 dK, else idle
    auto product = [&](uint32_t oA, uint32_t oB, f32x16& acc) {      // acc += ...
        const int ca = 4 * dt + cl, cb = 4 * lb + cl;
#pragma unroll
        for (int ks = 0; ks < kMaxAJ / 16; ++ks) {
            const int r0 = 16 * ks + rl, r1 = r0 + 8;                     // rows aj of the two halves of the operands
            const u32x2 alo = br_read_tr(lds, oA + (uint32_t)r0 * kPitch + (uint32_t)((ca ^ br_swz<CPR>(r0)) << 4) + sub);
            const u32x2 ahi = br_read_tr(lds, oA + (uint32_t)r1 * kPitch + (uint32_t)((ca ^ br_swz<CPR>(r1)) << 4) + sub);
            const u32x2 blo = br_read_tr(lds, oB + (uint32_t)r0 * 128 + (uint32_t)((cb ^ br_swz<8>(r0)) << 4) + sub);
            const u32x2 bhi = br_read_tr(lds, oB + (uint32_t)r1 * 128 + (uint32_t)((cb ^ br_swz<8>(r1)) << 4) + sub);
            const u32x4 aop = {alo.x, alo.y, ahi.x, ahi.y};
            const u32x4 bop = {blo.x, blo.y, bhi.x, bhi.y};
            acc = E::mfma32(aop, bop, acc);
        }
    };
    // lane (l, hf) holds head-dim 32 dt + 8 g + 4 hf + 0..3 of key row l; the half swap leaves 8 consecutive ones per lane
    const int64_t obase = (int64_t)(unit / p.H) * p.s0 + (int64_t)(unit % p.H) * p.s2 + (p.kmap.row(f, k) - p.row0) * p.s1;
    auto store = [&](uint16_t* dst, const f32x16& acc) {
        const int l = 32 * lb + m;
        uint16_t* row = dst + obase + min(l, b2 - 1) * p.s1 + 32 * dt + 8 * hf;
#pragma unroll
        for (int gp = 0; gp < 2; ++gp) {
            const int g0 = 8 * gp, g1 = 8 * gp + 4;
            auto rx = __builtin_amdgcn_permlane32_swap(pack2<E>(acc[g0 + 0], acc[g0 + 1]), pack2<E>(acc[g1 + 0], acc[g1 + 1]), false, false);
            auto ry = __builtin_amdgcn_permlane32_swap(pack2<E>(acc[g0 + 2], acc[g0 + 3]), pack2<E>(acc[g1 + 2], acc[g1 + 3]), false, false);
            const u32x4 w = {(uint32_t)rx[0], (uint32_t)ry[0], (uint32_t)rx[1], (uint32_t)ry[1]};
            if (l < b2) *(u32x4*)(row + 16 * gp) = w;
        }
    };

    const bool active = wave < 10;                                       // phase 1: waves 0..9 = (32 columns, 32 rows l) blocks of dS1
    const int cblk = wave % 5, tl = (wave / 5) & 1;
    const int col = 32 * cblk + m;                                       // column within the pass, < 160
    const char* qbase = p.q + ((int64_t)(unit / p.H) * p.qs0 + (int64_t)(unit % p.H) * p.qs2) * 2;
    const uint32_t qrb = (uint32_t)(p.qs1 * 2);
    f32x16 acc, accq;                                                    // dV^T, or R^T dKbar and dS1^T q of dK^T
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[v] = accq[v] = 0.f;

    // the tile's columns (a, j), up to 160 per pass
    auto pass = [&](auto pi_c) {
    constexpr int pi = decltype(pi_c)::value;
    constexpr int c0 = pi * kMaxAJ;
    const int nrows = MULTI ? min(kMaxAJ, AJ - c0) : AJ;
    stage(p.dkbar + (t * AJ + c0) * kPitch, kPitch, nrows * CPR, oG, c_d{});
    stage(p.dy + (t * AJ + c0) * kPitch, kPitch, nrows * CPR, oH, c_d{});
    stage(p.rb + (t * AJ + c0) * 128, 128, nrows * 8, oR, c_r{});
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (nrows < kMaxAJ || c0 == 0) {                                     // rows past the end are zero: they add nothing to any contraction
        const u32x4 z = {0u, 0u, 0u, 0u};
        if (c0 == 0)                                                     // K, V rows past b2: what the logits pick up there is masked, but must be finite
            for (int i = tid; i < (64 - b2) * CPR; i += kThreads) {
                *(u32x4*)(lds + oK + b2 * kPitch + i * 16) = z;
                *(u32x4*)(lds + oV + b2 * kPitch + i * 16) = z;
            }
        for (int i = tid; i < (kMaxAJ - nrows) * CPR; i += kThreads) {
            *(u32x4*)(lds + oG + nrows * kPitch + i * 16) = z;
            *(u32x4*)(lds + oH + nrows * kPitch + i * 16) = z;
        }
        for (int i = tid; i < (kMaxAJ - nrows) * 8; i += kThreads) *(u32x4*)(lds + oR + nrows * 128 + i * 16) = z;
        __syncthreads();
    }

    // ---- phase 1, products: dR^T
    f32x16 dr;
#pragma unroll
    for (int v = 0; v < 16; ++v) dr[v] = 0.f;
    if (active) {
        const uint32_t a_off = (uint32_t)(32 * tl + m) * kPitch + (uint32_t)((hf ^ br_swz<CPR>(m)) << 4);   // swz depends on r mod 16
        const uint32_t b_off = (uint32_t)col * kPitch + (uint32_t)((hf ^ br_swz<CPR>(col)) << 4);
#pragma unroll
        for (int ds = 0; ds < DS; ++ds) {
            const u32x4 bg = *(const u32x4*)(lds + oG + (b_off ^ (uint32_t)(ds << 5)));
            const u32x4 bh = *(const u32x4*)(lds + oH + (b_off ^ (uint32_t)(ds << 5)));
            const u32x4 ak = *(const u32x4*)(lds + oK + (a_off ^ (uint32_t)(ds << 5)));
            const u32x4 av = *(const u32x4*)(lds + oV + (a_off ^ (uint32_t)(ds << 5)));
            dr = E::mfma32(ak, bg, dr);
            dr = E::mfma32(av, bh, dr);
        }
    }
    // ---- phase 2, the products that only need the loaded tiles: dV += R^T dY, dK += R^T dKbar
    if (want) {
        if (which == 0) {
            product(oH, oR, acc);
        } else if (which == 1) {
            product(oG, oR, acc);
        }
    }
    __syncthreads();                                                     // K, V, dKbar, dY tiles are free
    // the query rows of (unit, k) take the place of the dY tile while the softmax backward runs
    if (want) {
        const int nchunks = nrows * CPR;
        for (int g = wave; g * 64 < nchunks; g += kWaves) {
            const int P = min(g * 64 + lane, nchunks - 1);
            const int r = P / CPR, c = (P % CPR) ^ br_swz<CPR>(r);
            const int aj = c0 + r;
            const uint32_t tok = (uint32_t)(p.qmap.row(aj / b2, k) + aj % b2);
            br_load_lds16(qbase, tok * qrb + (uint32_t)(c * 16), lds0 + oH + (uint32_t)g * 1024);
        }
    }

    // ---- phase 1, softmax backward.  R[col][l] for the l this lane holds: l = 32 tl + 8 g + 4 hf + 0..3, 8 bytes of chunk 4 tl + g
    float rv[16];
    float dot = 0.f;
    if (active) {
        const float dcv = c0 + col < AJ ? p.dc[(u * AJ + c0 + col) * ((int64_t)nf * p.b1) + (int64_t)k * nf + f] : 0.f;
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const int c = 4 * tl + g;
            const u32x2 w = *(const u32x2*)(lds + oR + col * 128 + ((c ^ br_swz<8>(col)) << 4) + 8 * hf);
            const float r0 = E::to_float((uint16_t)(w.x & 0xffffu)), r1 = E::to_float((uint16_t)(w.x >> 16));
            const float r2 = E::to_float((uint16_t)(w.y & 0xffffu)), r3 = E::to_float((uint16_t)(w.y >> 16));
            const bool live = 32 * tl + 8 * g + 4 * hf < b2;            // b2 is a multiple of 4: whole pieces
            const float rr[4] = {live ? r0 : 0.f, live ? r1 : 0.f, live ? r2 : 0.f, live ? r3 : 0.f};
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int v = 4 * g + e;
                float gv = dr[v];
                if (rr[e] > 0.f) gv += dcv * __logf(rr[e]);              // dR + dc ln R
                else gv = 0.f;
                rv[v] = rr[e];
                dr[v] = gv;
                dot += rr[e] * gv;
            }
        }
        dot = xhalf_sum(dot);
        if (hf == 0) *(float*)(lds + oDot + (tl * kMaxAJ + col) * 4) = dot;
    }
    lds_barrier();                                                       // (the query rows stay in flight)
    if (active) {
        dot = *(const float*)(lds + oDot + col * 4) + *(const float*)(lds + oDot + (kMaxAJ + col) * 4);
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            u32x2 w;
            w.x = pack2<E>(rv[4 * g + 0] * (dr[4 * g + 0] - dot), rv[4 * g + 1] * (dr[4 * g + 1] - dot));
            w.y = pack2<E>(rv[4 * g + 2] * (dr[4 * g + 2] - dot), rv[4 * g + 3] * (dr[4 * g + 3] - dot));
            // into the dS1 tile, laid out like R's (columns past the end and l >= b2 come out as zeros)
            *(u32x2*)(lds + oS + col * 128 + (((4 * tl + g) ^ br_swz<8>(col)) << 4) + 8 * hf) = w;
        }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");                     // the query rows have landed
    __syncthreads();                                                     // the dS1 tile is complete
    // dS1 to memory for dQ = s dS1 K: row aj is b2 consecutive elements, 8-byte pieces, consecutive lanes along a row
    {
        const int ppr = b2 / 4;                                          // pieces per row
        uint16_t* out = p.ds1 + (uk * AJ + c0) * ((int64_t)nf * b2) + (int64_t)f * b2;
        for (int i = tid; i < nrows * ppr; i += kThreads) {
            const int row = i / ppr, pc = i % ppr;
            const u32x2 w = *(const u32x2*)(lds + oS + row * 128 + (((pc >> 1) ^ br_swz<8>(row)) << 4) + 8 * (pc & 1));
            *(u32x2*)(out + (int64_t)row * nf * b2 + 4 * pc) = w;
        }
    }
    if (want) {
        if ((nrows * CPR) % 64) {                                        // the last load spilled copies of a chunk into the zero rows
            const u32x4 z = {0u, 0u, 0u, 0u};
            for (int i = tid; i < (kMaxAJ - nrows) * CPR; i += kThreads) *(u32x4*)(lds + oH + nrows * kPitch + i * 16) = z;
            __syncthreads();
        }
        // ---- phase 2, the product that needs dS1: dS1^T q
        if (which == 1) product(oH, oS, accq);
    }
    if (pi + 1 < NP) __syncthreads();                                    // every wave is done with this pass's rows
    };
    pass(std::integral_constant<int, 0>{});
    if constexpr (NP > 1) pass(std::integral_constant<int, 1>{});
    if constexpr (NP > 2) pass(std::integral_constant<int, 2>{});
    if (!want) return;
    // dK = R^T dKbar + s dS1^T q
    if (which == 1) {
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[v] += p.scale * accq[v];
        store(p.dk, acc);
    } else if (which == 0) {
        store(p.dv, acc);
    }
}


// ---------------------------------------------------------------------------------------------------------------
// dQ of the right factor: dQk[(u, k)][aj, :] = s sum_{f, l} dS1[(u, k)][aj, (f, l)] K[(f, k, l), :], float, for the
// left-factor dQ kernel to add.  One workgroup per (unit, k), one wave per 32 columns (a, j); the K rows of the nf
// block-frames stream through LDS 64 at a time straight from the caller's tensor (global_load_lds_dwordx4, double
// buffered, chunk swizzle) and come back transposed as the B operand [n = d, k = (f, l)]; the A operand is dS1 straight
// from memory, two 8-byte pieces per step in the order in which the transposing reads deliver the rows.
struct DqkArgs {
    const char* k;           // caller's tensor: row kmap.row(f, k) + l, strides ks0 (batch), ks1 (row), ks2 (head), in elements
    int64_t ks0, ks1, ks2;
    TokMap kmap;
    const uint16_t* ds1;     // [(u, k)][AJ][nf * b2]
    float* dqk;              // [(u, k)][AJ][D]
    int b1, b2, AJ, nf, H, unit0;
    float scale;
};

template <class E, int D>
__global__ __launch_bounds__(1024) void monarch_bwd_dqk_kernel(DqkArgs p) {
    constexpr int DT = D / 32, CPR = D / 8;
    constexpr int kPitch = 2 * D;
    constexpr int kTile = 64 * kPitch;
    extern __shared__ __attribute__((aligned(256))) char lds[];          // two tiles of 64 K rows
    const uint32_t lds0 = (uint32_t)(size_t)(__attribute__((address_space(3))) char*)lds;

    const int tid = threadIdx.x, lane = tid & 63, m = lane & 31, hf = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int nwaves = __builtin_amdgcn_readfirstlane((int)blockDim.x >> 6);
    const int64_t uk = blockIdx.x;
    const int k = (int)(uk % p.b1);
    const int unit = p.unit0 + (int)(uk / p.b1);
    const int b2 = p.b2, AJ = p.AJ, NL = p.nf * b2;
    const int nt = (NL + 63) / 64;

    const char* kbase = p.k + ((int64_t)(unit / p.H) * p.ks0 + (int64_t)(unit % p.H) * p.ks2) * 2;
    const uint32_t krb = (uint32_t)(p.ks1 * 2);
    // LDS position P (16-byte units) of a tile holds chunk (P % CPR) ^ swz(row) of row P / CPR; row x of the flat (f, l)
    // axis is token kmap.row(x / b2, k) + x % b2 (rows past the end repeat the last one; dS1 is zero there)
    auto stage = [&](int t) {
        for (int g = wave; g < CPR; g += nwaves) {
            const int P = g * 64 + lane;
            const int r = P / CPR, c = (P % CPR) ^ br_swz<CPR>(r);
            const int x = min(64 * t + r, NL - 1);
            const uint32_t tok = (uint32_t)(p.kmap.row(x / b2, k) + x % b2);
            br_load_lds16(kbase, tok * krb + (uint32_t)(c * 16), lds0 + (uint32_t)(t & 1) * kTile + (uint32_t)g * 1024);
        }
    };
    // dS1 pieces of row aj = 32 wave + m: x = 64 t + 16 ks + 4 hf + {0..3} and + 8 + {0..3}
    const int aj = min(32 * wave + m, AJ - 1);
    const uint16_t* arow = p.ds1 + (uk * AJ + aj) * (int64_t)NL + 4 * hf;
    auto load_a = [&](int t, u32x4 (&a)[4]) {
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
            const int x0 = 64 * t + 16 * ks + 4 * hf;
            u32x2 lo = {0u, 0u}, hi = {0u, 0u};
            if (x0 + 4 <= NL) lo = *(const u32x2*)(arow + 64 * t + 16 * ks);           // NL is a multiple of 4: whole pieces
            if (x0 + 12 <= NL) hi = *(const u32x2*)(arow + 64 * t + 16 * ks + 8);
            a[ks] = u32x4{lo.x, lo.y, hi.x, hi.y};
        }
    };
    uint32_t tr[DT][2];
    {
        const int s16 = lane & 15, g16 = lane >> 4;
        const int rl = 4 * hf + (s16 >> 2);
        const int cl = 2 * (g16 & 1) + ((s16 & 3) >> 1);
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int half = 0; half < 2; ++half) {
                const int r = rl + 8 * half;             // swz depends on r mod 16 only
                tr[dt][half] = (uint32_t)(r * kPitch + (((4 * dt + cl) ^ br_swz<CPR>(r)) << 4) + (s16 & 1) * 8);
            }
    }
    f32x16 acc[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[dt][v] = 0.f;

    u32x4 acur[4], anext[4];
    stage(0);
    load_a(0, acur);
    for (int t = 0; t < nt; ++t) {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();                                   // tile t is in LDS; every wave is done with tile t - 1
        if (t + 1 < nt) {
            stage(t + 1);
            load_a(t + 1, anext);
        }
        const char* tile = lds + (t & 1) * kTile;
#pragma unroll
        for (int ks = 0; ks < 4; ++ks)
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
                const u32x2 lo = br_read_tr(tile, tr[dt][0] + ks * 16 * kPitch);
                const u32x2 hi = br_read_tr(tile, tr[dt][1] + ks * 16 * kPitch);
                const u32x4 bop = {lo.x, lo.y, hi.x, hi.y};
                acc[dt] = E::mfma32(acur[ks], bop, acc[dt]);
            }
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) acur[ks] = anext[ks];
    }
    // lane (d = 32 dt + m) holds rows aj = 32 wave + 8 g + 4 hf + e
    float* out = p.dqk + uk * AJ * D;
#pragma unroll
    for (int v = 0; v < 16; ++v) {
        const int row = 32 * wave + 8 * (v >> 2) + 4 * hf + (v & 3);
        if (row < AJ) {
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) out[(int64_t)row * D + 32 * dt + m] = acc[dt][v] * p.scale;
        }
    }
}

}  // namespace

bool monarch_bwd_right_supported(int dtype, int D, int b2, int AJ) {
    // up to three passes of 160 columns over a tile
    return (dtype == SFM_BF16 || dtype == SFM_F16) && (D == 64 || D == 128) && b2 >= 4 && b2 <= 64 && b2 % 4 == 0 && AJ <= 3 * kMaxAJ;
}

int launch_monarch_bwd_right(int dtype, int D, int64_t ntiles, int b1, int b2, int AJ, int nf, float scale, const void* kk,
                             const int64_t* ks, const void* v, const int64_t* vs, const void* rb, const void* dkbar, const void* dy, const float* dc, const void* q,
                             const int64_t* qs, const TokMap& qmap, void* ds1, void* dk, void* dv, const int64_t* dks, int64_t row0,
                             const TokMap& kmap, int H, int unit0, int f0, int f1, hipStream_t stream) {
    if ((dks[0] | dks[1] | dks[2] | vs[0] | vs[1] | vs[2] | ks[0] | ks[1] | ks[2]) % 8 ||
        ((uintptr_t)dk | (uintptr_t)dv | (uintptr_t)v | (uintptr_t)kk) % 16 || (int64_t)(b2 - 1) * vs[1] * 2 + 2 * D > 0xffffffffll ||
        (int64_t)(b2 - 1) * ks[1] * 2 + 2 * D > 0xffffffffll) {
        set_error("monarch backward (right factor): k / v / dk / dv strides must be multiples of 8 elements and the pointers 16-byte aligned");
        return SFM_ERR_STRIDE;
    }
    RightArgs a;
    a.kk = (const char*)kk; a.rb = (const char*)rb;
    a.v = (const char*)v; a.vs0 = vs[0]; a.vs1 = vs[1]; a.vs2 = vs[2];
    a.ks0 = ks[0]; a.ks1 = ks[1]; a.ks2 = ks[2];
    a.dkbar = (const char*)dkbar; a.dy = (const char*)dy;
    a.dc = dc;
    a.q = (const char*)q; a.qs0 = qs[0]; a.qs1 = qs[1]; a.qs2 = qs[2];
    a.qmap = qmap;
    a.ds1 = (uint16_t*)ds1;
    a.dk = (uint16_t*)dk; a.dv = (uint16_t*)dv;
    a.s0 = dks[0]; a.s1 = dks[1]; a.s2 = dks[2]; a.row0 = row0;
    a.kmap = kmap;
    a.b1 = b1; a.b2 = b2; a.AJ = AJ; a.nf = nf; a.H = H; a.unit0 = unit0; a.f0 = f0; a.f1 = f1;
    a.scale = scale;
    const size_t kv = (size_t)2 * 64 * 2 * D, rt = (size_t)kMaxAJ * 128;
    const size_t ldsb = kv + (size_t)2 * kMaxAJ * 2 * D + rt + (rt <= kv && AJ <= kMaxAJ ? 0 : rt) + 2 * kMaxAJ * 4;
    const int np = (AJ + kMaxAJ - 1) / kMaxAJ;                         // 1, 2 or 3 (monarch_bwd_right_supported)
    const void* fn = nullptr;
#define SFM_RIGHT_FN(E, D) \
    (np == 1 ? (const void*)monarch_bwd_right_kernel<E, D, 1> : np == 2 ? (const void*)monarch_bwd_right_kernel<E, D, 2> : (const void*)monarch_bwd_right_kernel<E, D, 3>)
    if (dtype == SFM_BF16) fn = D == 128 ? SFM_RIGHT_FN(BF16, 128) : SFM_RIGHT_FN(BF16, 64);
    else fn = D == 128 ? SFM_RIGHT_FN(F16, 128) : SFM_RIGHT_FN(F16, 64);
#undef SFM_RIGHT_FN
    if (ldsb > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)ldsb);
        if (e != hipSuccess) {
            set_error("monarch backward (right factor): cannot reserve %zu bytes of LDS: %s", ldsb, hipGetErrorString(e));
            return SFM_ERR_HIP;
        }
    }
    const dim3 grid((unsigned)ntiles);
    void* kargs[] = {(void*)&a};
    hipError_t le = hipLaunchKernel(fn, grid, dim3(kThreads), kargs, ldsb, stream);
    if (le != hipSuccess) {
        set_error("monarch backward (right factor): launch failed: %s", hipGetErrorString(le));
        return SFM_ERR_HIP;
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        set_error("monarch backward (right factor): launch failed: %s", hipGetErrorString(e));
        return SFM_ERR_HIP;
    }
    return SFM_OK;
}

// at most 16 waves of 32 columns each
bool monarch_bwd_dqk_supported(int dtype, int D, int b2, int AJ) {
    return (dtype == SFM_BF16 || dtype == SFM_F16) && (D == 64 || D == 128) && b2 % 4 == 0 && AJ <= 512;
}

int launch_monarch_bwd_dqk(int dtype, int D, int64_t nuk, int b1, int b2, int AJ, int nf, float scale, const void* k, const int64_t* ks,
                           const TokMap& kmap, const void* ds1, float* dqk, int H, int unit0, hipStream_t stream) {
    if ((ks[0] | ks[1] | ks[2]) % 8 || ((uintptr_t)k) % 16 || (int64_t)nf * b1 * b2 * ks[1] * 2 > 0xffffffffll) {
        set_error("monarch backward (dQ of the right factor): k rows must be 16-byte aligned and a (batch, head) slice under 4 GiB");
        return SFM_ERR_STRIDE;
    }
    DqkArgs a;
    a.k = (const char*)k; a.ks0 = ks[0]; a.ks1 = ks[1]; a.ks2 = ks[2];
    a.kmap = kmap;
    a.ds1 = (const uint16_t*)ds1;
    a.dqk = dqk;
    a.b1 = b1; a.b2 = b2; a.AJ = AJ; a.nf = nf; a.H = H; a.unit0 = unit0;
    a.scale = scale;
    const int nwaves = (AJ + 31) / 32;
    const size_t ldsb = (size_t)2 * 64 * 2 * D;
    const dim3 grid((unsigned)nuk), block((unsigned)(64 * nwaves));
    if (dtype == SFM_BF16) {
        if (D == 128) hipLaunchKernelGGL((monarch_bwd_dqk_kernel<BF16, 128>), grid, block, ldsb, stream, a);
        else hipLaunchKernelGGL((monarch_bwd_dqk_kernel<BF16, 64>), grid, block, ldsb, stream, a);
    } else {
        if (D == 128) hipLaunchKernelGGL((monarch_bwd_dqk_kernel<F16, 128>), grid, block, ldsb, stream, a);
        else hipLaunchKernelGGL((monarch_bwd_dqk_kernel<F16, 64>), grid, block, ldsb, stream, a);
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        set_error("monarch backward (dQ of the right factor): launch failed: %s", hipGetErrorString(e));
        return SFM_ERR_HIP;
    }
    return SFM_OK;
}

}  // namespace sfm
