// Backward of the dense attention on gfx950 MFMA (bf16 / fp16, head_dim 64 or 128).
//
// Replaces `_attn_bwd_preprocess`, `_attn_bwd` and their orchestration in `_attention.backward`
// (wan/modules/attn_patch.py:121-166, 169-302, 354-413).  With P = softmax(s q k^T) recomputed from the forward's
// log-sum-exp, delta_i = dO_i . O_i and dS = P (dO v^T - delta):
//     dQ = s dS k      dK = s dS^T q      dV = P^T dO
// The reference accumulates dQ with float atomics from a grid over key blocks; here dQ has its own kernel (a grid
// over query blocks, looping over the keys) and dK / dV theirs (a grid over key blocks, looping over the queries), so
// that no sum crosses workgroups.  Both recompute the logits and dP, 9 block products in all instead of 5.
//
// Both kernels keep their own 32 rows as the B operand of the logits in registers and stream the other side through
// LDS in tiles of 64 rows (global_load_lds_dwordx4, double buffered, 16-byte chunks XOR-swizzled per row): the logits
// come out transposed, [streamed row, own row], one own row per lane, which is directly the B operand of the gradient
// products whose A operands are transposing LDS reads (ds_read_tr16_b64) of the streamed tile.
//   dq kernel:  own = 32 queries per wave (4 waves, 128 queries per workgroup), streamed = K and V tiles.
//   dkv kernel: own = 32 keys per wave (4 waves, 128 keys per workgroup), streamed = q and dO tiles plus the tile's
//               log-sum-exp and delta values; three tiles in LDS, one wave per SIMD.

#include <hip/hip_runtime.h>

#include <type_traits>

#include "sfm_attn.h"
#include "sfm_common.hpp"

namespace sfm {
namespace {

struct DenseBwdArgs {
    const char *q, *k, *v, *out, *dout;
    const float* lse;        // [B][H][Sq], natural log
    float* lse2;             // [B][H][Sq], the same in base-2 units (scratch)
    float* delta;            // [B][H][Sq] (scratch)
    float* dq;
    char *dk, *dv;
    int64_t qs[3], ks[3], vs[3], os[3], dqs[3], dks[3];      // batch, token, head; in elements
    int B, H, Sq, Skv;
    int kv0, kv1;            // keys whose dK / dV are produced
    float scale;
};

typedef short db_s16x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ u32x2 db_read_tr(const char* lds, uint32_t off) {
    db_s16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((db_s16x4 __attribute__((address_space(3)))*)(lds + off));
    return __builtin_bit_cast(u32x2, v);
}
__device__ __forceinline__ void db_load_lds16(const char* base, uint32_t off, uint32_t lds_addr) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_addr), "v"(off), "s"(base) : "memory", "m0");
}
__device__ __forceinline__ void db_load_lds4(const float* base, uint32_t off, uint32_t lds_addr) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2" ::"s"(lds_addr), "v"(off), "s"(base) : "memory", "m0");
}
// chunk c (16 bytes) of row r sits at chunk position c ^ swz(r); depends on r mod 16 only
template <int CPR>
__device__ __forceinline__ int db_swz(int r) {
    return CPR >= 16 ? (((r & 3) << 2) | ((r >> 2) & 3)) : ((((r >> 1) & 1) << 2) | ((r >> 2) & 3));
}

// delta[b][h][i] = dO_i . O_i (16-byte chunks, D / 8 consecutive lanes per row) and the log-sum-exp in base-2 units
template <class E, int D>
__global__ __launch_bounds__(256) void dense_bwd_delta_kernel(DenseBwdArgs p) {
    constexpr int CH = D / 8, RPB = 256 / CH;
    const int tid = threadIdx.x, ch = tid % CH;
    const int64_t total = (int64_t)p.B * p.H * p.Sq;
    const int64_t row = (int64_t)blockIdx.x * RPB + tid / CH;
    float dot = 0.f;
    if (row < total) {
        const int i = (int)(row % p.Sq);
        const int64_t bh = row / p.Sq;
        const int h = (int)(bh % p.H);
        const int64_t b = bh / p.H;
        const int64_t off = (b * p.os[0] + (int64_t)i * p.os[1] + (int64_t)h * p.os[2]) * 2 + ch * 16;
        const u32x4 o = *(const u32x4*)(p.out + off), g = *(const u32x4*)(p.dout + off);
#pragma unroll
        for (int e = 0; e < 4; ++e)
            dot += E::to_float((uint16_t)(o[e] & 0xffffu)) * E::to_float((uint16_t)(g[e] & 0xffffu)) +
                   E::to_float((uint16_t)(o[e] >> 16)) * E::to_float((uint16_t)(g[e] >> 16));
    }
#pragma unroll
    for (int o = 1; o < CH; o <<= 1) dot += __shfl_xor(dot, o);
    if (ch == 0 && row < total) {
        p.delta[row] = dot;
        p.lse2[row] = p.lse[row] * kLog2e;
    }
}

// Shared pieces of the two kernels.  A tile is 64 rows of D elements, row pitch 2 D bytes.
template <int D>
struct Tile {
    static constexpr int DS = D / 16, DT = D / 32, CPR = D / 8, kPitch = 2 * D, kBytes = 64 * kPitch;
};

// logits of the tile's rows 32 tl + 0..31 against the wave's own rows: A = tile rows, B = own rows (registers)
template <class E, int D>
__device__ __forceinline__ void tile_products(const char* ta, const char* tb, uint32_t a_off, const u32x4 (&oa)[D / 16],
                                              const u32x4 (&ob)[D / 16], f32x16 (&s)[2], f32x16 (&d)[2]) {
    using T = Tile<D>;
#pragma unroll
    for (int tl = 0; tl < 2; ++tl)
#pragma unroll
        for (int v = 0; v < 16; ++v) s[tl][v] = d[tl][v] = 0.f;
#pragma unroll
    for (int ds = 0; ds < T::DS; ++ds)
#pragma unroll
        for (int tl = 0; tl < 2; ++tl) {
            const u32x4 xa = *(const u32x4*)(ta + tl * 32 * T::kPitch + (a_off ^ (uint32_t)(ds << 5)));
            const u32x4 xb = *(const u32x4*)(tb + tl * 32 * T::kPitch + (a_off ^ (uint32_t)(ds << 5)));
            s[tl] = E::mfma32(xa, oa[ds], s[tl]);
            d[tl] = E::mfma32(xb, ob[ds], d[tl]);
        }
}

// 16 accumulator values (streamed rows 8 g + 4 hf + e of a 32-row half) -> the B operands of the two 16-row steps
template <class E>
__device__ __forceinline__ void pack_steps(const f32x16& x, u32x4& lo, u32x4& hi) {
    lo.x = pack2<E>(x[0], x[1]); lo.y = pack2<E>(x[2], x[3]); lo.z = pack2<E>(x[4], x[5]); lo.w = pack2<E>(x[6], x[7]);
    hi.x = pack2<E>(x[8], x[9]); hi.y = pack2<E>(x[10], x[11]); hi.z = pack2<E>(x[12], x[13]); hi.w = pack2<E>(x[14], x[15]);
}

// A operand [m = head-dim 32 dt + lane % 32, k = the 16 rows of step st in accumulator order] of a tile, transposed
template <int D>
__device__ __forceinline__ u32x4 tile_tr(const char* tile, uint32_t tr_lo, uint32_t tr_hi, int st) {
    const u32x2 lo = db_read_tr(tile, tr_lo + st * 16 * Tile<D>::kPitch);
    const u32x2 hi = db_read_tr(tile, tr_hi + st * 16 * Tile<D>::kPitch);
    return u32x4{lo.x, lo.y, hi.x, hi.y};
}

template <class E, int D>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void dense_bwd_dq_kernel(DenseBwdArgs p) {
    using T = Tile<D>;
    extern __shared__ __attribute__((aligned(256))) char lds[];          // [buffer][K tile | V tile]
    const uint32_t lds0 = (uint32_t)(size_t)(__attribute__((address_space(3))) char*)lds;
    const int tid = threadIdx.x, lane = tid & 63, m = lane & 31, hf = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    // the query blocks of one (batch, head) go to one XCD, which then fetches that head's K / V rows once
    const int nblk = (p.Sq + 127) / 128;
    const int item = xcd_item(nblk * p.B * p.H);
    if (item >= nblk * p.B * p.H) return;
    const int bh = item / nblk, b = bh / p.H, h = bh % p.H;
    const int i = (item - bh * nblk) * 128 + wave * 32 + m;
    const int ic = min(i, p.Sq - 1);

    const char* qrow = p.q + ((int64_t)b * p.qs[0] + (int64_t)ic * p.qs[1] + (int64_t)h * p.qs[2]) * 2 + 16 * hf;
    const char* grow = p.dout + ((int64_t)b * p.os[0] + (int64_t)ic * p.os[1] + (int64_t)h * p.os[2]) * 2 + 16 * hf;
    u32x4 qb[T::DS], gb[T::DS];
#pragma unroll
    for (int ds = 0; ds < T::DS; ++ds) {
        qb[ds] = *(const u32x4*)(qrow + 32 * ds);
        gb[ds] = *(const u32x4*)(grow + 32 * ds);
    }
    const float lse2 = p.lse2[(int64_t)bh * p.Sq + ic];
    const float dl = p.delta[(int64_t)bh * p.Sq + ic];
    const float sc2 = p.scale * kLog2e;

    const char* kbase = p.k + ((int64_t)b * p.ks[0] + (int64_t)h * p.ks[2]) * 2;
    const char* vbase = p.v + ((int64_t)b * p.vs[0] + (int64_t)h * p.vs[2]) * 2;
    const uint32_t krb = (uint32_t)(p.ks[1] * 2), vrb = (uint32_t)(p.vs[1] * 2);
    auto stage = [&](int t) {
        const uint32_t dst = lds0 + (uint32_t)(t & 1) * 2 * T::kBytes;
        for (int g = wave; g < T::CPR; g += 4) {
            const int P = g * 64 + lane;
            const int r = P / T::CPR, c = (P % T::CPR) ^ db_swz<T::CPR>(r);
            const uint32_t row = (uint32_t)min(64 * t + r, p.Skv - 1);      // rows past the end repeat the last key (masked below)
            db_load_lds16(kbase, row * krb + (uint32_t)c * 16, dst + (uint32_t)g * 1024);
            db_load_lds16(vbase, row * vrb + (uint32_t)c * 16, dst + T::kBytes + (uint32_t)g * 1024);
        }
    };
    const uint32_t a_off = (uint32_t)m * T::kPitch + (uint32_t)((hf ^ db_swz<T::CPR>(m)) << 4);
    uint32_t tr[T::DT][2];
    {
        const int s16 = lane & 15, g16 = lane >> 4;
        const int rl = 4 * hf + (s16 >> 2);
        const int cl = 2 * (g16 & 1) + ((s16 & 3) >> 1);
#pragma unroll
        for (int dt = 0; dt < T::DT; ++dt)
#pragma unroll
            for (int half = 0; half < 2; ++half) {
                const int r = rl + 8 * half;
                tr[dt][half] = (uint32_t)(r * T::kPitch + (((4 * dt + cl) ^ db_swz<T::CPR>(r)) << 4) + (s16 & 1) * 8);
            }
    }

    f32x16 acc[T::DT];
#pragma unroll
    for (int dt = 0; dt < T::DT; ++dt)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[dt][v] = 0.f;

    const int nt = (p.Skv + 63) / 64;
    // one tile; RAGGED (only the last tile can be) masks the keys past the end
    auto tile = [&](int t, auto ragged_c) {
        constexpr bool ragged = decltype(ragged_c)::value;
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();                                   // tile t is in LDS; every wave is done with tile t - 1
        if (t + 1 < nt) stage(t + 1);
        const char* kt = lds + (t & 1) * 2 * T::kBytes;
        const char* vt = kt + T::kBytes;
        // Four stages per tile, each a run of MFMAs with its A operands read two ahead (ring) and a slice of the softmax
        // backward of the half tile before it pinned beside every MFMA:
        //   1  logits and dP of keys 0..31           2  those of keys 32..63 | softmax backward of keys 0..31
        //   3  dQ^T += K^T dS of keys 0..31 | softmax backward of keys 32..63          4  dQ^T += K^T dS of keys 32..63
        constexpr int NA = 2 * T::DS, NO = 2 * T::DT;       // MFMAs of a half's products / of a half's output
        constexpr int VA = 16 / NA, VO = 16 / NO;           // values of the softmax backward beside each of them
        f32x16 s[2], dp[2];
        u32x4 pb[4], ring[4];
        auto read_prod = [&](int tl, int j) {               // j even: K rows for the logits, odd: V rows for dP
            return *(const u32x4*)(((j & 1) ? vt : kt) + tl * 32 * T::kPitch + (a_off ^ (uint32_t)((j >> 1) << 5)));
        };
        auto read_out = [&](int tl, int j) { return tile_tr<D>(kt, tr[j % T::DT][0], tr[j % T::DT][1], 2 * tl + j / T::DT); };
        auto soft = [&](int tl, int v) {
            float pv = fast_exp2(fmaf(s[tl][v], sc2, -lse2));
            if (ragged) pv = 64 * t + 32 * tl + 8 * (v >> 2) + 4 * hf + (v & 3) < p.Skv ? pv : 0.f;
            s[tl][v] = pv * (dp[tl][v] - dl);               // dS^T[l, i]
            if (v & 1) pb[2 * tl + (v >> 3)][(v >> 1) & 3] = pack2<E>(s[tl][v - 1], s[tl][v]);
        };
#pragma unroll
        for (int tl = 0; tl < 2; ++tl)
#pragma unroll
            for (int v = 0; v < 16; ++v) s[tl][v] = dp[tl][v] = 0.f;
        ring[0] = read_prod(0, 0);
        ring[1] = read_prod(0, 1);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int j = 0; j < NA; ++j) {                      // stage 1
            ring[(j + 2) % 4] = j + 2 < NA ? read_prod(0, j + 2) : read_prod(1, j + 2 - NA);
            if (j & 1) dp[0] = E::mfma32(ring[j % 4], gb[j >> 1], dp[0]);
            else s[0] = E::mfma32(ring[j % 4], qb[j >> 1], s[0]);
            __builtin_amdgcn_sched_barrier(0);
        }
#pragma unroll
        for (int j = 0; j < NA; ++j) {                      // stage 2
            ring[(NA + j + 2) % 4] = j + 2 < NA ? read_prod(1, j + 2) : read_out(0, j + 2 - NA);
            if (j & 1) dp[1] = E::mfma32(ring[(NA + j) % 4], gb[j >> 1], dp[1]);
            else s[1] = E::mfma32(ring[(NA + j) % 4], qb[j >> 1], s[1]);
#pragma unroll
            for (int v = VA * j; v < VA * (j + 1); ++v) soft(0, v);
            __builtin_amdgcn_sched_barrier(0);
        }
#pragma unroll
        for (int j = 0; j < NO; ++j) {                      // stage 3
            ring[(2 * NA + j + 2) % 4] = j + 2 < NO ? read_out(0, j + 2) : read_out(1, j + 2 - NO);
            acc[j % T::DT] = E::mfma32(ring[(2 * NA + j) % 4], pb[j / T::DT], acc[j % T::DT]);
#pragma unroll
            for (int v = VO * j; v < VO * (j + 1); ++v) soft(1, v);
            __builtin_amdgcn_sched_barrier(0);
        }
#pragma unroll
        for (int j = 0; j < NO; ++j) {                      // stage 4
            if (j + 2 < NO) ring[(2 * NA + NO + j + 2) % 4] = read_out(1, j + 2);
            acc[j % T::DT] = E::mfma32(ring[(2 * NA + NO + j) % 4], pb[2 + j / T::DT], acc[j % T::DT]);
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    stage(0);
    for (int t = 0; t + 1 < nt; ++t) tile(t, std::false_type{});
    if (p.Skv % 64) tile(nt - 1, std::true_type{});
    else tile(nt - 1, std::false_type{});
    if (i < p.Sq) {
        float* row = p.dq + (int64_t)b * p.dqs[0] + (int64_t)i * p.dqs[1] + (int64_t)h * p.dqs[2] + 4 * hf;
#pragma unroll
        for (int dt = 0; dt < T::DT; ++dt)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const f32x4 w = {acc[dt][4 * g + 0] * p.scale, acc[dt][4 * g + 1] * p.scale, acc[dt][4 * g + 2] * p.scale,
                                 acc[dt][4 * g + 3] * p.scale};
                *(f32x4*)(row + 32 * dt + 8 * g) = w;
            }
    }
}

// One wave per SIMD: the wave's K and V rows (64 registers), dK^T and dV^T of a full head dim (128) and two half tiles
// of logits and dP do not fit 256 registers, and with the MFMAs' operands read ahead and the softmax backward pinned
// beside them a second wave would add little.
template <class E, int D>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1))) void dense_bwd_dkv_kernel(DenseBwdArgs p) {
    using T = Tile<D>;
    constexpr int kBuf = 3;                                // tiles in LDS: the one in use and two on their way
    constexpr int oStat = kBuf * 2 * T::kBytes;            // [buffer][lse 64 floats | delta 64 floats | 128 unused]
    extern __shared__ __attribute__((aligned(256))) char lds[];          // [buffer][q tile | dO tile], then the row values
    const uint32_t lds0 = (uint32_t)(size_t)(__attribute__((address_space(3))) char*)lds;
    const int tid = threadIdx.x, lane = tid & 63, m = lane & 31, hf = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    // the key blocks of one (batch, head) go to one XCD, which then fetches that head's q / dO rows once
    const int nblk = (p.kv1 - p.kv0 + 127) / 128;
    const int item = xcd_item(nblk * p.B * p.H);
    if (item >= nblk * p.B * p.H) return;
    const int bh = item / nblk, b = bh / p.H, h = bh % p.H;
    const int l = p.kv0 + (item - bh * nblk) * 128 + wave * 32 + m;
    const int lc = min(l, p.kv1 - 1);

    const char* krow = p.k + ((int64_t)b * p.ks[0] + (int64_t)lc * p.ks[1] + (int64_t)h * p.ks[2]) * 2 + 16 * hf;
    const char* vrow = p.v + ((int64_t)b * p.vs[0] + (int64_t)lc * p.vs[1] + (int64_t)h * p.vs[2]) * 2 + 16 * hf;
    u32x4 kb[T::DS], vb[T::DS];
#pragma unroll
    for (int ds = 0; ds < T::DS; ++ds) {
        kb[ds] = *(const u32x4*)(krow + 32 * ds);
        vb[ds] = *(const u32x4*)(vrow + 32 * ds);
    }
    const float sc2 = p.scale * kLog2e;

    const char* qbase = p.q + ((int64_t)b * p.qs[0] + (int64_t)h * p.qs[2]) * 2;
    const char* gbase = p.dout + ((int64_t)b * p.os[0] + (int64_t)h * p.os[2]) * 2;
    const float* lsep = p.lse2 + (int64_t)bh * p.Sq;
    const float* dlp = p.delta + (int64_t)bh * p.Sq;
    const uint32_t qrb = (uint32_t)(p.qs[1] * 2), grb = (uint32_t)(p.os[1] * 2);
    // every wave issues the same number of loads per tile (T::CPR / 2 + 1), so that one count waits for a tile
    auto stage = [&](int t) {
        const uint32_t dst = lds0 + (uint32_t)(t % kBuf) * 2 * T::kBytes;
        for (int g = wave; g < T::CPR; g += 4) {
            const int P = g * 64 + lane;
            const int r = P / T::CPR, c = (P % T::CPR) ^ db_swz<T::CPR>(r);
            const uint32_t row = (uint32_t)min(64 * t + r, p.Sq - 1);       // rows past the end repeat the last query (masked below)
            db_load_lds16(qbase, row * qrb + (uint32_t)c * 16, dst + (uint32_t)g * 1024);
            db_load_lds16(gbase, row * grb + (uint32_t)c * 16, dst + T::kBytes + (uint32_t)g * 1024);
        }
        const uint32_t row = (uint32_t)min(64 * t + lane, p.Sq - 1);
        db_load_lds4((wave & 1) ? dlp : lsep, row * 4, lds0 + oStat + (uint32_t)(t % kBuf) * 1024 + (uint32_t)wave * 256);
    };
    const uint32_t a_off = (uint32_t)m * T::kPitch + (uint32_t)((hf ^ db_swz<T::CPR>(m)) << 4);
    uint32_t tr[T::DT][2];
    {
        const int s16 = lane & 15, g16 = lane >> 4;
        const int rl = 4 * hf + (s16 >> 2);
        const int cl = 2 * (g16 & 1) + ((s16 & 3) >> 1);
#pragma unroll
        for (int dt = 0; dt < T::DT; ++dt)
#pragma unroll
            for (int half = 0; half < 2; ++half) {
                const int r = rl + 8 * half;
                tr[dt][half] = (uint32_t)(r * T::kPitch + (((4 * dt + cl) ^ db_swz<T::CPR>(r)) << 4) + (s16 & 1) * 8);
            }
    }

    f32x16 dka[T::DT], dva[T::DT];
#pragma unroll
    for (int dt = 0; dt < T::DT; ++dt)
#pragma unroll
        for (int v = 0; v < 16; ++v) dka[dt][v] = dva[dt][v] = 0.f;

    const int nt = (p.Sq + 63) / 64;
    // one tile; RAGGED (only the last tile can be) masks the queries past the end
    auto tile = [&](int t, auto ragged_c) {
        constexpr bool ragged = decltype(ragged_c)::value;
        // tile t has landed when at most the loads of tile t + 1 are outstanding
        if (t + 1 < nt) {
            if (T::CPR == 16) asm volatile("s_waitcnt vmcnt(9)" ::: "memory");
            else asm volatile("s_waitcnt vmcnt(5)" ::: "memory");
        } else {
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        }
        __syncthreads();                                   // tile t is in LDS; every wave is done with tile t - 1
        if (t + 2 < nt) stage(t + 2);
        const char* qt = lds + (t % kBuf) * 2 * T::kBytes;
        const char* gt = qt + T::kBytes;
        const char* st_ = lds + oStat + (t % kBuf) * 1024;

        // Four stages per tile as in the dq kernel; lane = key, registers = queries:
        //   1  S, dP of queries 0..31            2  those of queries 32..63 | softmax backward of queries 0..31
        //   3  dV^T += dO^T P, dK^T += q^T dS of queries 0..31 | softmax backward of queries 32..63      4  the same of queries 32..63
        constexpr int NA = 2 * T::DS, NO = 4 * T::DT;
        constexpr int VA = 16 / NA > 0 ? 16 / NA : 1, VO = 16 / NO > 0 ? 16 / NO : 1;
        f32x16 s[2], dp[2];
        constexpr int kAhead = 4, kRing = 8;                // A operands read this many MFMAs ahead
        u32x4 pb[4], sb[4], ring[kRing];
        auto read_prod = [&](int tl, int j) {               // j even: q rows for S, odd: dO rows for dP
            return *(const u32x4*)(((j & 1) ? gt : qt) + tl * 32 * T::kPitch + (a_off ^ (uint32_t)((j >> 1) << 5)));
        };
        // output MFMA j of a half: step st = 2 tl + j / (2 DT), head-dim block dt = (j / 2) % DT, j even: dV (dO^T), odd: dK (q^T)
        auto read_out = [&](int tl, int j) {
            const int dt = (j >> 1) % T::DT;
            return tile_tr<D>((j & 1) ? qt : gt, tr[dt][0], tr[dt][1], 2 * tl + j / (2 * T::DT));
        };
        f32x4 ls4, dl4;                                     // row values of the four queries v & ~3 .. + 3
        auto soft = [&](int tl, int v) {
            const int r = 32 * tl + 8 * (v >> 2) + 4 * hf + (v & 3);
            if ((v & 3) == 0) {
                ls4 = *(const f32x4*)(st_ + r * 4);
                dl4 = *(const f32x4*)(st_ + 256 + r * 4);
            }
            float pv = fast_exp2(fmaf(s[tl][v], sc2, -ls4[v & 3]));
            if (ragged) pv = 64 * t + r < p.Sq ? pv : 0.f;
            s[tl][v] = pv;
            dp[tl][v] = pv * (dp[tl][v] - dl4[v & 3]);
            if (v & 1) {
                pb[2 * tl + (v >> 3)][(v >> 1) & 3] = pack2<E>(s[tl][v - 1], s[tl][v]);
                sb[2 * tl + (v >> 3)][(v >> 1) & 3] = pack2<E>(dp[tl][v - 1], dp[tl][v]);
            }
        };
        auto out_mfma = [&](int tl, int j, const u32x4& a) {
            const int dt = (j >> 1) % T::DT, st = 2 * tl + j / (2 * T::DT);
            if (j & 1) dka[dt] = E::mfma32(a, sb[st], dka[dt]);
            else dva[dt] = E::mfma32(a, pb[st], dva[dt]);
        };
#pragma unroll
        for (int tl = 0; tl < 2; ++tl)
#pragma unroll
            for (int v = 0; v < 16; ++v) s[tl][v] = dp[tl][v] = 0.f;
#pragma unroll
        for (int j = 0; j < kAhead; ++j) ring[j] = read_prod(0, j);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int j = 0; j < NA; ++j) {                      // stage 1
            ring[(j + kAhead) % kRing] = j + kAhead < NA ? read_prod(0, j + kAhead) : read_prod(1, j + kAhead - NA);
            if (j & 1) dp[0] = E::mfma32(ring[j % kRing], vb[j >> 1], dp[0]);
            else s[0] = E::mfma32(ring[j % kRing], kb[j >> 1], s[0]);
            __builtin_amdgcn_sched_barrier(0);
        }
#pragma unroll
        for (int j = 0; j < NA; ++j) {                      // stage 2
            ring[(NA + j + kAhead) % kRing] = j + kAhead < NA ? read_prod(1, j + kAhead) : read_out(0, j + kAhead - NA);
            if (j & 1) dp[1] = E::mfma32(ring[(NA + j) % kRing], vb[j >> 1], dp[1]);
            else s[1] = E::mfma32(ring[(NA + j) % kRing], kb[j >> 1], s[1]);
#pragma unroll
            for (int v = VA * j; v < VA * (j + 1) && v < 16; ++v) soft(0, v);
            __builtin_amdgcn_sched_barrier(0);
        }
#pragma unroll
        for (int j = 0; j < NO; ++j) {                      // stage 3
            ring[(2 * NA + j + kAhead) % kRing] = j + kAhead < NO ? read_out(0, j + kAhead) : read_out(1, j + kAhead - NO);
            out_mfma(0, j, ring[(2 * NA + j) % kRing]);
#pragma unroll
            for (int v = VO * j; v < VO * (j + 1) && v < 16; ++v) soft(1, v);
            __builtin_amdgcn_sched_barrier(0);
        }
#pragma unroll
        for (int j = 0; j < NO; ++j) {                      // stage 4
            if (j + kAhead < NO) ring[(2 * NA + NO + j + kAhead) % kRing] = read_out(1, j + kAhead);
            out_mfma(1, j, ring[(2 * NA + NO + j) % kRing]);
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    stage(0);
    if (nt > 1) stage(1);
    for (int t = 0; t + 1 < nt; ++t) tile(t, std::false_type{});
    if (p.Sq % 64) tile(nt - 1, std::true_type{});
    else tile(nt - 1, std::false_type{});
    // lane (key, hf) holds head-dim 32 dt + 8 g + 4 hf + 0..3; the half swap leaves 8 consecutive ones per lane
    const int64_t obase = ((int64_t)b * p.dks[0] + (int64_t)(lc - p.kv0) * p.dks[1] + (int64_t)h * p.dks[2]) * 2;
    auto store = [&](char* dst, const f32x16& a, int dt, float sc) {
#pragma unroll
        for (int gp = 0; gp < 2; ++gp) {
            const int g0 = 8 * gp, g1 = 8 * gp + 4;
            auto rx = __builtin_amdgcn_permlane32_swap(pack2<E>(a[g0 + 0] * sc, a[g0 + 1] * sc), pack2<E>(a[g1 + 0] * sc, a[g1 + 1] * sc), false, false);
            auto ry = __builtin_amdgcn_permlane32_swap(pack2<E>(a[g0 + 2] * sc, a[g0 + 3] * sc), pack2<E>(a[g1 + 2] * sc, a[g1 + 3] * sc), false, false);
            const u32x4 w = {(uint32_t)rx[0], (uint32_t)ry[0], (uint32_t)rx[1], (uint32_t)ry[1]};
            if (l < p.kv1) *(u32x4*)(dst + obase + (32 * dt + 16 * gp + 8 * hf) * 2) = w;
        }
    };
#pragma unroll
    for (int dt = 0; dt < T::DT; ++dt) {
        store(p.dk, dka[dt], dt, p.scale);
        store(p.dv, dva[dt], dt, 1.f);
    }
}

template <class E, int D>
int launch_t(const DenseBwdArgs& a, hipStream_t stream) {
    using T = Tile<D>;
    const int64_t rows = (int64_t)a.B * a.H * a.Sq;
    constexpr int RPB = 256 / (D / 8);
    hipLaunchKernelGGL((dense_bwd_delta_kernel<E, D>), dim3((unsigned)((rows + RPB - 1) / RPB)), dim3(256), 0, stream, a);
    const size_t lds_dq = 4 * T::kBytes, lds_dkv = 6 * T::kBytes + 3 * 1024;
    if (lds_dkv > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute((const void*)dense_bwd_dkv_kernel<E, D>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_dkv);
        if (e == hipSuccess)
            e = hipFuncSetAttribute((const void*)dense_bwd_dq_kernel<E, D>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_dq);
        if (e != hipSuccess) {
            set_error("dense backward: cannot reserve %zu bytes of LDS: %s", lds_dkv, hipGetErrorString(e));
            return SFM_ERR_HIP;
        }
    }
    hipLaunchKernelGGL((dense_bwd_dq_kernel<E, D>), dim3(xcd_grid((a.Sq + 127) / 128 * a.B * a.H)), dim3(256), lds_dq, stream, a);
    if (a.kv1 > a.kv0)
        hipLaunchKernelGGL((dense_bwd_dkv_kernel<E, D>), dim3(xcd_grid((a.kv1 - a.kv0 + 127) / 128 * a.B * a.H)), dim3(256), lds_dkv, stream, a);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        set_error("dense backward: launch failed: %s", hipGetErrorString(e));
        return SFM_ERR_HIP;
    }
    return SFM_OK;
}

}  // namespace

bool dense_bwd_supported(int dtype, int D) { return (dtype == SFM_BF16 || dtype == SFM_F16) && (D == 64 || D == 128); }

int launch_dense_bwd(const sfm_dense_desc& d, const int64_t* dq_stride, const int64_t* dkv_stride, int64_t kv0, int64_t kv1,
                     const void* q, const void* k, const void* v, const void* out, const float* lse, const void* dout, float* dq,
                     void* dk, void* dv, float* scratch, hipStream_t stream) {
    if (!dense_bwd_supported(d.dtype, d.D)) {
        set_error("dense backward: bf16 / fp16 tensors with head_dim 64 or 128 only");
        return SFM_ERR_UNSUPPORTED;
    }
    DenseBwdArgs a;
    a.q = (const char*)q; a.k = (const char*)k; a.v = (const char*)v; a.out = (const char*)out; a.dout = (const char*)dout;
    a.lse = lse; a.delta = scratch; a.lse2 = scratch + (int64_t)d.B * d.H * d.q_tokens; a.dq = dq; a.dk = (char*)dk; a.dv = (char*)dv;
    int64_t bad = 0;
    for (int i = 0; i < 3; ++i) {
        a.qs[i] = d.q_stride[i]; a.ks[i] = d.k_stride[i]; a.vs[i] = d.v_stride[i]; a.os[i] = d.o_stride[i];
        a.dqs[i] = dq_stride[i]; a.dks[i] = dkv_stride[i];
        bad |= (a.qs[i] | a.ks[i] | a.vs[i] | a.os[i] | a.dks[i]) % 8 | a.dqs[i] % 4;
    }
    if (bad) {
        set_error("dense backward: strides must keep every row 16-byte aligned");
        return SFM_ERR_STRIDE;
    }
    const int64_t lim = (int64_t)1 << 32;
    if ((int64_t)d.kv_tokens * d.k_stride[1] * 2 >= lim || (int64_t)d.kv_tokens * d.v_stride[1] * 2 >= lim ||
        (int64_t)d.q_tokens * d.q_stride[1] * 2 >= lim || (int64_t)d.q_tokens * d.o_stride[1] * 2 >= lim) {
        set_error("dense backward: a (batch, head) slice of q, k, v or dout spans 4 GiB or more");
        return SFM_ERR_UNSUPPORTED;
    }
    a.B = d.B; a.H = d.H; a.Sq = d.q_tokens; a.Skv = d.kv_tokens;
    a.kv0 = (int)kv0; a.kv1 = (int)kv1;
    a.scale = d.sm_scale;
    if (d.dtype == SFM_BF16) return d.D == 128 ? launch_t<BF16, 128>(a, stream) : launch_t<BF16, 64>(a, stream);
    return d.D == 128 ? launch_t<F16, 128>(a, stream) : launch_t<F16, 64>(a, stream);
}

}  // namespace sfm
