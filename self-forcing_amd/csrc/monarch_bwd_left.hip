// Left-factor part of the Monarch backward on gfx950 MFMA (bf16 / fp16, head_dim 64 or 128, block rows b1 <= 128).
//
// Replaces, inside the backward of the two-step attention, the per-(a, j) products and row kernels
//     S2 = q_i . Kbar_r,  dLm = dO_i . Y_r,  L = softmax_r(s S2 - c),  dS2 = L (dLm - sum_r L dLm),
//     dc_r = - sum_i dS2,  dY_r = sum_i L dO_i,  dKbar_r = s sum_i dS2 q_i
// (wan/modules/monarch_attn.py:852-886 `_z_bwd_preprocess`, :1034-1222 `_z_bwd`) with one kernel that never writes
// the [i x r] matrices S2, dLm, L.  dS2 is still written (16 bit) because the product dQ = s dS2 Kbar contracts over
// r and stays a batched library GEMM.
//
// One wave per (unit, a, j); its b1 query rows and their dO rows sit in LDS, the r = (k, f) rows of Kbar and Y stream
// from global memory 32 at a time (through the wave's own part of LDS, global_load_lds_dwordx4), twice: pass 1 for the softmax statistics (row maximum, sum, and sum of L dLm, kept
// per lane and merged across lanes once at the end), pass 2 for the gradients.  Logits are computed as
// S2[i, r] (A = query rows, B = Kbar rows), so that a lane owns one r and holds 16 of the i: the accumulator layout
// is then directly the B operand [n = r, k = i] of dY^T = dO^T L and dKbar^T = s Q^T dS2, whose A operands are
// transposing LDS reads of the dO / Q rows, and dc is an in-lane sum.
//
// More than 32 block rows (three frames tied per block: b1 = 90) run one grid slice per 32-row tile of the query rows
// (blockIdx.z): a slice owns its rows' statistics and dS2 rows, and writes its own partial dKbar / dY / dc (sums over
// its i) into a slab of its own; monarch_bwd_left_sum_kernel adds the slabs into the first one.

#include <hip/hip_runtime.h>

#include <type_traits>

#include "sfm_attn.h"
#include "sfm_common.hpp"

namespace sfm {
namespace {

struct LeftArgs {
    const char* q;           // callers' tensors: row i of (unit, a, j) is token qmap.row(a, i) + j; strides batch, token, head
    const char* dout;        // (in elements); out, optional, shares dout's strides
    const char* out;
    int64_t qs[3], os[3];
    TokMap qmap;
    int H;
    const uint16_t* kbar;    // row r of (u, aj) at ((u * RR + r) * AJ + aj) * D
    const uint16_t* y;
    const float* c;          // c_rows == 0: [u][aj][RR], natural log units; c_rows == 1: [(u * RR + r) * AJ + aj], log2 units
    int c_rows;
    uint16_t* dkbar;         // like kbar
    uint16_t* dy;
    float* dc;               // [u][aj][RR]
    uint16_t* ds2;           // [u][aj][b1][ds2_ld], ds2_ld >= RR
    int ds2_ld;
    const float* stats;      // optional, with out:      // log2-sum-exp of the logits of row (unit, aj, i) at ((unit0 + u) * AJ + aj) * stats_ld + i
    int stats_ld, unit0;
    int b1, b2, AJ, nf, RR, causal;
    float scale;
    int64_t slab_rows, slab_dc;   // elements between the dkbar / dy slabs and between the dc slabs of two query-row tiles
    int nunits, nz;               // units of this launch, 32-row query slices per column
};

typedef short bl_s16x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ u32x2 bl_read_tr(const char* lds, uint32_t off) {
    bl_s16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((bl_s16x4 __attribute__((address_space(3)))*)(lds + off));
    return __builtin_bit_cast(u32x2, v);
}

template <int CPR>
__device__ __forceinline__ int bl_swz(int r) {
    return CPR >= 16 ? (((r & 3) << 2) | ((r >> 2) & 3)) : ((((r >> 1) & 1) << 2) | ((r >> 2) & 3));
}
__device__ __forceinline__ void bl_load_lds16(const char* base, uint32_t off, uint32_t lds_addr) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_addr), "v"(off), "s"(base) : "memory", "m0");
}
// the same with the LDS address as a scalar base plus a compile-time offset (one scalar register for all of a chunk's loads)
template <int OFF>
__device__ __forceinline__ void bl_load_lds16_at(const char* base, uint32_t off, uint32_t lds_base) {
    asm volatile("s_add_u32 m0, %0, %3\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_base), "v"(off), "s"(base), "n"(OFF) : "memory", "m0", "scc");
}
template <int OFF>
__device__ __forceinline__ void bl_load_lds4_at(const char* base, uint32_t off, uint32_t lds_base) {
    asm volatile("s_add_u32 m0, %0, %3\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2" ::"s"(lds_base), "v"(off), "s"(base), "n"(OFF) : "memory", "m0", "scc");
}

// LDS per wave: q rows, dO rows, 32 floats, then the chunk being loaded: 32 Kbar rows, 32 Y rows (row-major, 16-byte
// pieces XOR-swizzled per row) and their 32 c values (twice)
template <int D>
struct LeftLds {
    static constexpr int kPitch = (D + 8) * 2;            // bytes per staged q / dO row
    static constexpr int kRows = 2 * 32 * kPitch + 128;
    static constexpr int kTile = 32 * 2 * D;
    static constexpr int kPerWave = (kRows + 2 * kTile + 256 + 255) / 256 * 256;
};

template <class E, int D>
__global__ __launch_bounds__(256) void monarch_bwd_left_kernel(LeftArgs p) {
    constexpr int DS = D / 16, DT = D / 32, CPR = D / 8;
    constexpr int kPitch = LeftLds<D>::kPitch;
    constexpr int kPerWave = LeftLds<D>::kPerWave;
    constexpr int kTile = LeftLds<D>::kTile;
    extern __shared__ __attribute__((aligned(256))) char lds[];

    const int tid = threadIdx.x, lane = tid & 63, m = lane & 31, hf = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    // work item = (unit, group of 4 columns, slice), slices fastest, one contiguous range of items per XCD: the slices
    // of a column, which stream the same Kbar / Y rows, meet in one L2
    const int njg = (p.AJ + 3) / 4;
    const int item = xcd_item(njg * p.nunits * p.nz);
    if (item >= njg * p.nunits * p.nz) return;
    const int zi = item % p.nz, jg = (item / p.nz) % njg;
    const int ajraw = jg * 4 + wave;
    const bool aj_ok = ajraw < p.AJ;
    const int aj = aj_ok ? ajraw : p.AJ - 1;              // a wave past the end repeats the last column and stores nothing
    const int u = item / (p.nz * njg);
    const int i0 = zi * 32;                               // first query row of this slice
    const int RR = p.RR, b1 = p.b1;
    const int64_t uaj = (int64_t)u * p.AJ + aj;

    char* qs = lds + wave * kPerWave;
    char* dos = qs + 32 * kPitch;
    float* dls = (float*)(dos + 32 * kPitch);
    const bool saved = p.stats != nullptr;                // uniform: the forward's output and row statistics are at hand
    {
        const int unit = p.unit0 + u, bb = unit / p.H, hh = unit % p.H;
        const int a_q = aj / p.b2, j_q = aj % p.b2;
        const char* qg = p.q + ((int64_t)bb * p.qs[0] + (int64_t)hh * p.qs[2]) * 2;
        const char* dg = p.dout + ((int64_t)bb * p.os[0] + (int64_t)hh * p.os[2]) * 2;
        const char* og = saved ? p.out + ((int64_t)bb * p.os[0] + (int64_t)hh * p.os[2]) * 2 : dg;
        constexpr int CH = D / 8;
        for (int cidx = lane; cidx < 32 * CH; cidx += 64) {
            const int r = cidx / CH, ch = cidx % CH;
            u32x4 a = {0u, 0u, 0u, 0u}, b = a;
            float dot = 0.f;
            if (i0 + r < b1) {
                const int64_t tok = p.qmap.row(a_q, i0 + r) + j_q;
                a = *(const u32x4*)(qg + tok * p.qs[1] * 2 + ch * 16);
                b = *(const u32x4*)(dg + tok * p.os[1] * 2 + ch * 16);
                if (saved) {                              // sum_r L dLm of row i is dO_i . O_i
                    const u32x4 o = *(const u32x4*)(og + tok * p.os[1] * 2 + ch * 16);
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        dot += E::to_float((uint16_t)(b[e] & 0xffffu)) * E::to_float((uint16_t)(o[e] & 0xffffu)) +
                               E::to_float((uint16_t)(b[e] >> 16)) * E::to_float((uint16_t)(o[e] >> 16));
                }
            }
            *(u32x4*)(qs + r * kPitch + ch * 16) = a;
            *(u32x4*)(dos + r * kPitch + ch * 16) = b;
            if (saved) {
#pragma unroll
                for (int o = 1; o < CH; o <<= 1) dot += __shfl_xor(dot, o);
                if (ch == 0) dls[r] = dot;
            }
        }
    }
    __syncthreads();

    const int a_blk = aj / p.b2;
    const int flim = p.causal ? min(p.nf, (a_blk / p.causal + 1) * p.causal) : p.nf;      // visible kv block-frames
    const int64_t rstride = (int64_t)p.AJ * D;                                           // elements between rows r, r + 1
    const uint16_t* kb = p.kbar + ((int64_t)u * RR * p.AJ + aj) * D;
    const uint16_t* yb = p.y + ((int64_t)u * RR * p.AJ + aj) * D;
    const float* cp = p.c_rows ? p.c + (int64_t)u * RR * p.AJ + aj : p.c + uaj * RR;
    const int64_t cstep = p.c_rows ? p.AJ : 1;
    const float cmul = p.c_rows ? 1.f : kLog2e;
    const float sc2 = p.scale * kLog2e;
    const int nch = (RR + 31) / 32;

    // A chunk of 32 rows r goes from global memory into the wave's LDS (global_load_lds_dwordx4: a row's 2 D bytes
    // by consecutive lanes) and from there into the operand registers; the chunk after it is requested as soon as the
    // registers are filled, and is waited for (with everything else this wave has in flight) before they are filled
    // again.  Nothing is shared between waves.
    char* const kt = qs + LeftLds<D>::kRows;
    const uint32_t kt0 = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(size_t)(__attribute__((address_space(3))) char*)kt);
    const char* const kbb = (const char*)kb;
    const char* const ybb = (const char*)yb;
    const char* const cpb = (const char*)cp;
    const uint32_t rsb = (uint32_t)(rstride * 2), csb = (uint32_t)(cstep * 4);
    auto request_piece = [&](int n, auto g_c) {
        constexpr int g = decltype(g_c)::value;
        const int P = g * 64 + lane;
        const int r = P / CPR, c = (P % CPR) ^ bl_swz<CPR>(r);
        const uint32_t off = (uint32_t)min(32 * n + r, RR - 1) * rsb + (uint32_t)c * 16;
        bl_load_lds16_at<g * 1024>(kbb, off, kt0);
        bl_load_lds16_at<kTile + g * 1024>(ybb, off, kt0);
    };
    auto request = [&](int n) {
        request_piece(n, std::integral_constant<int, 0>{});
        request_piece(n, std::integral_constant<int, 1>{});
        request_piece(n, std::integral_constant<int, 2>{});
        request_piece(n, std::integral_constant<int, 3>{});
        if constexpr (CPR / 2 > 4) {
            request_piece(n, std::integral_constant<int, 4>{});
            request_piece(n, std::integral_constant<int, 5>{});
            request_piece(n, std::integral_constant<int, 6>{});
            request_piece(n, std::integral_constant<int, 7>{});
        }
        bl_load_lds4_at<2 * kTile>(cpb, (uint32_t)min(32 * n + m, RR - 1) * csb, kt0);
    };
    const uint32_t b_off = (uint32_t)m * (2 * D) + (uint32_t)((hf ^ bl_swz<CPR>(m)) << 4);     // row m as a B operand
    u32x4 kcur[DS], ycur[DS];
    float ccur = 0.f;
    // fills the operand registers with the chunk that was requested last and requests chunk `next`
    auto load_tile = [&](int next) {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#pragma unroll
        for (int ds = 0; ds < DS; ++ds) {
            kcur[ds] = *(const u32x4*)(kt + (b_off ^ (uint32_t)(ds << 5)));
            ycur[ds] = *(const u32x4*)(kt + kTile + (b_off ^ (uint32_t)(ds << 5)));
        }
        ccur = *(const float*)(kt + 2 * kTile + m * 4) * cmul;
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");       // the registers are filled: the buffer may be overwritten
        if (next >= 0) request(next);
    };
    // logits S2[i, r] and dLm[i, r]: lane -> r = 32 n + m, register v -> i = 8 (v >> 2) + 4 hf + (v & 3)
    auto products = [&](f32x16& s, f32x16& d) {
#pragma unroll
        for (int v = 0; v < 16; ++v) s[v] = d[v] = 0.f;
#pragma unroll
        for (int ds = 0; ds < DS; ++ds) {
            const u32x4 qb = *(const u32x4*)(qs + m * kPitch + (16 * ds + 8 * hf) * 2);
            const u32x4 db = *(const u32x4*)(dos + m * kPitch + (16 * ds + 8 * hf) * 2);
            s = E::mfma32(qb, kcur[ds], s);
            d = E::mfma32(db, ycur[ds], d);
        }
    };
    auto row_ok = [&](int n) {
        const int r = 32 * n + m;
        return r < RR && (r % p.nf) < flim;
    };

    float lse[16], delta[16];
    if (saved) {
        const float* st = p.stats + ((int64_t)(p.unit0 + u) * p.AJ + aj) * p.stats_ld;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int i = 8 * (v >> 2) + 4 * hf + (v & 3);
            lse[v] = st[min(i0 + i, b1 - 1)];
            delta[v] = dls[i];
        }
    } else {
        // ---- pass 1: per lane, for its 16 rows i, the running maximum, sum and sum of L dLm over the lane's own r
        float mloc[16], lloc[16], dloc[16];
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            mloc[v] = -INFINITY;
            lloc[v] = dloc[v] = 0.f;
        }
        request(0);
        for (int n = 0; n < nch; ++n) {
            load_tile(n + 1 < nch ? n + 1 : -1);
            f32x16 s, d;
            products(s, d);
            const float cl2 = ccur;
            const bool ok = row_ok(n);
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const float z = ok ? s[v] * sc2 - cl2 : -INFINITY;
                const float mnew = fmaxf(mloc[v], z);
                const float mref = mnew == -INFINITY ? 0.f : mnew;
                const float alpha = fast_exp2(mloc[v] - mref), e = fast_exp2(z - mref);
                lloc[v] = lloc[v] * alpha + e;
                dloc[v] = dloc[v] * alpha + e * d[v];
                mloc[v] = mnew;
            }
        }
        // merge over the 32 lanes of a half (they hold the same rows i); every row has at least one visible r
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            float mm = mloc[v], ll = lloc[v], dd = dloc[v];
#pragma unroll
            for (int o = 1; o < 32; o <<= 1) {
                const float m2 = __shfl_xor(mm, o), l2 = __shfl_xor(ll, o), d2 = __shfl_xor(dd, o);
                const float mnew = fmaxf(mm, m2);
                const float mref = mnew == -INFINITY ? 0.f : mnew;
                const float a1 = fast_exp2(mm - mref), a2 = fast_exp2(m2 - mref);
                ll = ll * a1 + l2 * a2;
                dd = dd * a1 + d2 * a2;
                mm = mnew;
            }
            lse[v] = mm + log2f(ll);
            delta[v] = dd / ll;
        }
    }

    // ---- pass 2: gradients
    // transposing reads of the staged rows: lane (m, hf) gets, for head-dim column 32 dt + m, rows i = 16 ks + 4 hf +
    // {0..3} and + 8 + {0..3}, the order in which the packed accumulators hold i (two reads, see perm_row)
    uint32_t tr0, tr1;
    {
        const int s16 = lane & 15, g16 = lane >> 4;
        const int rl = 4 * hf + (s16 >> 2);
        const int cl = 2 * (g16 & 1) + ((s16 & 3) >> 1);
        tr0 = (uint32_t)(rl * kPitch + cl * 16 + (s16 & 1) * 8);
        tr1 = tr0 + 8 * kPitch;
    }
    uint16_t* const dkb = p.dkbar + zi * p.slab_rows + ((int64_t)u * RR * p.AJ + aj) * D;
    uint16_t* const dyb = p.dy + zi * p.slab_rows + ((int64_t)u * RR * p.AJ + aj) * D;
    float* const dcp = p.dc + zi * p.slab_dc + uaj * RR;
    uint16_t* const ds2p = p.ds2 + uaj * b1 * p.ds2_ld;

    request(0);
    for (int n = 0; n < nch; ++n) {
        load_tile(n + 1 < nch ? n + 1 : -1);
        f32x16 s, d;
        products(s, d);
        const float cl2 = ccur;
        const bool ok = row_ok(n);
        const int r = 32 * n + m;
        const bool r_in = r < RR;
        float dsum = 0.f;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const float pv = ok ? fast_exp2(s[v] * sc2 - cl2 - lse[v]) : 0.f;
            const float gv = pv * (d[v] - delta[v]);
            s[v] = pv;                                   // L[i, r]
            d[v] = gv;                                   // dS2[i, r]
            dsum += gv;
        }
        dsum = xhalf_sum(dsum);
        if (aj_ok && r_in && hf == 0) dcp[r] = -dsum;
        if (aj_ok && r_in) {
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int i = 8 * (v >> 2) + 4 * hf + (v & 3);
                if (i0 + i < b1) ds2p[(int64_t)(i0 + i) * p.ds2_ld + r] = E::from_float(d[v]);
            }
        }
        u32x4 pl[2], pg[2];                              // B operands [n = r, k = i] for the two steps of 16 rows i
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
            pl[ks].x = pack2<E>(s[8 * ks + 0], s[8 * ks + 1]); pl[ks].y = pack2<E>(s[8 * ks + 2], s[8 * ks + 3]);
            pl[ks].z = pack2<E>(s[8 * ks + 4], s[8 * ks + 5]); pl[ks].w = pack2<E>(s[8 * ks + 6], s[8 * ks + 7]);
            pg[ks].x = pack2<E>(d[8 * ks + 0], d[8 * ks + 1]); pg[ks].y = pack2<E>(d[8 * ks + 2], d[8 * ks + 3]);
            pg[ks].z = pack2<E>(d[8 * ks + 4], d[8 * ks + 5]); pg[ks].w = pack2<E>(d[8 * ks + 6], d[8 * ks + 7]);
        }
        // dY^T[d, r] = sum_i dO^T[d, i] L[i, r],  dKbar^T[d, r] = s sum_i Q^T[d, i] dS2[i, r], 32 head-dim rows at a time.
        // A lane (r, hf) holds head-dim 32 dt + 8 g + 4 hf + 0..3 of its row r.  A half swap (v_permlane32_swap) leaves 8
        // consecutive ones per lane; then, over a pair of head-dim blocks, lane bit 4 is traded for the piece pair
        // (v_permlane16_swap) and lane bit 3 for the block within the pair (a rotation by 8 within rows of 16 lanes),
        // after which a lane holds the 16-byte piece 4 (bit 3) + 2 (bit 4) + hf of the rows (r & 7) + 8 rb, rb = 0..3:
        // one store instruction writes 128 contiguous bytes of each of 8 rows.
        int64_t rowoff[4];
        bool row_in[4];
#pragma unroll
        for (int rb = 0; rb < 4; ++rb) {
            const int rr = 32 * n + (m & 7) + 8 * rb;
            row_in[rb] = aj_ok && rr < RR;
            rowoff[rb] = (int64_t)min(rr, RR - 1) * rstride + (4 * ((m >> 3) & 1) + 2 * ((m >> 4) & 1) + hf) * 8;
        }
#pragma unroll
        for (int which = 0; which < 2; ++which) {
            const char* src = which == 0 ? dos : qs;
            uint16_t* const obase = which == 0 ? dyb : dkb;
            const float osc = which == 0 ? 1.f : p.scale;
#pragma unroll
            for (int dp = 0; dp < DT / 2; ++dp) {
                uint32_t w[2][2][4];                     // [block in pair][gp][dword]
#pragma unroll
                for (int dl = 0; dl < 2; ++dl) {
                    const int dt = 2 * dp + dl;
                    f32x16 o;
#pragma unroll
                    for (int v = 0; v < 16; ++v) o[v] = 0.f;
#pragma unroll
                    for (int ks = 0; ks < 2; ++ks) {
                        const u32x2 lo = bl_read_tr(src, tr0 + ks * 16 * kPitch + dt * 64);
                        const u32x2 hi = bl_read_tr(src, tr1 + ks * 16 * kPitch + dt * 64);
                        const u32x4 aop = {lo.x, lo.y, hi.x, hi.y};
                        o = E::mfma32(aop, which == 0 ? pl[ks] : pg[ks], o);
                    }
#pragma unroll
                    for (int gp = 0; gp < 2; ++gp) {
                        const int g0 = 2 * gp, g1 = 2 * gp + 1;
                        auto rx = __builtin_amdgcn_permlane32_swap(pack2<E>(o[4 * g0 + 0] * osc, o[4 * g0 + 1] * osc),
                                                                   pack2<E>(o[4 * g1 + 0] * osc, o[4 * g1 + 1] * osc), false, false);
                        auto ry = __builtin_amdgcn_permlane32_swap(pack2<E>(o[4 * g0 + 2] * osc, o[4 * g0 + 3] * osc),
                                                                   pack2<E>(o[4 * g1 + 2] * osc, o[4 * g1 + 3] * osc), false, false);
                        w[dl][gp][0] = rx[0]; w[dl][gp][1] = ry[0]; w[dl][gp][2] = rx[1]; w[dl][gp][3] = ry[1];
                    }
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        auto x = __builtin_amdgcn_permlane16_swap(w[dl][0][q], w[dl][1][q], false, false);
                        w[dl][0][q] = x[0]; w[dl][1][q] = x[1];
                    }
                }
#pragma unroll
                for (int r4 = 0; r4 < 2; ++r4) {
                    u32x4 lo, hi;
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        const uint32_t x0 = w[0][r4][q], x1 = w[1][r4][q];
                        // row_ror:8 within 16 lanes; bank mask 0xc writes lanes 8..15 of a row, 0x3 lanes 0..7
                        lo[q] = (uint32_t)__builtin_amdgcn_update_dpp((int)x0, (int)x1, 0x128, 0xf, 0xc, false);
                        hi[q] = (uint32_t)__builtin_amdgcn_update_dpp((int)x1, (int)x0, 0x128, 0xf, 0x3, false);
                    }
                    // non-temporal: the rows are read once, by the right factor's kernel, after this grid has finished
                    if (row_in[2 * r4 + 0]) __builtin_nontemporal_store(lo, (u32x4*)(obase + rowoff[2 * r4 + 0] + 64 * dp));
                    if (row_in[2 * r4 + 1]) __builtin_nontemporal_store(hi, (u32x4*)(obase + rowoff[2 * r4 + 1] + 64 * dp));
                }
            }
        }
    }
}


// slab 0 += slabs 1 .. nz - 1: 8 elements (16 bit) of dkbar / dy or one float of dc per thread
template <class E>
__global__ __launch_bounds__(256) void monarch_bwd_left_sum_kernel(uint16_t* dkbar, uint16_t* dy, int64_t slab_rows, float* dc,
                                                                   int64_t slab_dc, int nz) {
    const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int64_t n16 = slab_rows / 8;
    if (t < 2 * n16) {
        uint16_t* base = (t < n16 ? dkbar : dy) + (t < n16 ? t : t - n16) * 8;
        float acc[8];
        u32x4 w = *(const u32x4*)base;
        const uint32_t w0[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            acc[2 * i] = E::to_float((uint16_t)(w0[i] & 0xffffu));
            acc[2 * i + 1] = E::to_float((uint16_t)(w0[i] >> 16));
        }
        for (int z = 1; z < nz; ++z) {
            const u32x4 x = *(const u32x4*)(base + z * slab_rows);
            const uint32_t xx[4] = {x.x, x.y, x.z, x.w};
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                acc[2 * i] += E::to_float((uint16_t)(xx[i] & 0xffffu));
                acc[2 * i + 1] += E::to_float((uint16_t)(xx[i] >> 16));
            }
        }
        w.x = pack2<E>(acc[0], acc[1]); w.y = pack2<E>(acc[2], acc[3]); w.z = pack2<E>(acc[4], acc[5]); w.w = pack2<E>(acc[6], acc[7]);
        *(u32x4*)base = w;
    } else {
        const int64_t c = t - 2 * n16;
        if (c < slab_dc) {
            float a = dc[c];
            for (int z = 1; z < nz; ++z) a += dc[z * slab_dc + c];
            dc[c] = a;
        }
    }
}

// ---------------------------------------------------------------------------------------------------------------
// dQ of the left factor, dQ[i, :] = s sum_r dS2[i, r] Kbar[r, :] per (unit, a, j), plus the right factor's part
// (already reduced per (unit, k) by a library GEMM), written straight to the caller's dq rows.
// One wave per (unit, a, j): its Kbar rows go through LDS 32 at a time (global_load_lds_dwordx4, double buffered,
// 16-byte chunks XOR-swizzled per row) and come back as the B operand [n = d, k = r] through transposing reads; the
// A operand [m = i, k = r] is dS2 straight from memory, two 8-byte pieces per step in the order in which the
// transposing reads deliver r.
struct DqaArgs {
    const char* kbar;        // row r of (u, aj) at ((u * RR + r) * AJ + aj) * D elements
    const uint16_t* ds2;     // [u][aj][b1][ds2_ld], ds2_ld a multiple of 4
    const float* dqk;        // [u][i][aj][D]
    float* dq;               // caller's tensor, strides s0 (batch), s1 (token), s2 (head)
    int64_t s0, s1, s2;
    TokMap map;
    int ds2_ld, b1, b2, AJ, RR, H, unit0;
    float scale;
    int nunits, nz;               // units of this launch, 32-row query slices per column
};


template <class E, int D>
__global__ __launch_bounds__(256) void monarch_bwd_dqa_kernel(DqaArgs p) {
    constexpr int DT = D / 32, CPR = D / 8;
    constexpr int kPitch = 2 * D;
    constexpr int kTile = 32 * kPitch;
    constexpr int kInstr = 32 * CPR / 64;                 // 64-lane loads per tile
    extern __shared__ __attribute__((aligned(256))) char lds[];
    const uint32_t lds0 = (uint32_t)(size_t)(__attribute__((address_space(3))) char*)lds;

    const int tid = threadIdx.x, lane = tid & 63, m = lane & 31, hf = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int njg = (p.AJ + 3) / 4;                       // work items as in monarch_bwd_left_kernel
    const int item = xcd_item(njg * p.nunits * p.nz);
    if (item >= njg * p.nunits * p.nz) return;
    const int zi = item % p.nz, jg = (item / p.nz) % njg;
    const int ajraw = jg * 4 + wave;
    const bool aj_ok = ajraw < p.AJ;
    const int aj = aj_ok ? ajraw : p.AJ - 1;              // a wave past the end repeats the last column and stores nothing
    const int u = item / (p.nz * njg);
    const int i0 = zi * 32;                               // first query row of this slice (b1 > 32: one slice per 32 rows)
    const int RR = p.RR, b1 = p.b1;
    const int64_t uaj = (int64_t)u * p.AJ + aj;
    const int nch = (RR + 31) / 32;
    const uint32_t rstride = (uint32_t)p.AJ * kPitch;     // bytes between rows r, r + 1
    const char* kb = p.kbar + ((int64_t)u * RR * p.AJ + aj) * kPitch;
    const uint32_t buf0 = lds0 + (uint32_t)wave * 2 * kTile;
    const char* mine = lds + wave * 2 * kTile;

    // LDS position P (16-byte units) of a tile holds chunk (P % CPR) ^ swz(row) of row P / CPR
    auto stage = [&](int n) {
#pragma unroll
        for (int q = 0; q < kInstr; ++q) {
            const int P = 64 * q + lane;
            const int row = P / CPR, c = (P % CPR) ^ bl_swz<CPR>(row);
            const int r = min(32 * n + row, RR - 1);
            bl_load_lds16(kb, (uint32_t)r * rstride + (uint32_t)c * 16, buf0 + (uint32_t)(n & 1) * kTile + (uint32_t)q * 1024);
        }
    };
    // dS2 pieces of row i = m: r = 32 n + 16 ks + 4 hf + {0..3} and + 8 + {0..3}
    const uint16_t* arow = p.ds2 + (uaj * b1 + min(i0 + m, b1 - 1)) * p.ds2_ld + 4 * hf;
    u32x4 acur[2], anext[2];
    auto load_a = [&](int n, u32x4 (&a)[2]) {
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
            const int r0 = 32 * n + 16 * ks + 4 * hf;
            u32x2 lo = {0u, 0u}, hi = {0u, 0u};
            if (r0 + 4 <= RR) lo = *(const u32x2*)(arow + 32 * n + 16 * ks);
            else
                for (int e2 = 0; e2 < 4; ++e2)
                    if (r0 + e2 < RR) {
                        const uint32_t x = arow[32 * n + 16 * ks + e2];
                        if (e2 < 2) lo.x |= x << (16 * e2); else lo.y |= x << (16 * (e2 - 2));
                    }
            if (r0 + 12 <= RR) hi = *(const u32x2*)(arow + 32 * n + 16 * ks + 8);
            else
                for (int e2 = 0; e2 < 4; ++e2)
                    if (r0 + 8 + e2 < RR) {
                        const uint32_t x = arow[32 * n + 16 * ks + 8 + e2];
                        if (e2 < 2) hi.x |= x << (16 * e2); else hi.y |= x << (16 * (e2 - 2));
                    }
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
                tr[dt][half] = (uint32_t)(r * kPitch + (((4 * dt + cl) ^ bl_swz<CPR>(r)) << 4) + (s16 & 1) * 8);
            }
    }

    f32x16 acc[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[dt][v] = 0.f;

    stage(0);
    load_a(0, acur);
    for (int n = 0; n < nch; ++n) {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");          // tile n and its dS2 pieces have landed
        if (n + 1 < nch) {
            stage(n + 1);
            load_a(n + 1, anext);
        }
        const char* tile = mine + (n & 1) * kTile;
#pragma unroll
        for (int ks = 0; ks < 2; ++ks)
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
                const u32x2 lo = bl_read_tr(tile, tr[dt][0] + ks * 16 * kPitch);
                const u32x2 hi = bl_read_tr(tile, tr[dt][1] + ks * 16 * kPitch);
                const u32x4 bop = {lo.x, lo.y, hi.x, hi.y};
                acc[dt] = E::mfma32(acur[ks], bop, acc[dt]);
            }
        acur[0] = anext[0];
        acur[1] = anext[1];
    }
    if (!aj_ok) return;
    // lane (d = 32 dt + m) holds rows i = 8 g + 4 hf + e
    const int a_blk = aj / p.b2, j = aj % p.b2;
    const int unit = p.unit0 + u;
    const int b = unit / p.H, h = unit % p.H;
    float* const out = p.dq + b * p.s0 + h * p.s2;
#pragma unroll
    for (int v = 0; v < 16; ++v) {
        const int i = i0 + 8 * (v >> 2) + 4 * hf + (v & 3);
        if (i < b1) {
            const int64_t tok = p.map.row(a_blk, i) + j;
            const float* add = p.dqk + (((int64_t)u * b1 + i) * p.AJ + aj) * D;
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) out[tok * p.s1 + 32 * dt + m] = acc[dt][v] * p.scale + add[32 * dt + m];
        }
    }
}

}  // namespace

bool monarch_bwd_left_supported(int dtype, int D, int b1) {
    return (dtype == SFM_BF16 || dtype == SFM_F16) && (D == 64 || D == 128) && b1 >= 1 && b1 <= 128;
}

int launch_monarch_bwd_left(int dtype, int D, int n, int b1, int b2, int AJ, int nf, int causal, float scale, const void* q,
                            const int64_t* qs, const void* dout, const void* out, const int64_t* os, const TokMap& qmap, int H,
                            int unit0, const void* kbar, const void* y, const float* c, int c_rows, void* dkbar, void* dy, float* dc,
                            void* ds2, int ds2_ld, const float* stats, int stats_ld, hipStream_t stream) {
    LeftArgs a;
    a.ds2_ld = ds2_ld;
    a.q = (const char*)q; a.dout = (const char*)dout; a.out = (const char*)out;
    for (int i = 0; i < 3; ++i) {
        a.qs[i] = qs[i];
        a.os[i] = os[i];
    }
    a.qmap = qmap;
    a.H = H;
    a.stats = out ? stats : nullptr; a.stats_ld = stats_ld; a.unit0 = unit0;
    a.c_rows = c_rows;
    a.kbar = (const uint16_t*)kbar; a.y = (const uint16_t*)y;
    a.c = c;
    a.dkbar = (uint16_t*)dkbar; a.dy = (uint16_t*)dy;
    a.dc = dc;
    a.ds2 = (uint16_t*)ds2;
    a.b1 = b1; a.b2 = b2; a.AJ = AJ; a.nf = nf; a.RR = nf * b1; a.causal = causal;
    a.scale = scale;
    const int nz = (b1 + 31) / 32;
    a.slab_rows = (int64_t)n * a.RR * AJ * D;             // the caller's dkbar / dy / dc hold nz slabs
    a.slab_dc = (int64_t)n * AJ * a.RR;
    a.nunits = n;
    a.nz = nz;
    const dim3 grid((unsigned)xcd_grid((AJ + 3) / 4 * n * nz));
    const size_t ldsb = (size_t)4 * (D == 128 ? LeftLds<128>::kPerWave : LeftLds<64>::kPerWave);
    const void* fn = nullptr;
    if (dtype == SFM_BF16) fn = D == 128 ? (const void*)monarch_bwd_left_kernel<BF16, 128> : (const void*)monarch_bwd_left_kernel<BF16, 64>;
    else fn = D == 128 ? (const void*)monarch_bwd_left_kernel<F16, 128> : (const void*)monarch_bwd_left_kernel<F16, 64>;
    if (ldsb > 64 * 1024) {
        hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)ldsb);
        if (e != hipSuccess) {
            set_error("monarch backward (left factor): cannot reserve %zu bytes of LDS: %s", ldsb, hipGetErrorString(e));
            return SFM_ERR_HIP;
        }
    }
    if (dtype == SFM_BF16) {
        if (D == 128) hipLaunchKernelGGL((monarch_bwd_left_kernel<BF16, 128>), grid, dim3(256), ldsb, stream, a);
        else hipLaunchKernelGGL((monarch_bwd_left_kernel<BF16, 64>), grid, dim3(256), ldsb, stream, a);
    } else {
        if (D == 128) hipLaunchKernelGGL((monarch_bwd_left_kernel<F16, 128>), grid, dim3(256), ldsb, stream, a);
        else hipLaunchKernelGGL((monarch_bwd_left_kernel<F16, 64>), grid, dim3(256), ldsb, stream, a);
    }
    if (nz > 1) {
        const int64_t threads = 2 * (a.slab_rows / 8) + a.slab_dc;
        const dim3 gs((unsigned)((threads + 255) / 256));
        if (dtype == SFM_BF16) hipLaunchKernelGGL((monarch_bwd_left_sum_kernel<BF16>), gs, dim3(256), 0, stream, a.dkbar, a.dy, a.slab_rows, a.dc, a.slab_dc, nz);
        else hipLaunchKernelGGL((monarch_bwd_left_sum_kernel<F16>), gs, dim3(256), 0, stream, a.dkbar, a.dy, a.slab_rows, a.dc, a.slab_dc, nz);
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        set_error("monarch backward (left factor): launch failed: %s", hipGetErrorString(e));
        return SFM_ERR_HIP;
    }
    return SFM_OK;
}

int launch_monarch_bwd_dqa(int dtype, int D, int n, int b1, int b2, int AJ, int nf, float scale, const void* kbar, const void* ds2,
                           int ds2_ld, const float* dqk, float* dq, const int64_t* dqs, const TokMap& map, int H, int unit0,
                           hipStream_t stream) {
    if (ds2_ld % 4 || ds2_ld < nf * b1) {
        set_error("monarch backward (dQ of the left factor): row pitch %d of dS2 must be a multiple of 4 and >= %d", ds2_ld, nf * b1);
        return SFM_ERR_SHAPE;
    }
    DqaArgs a;
    a.kbar = (const char*)kbar;
    a.ds2 = (const uint16_t*)ds2;
    a.dqk = dqk;
    a.dq = dq;
    a.s0 = dqs[0]; a.s1 = dqs[1]; a.s2 = dqs[2];
    a.map = map;
    a.ds2_ld = ds2_ld; a.b1 = b1; a.b2 = b2; a.AJ = AJ; a.RR = nf * b1; a.H = H; a.unit0 = unit0;
    a.scale = scale;
    a.nunits = n;
    a.nz = (b1 + 31) / 32;
    const dim3 grid((unsigned)xcd_grid((AJ + 3) / 4 * n * a.nz));
    const size_t ldsb = (size_t)4 * 2 * 32 * 2 * D;
    if (dtype == SFM_BF16) {
        if (D == 128) hipLaunchKernelGGL((monarch_bwd_dqa_kernel<BF16, 128>), grid, dim3(256), ldsb, stream, a);
        else hipLaunchKernelGGL((monarch_bwd_dqa_kernel<BF16, 64>), grid, dim3(256), ldsb, stream, a);
    } else {
        if (D == 128) hipLaunchKernelGGL((monarch_bwd_dqa_kernel<F16, 128>), grid, dim3(256), ldsb, stream, a);
        else hipLaunchKernelGGL((monarch_bwd_dqa_kernel<F16, 64>), grid, dim3(256), ldsb, stream, a);
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        set_error("monarch backward (dQ of the left factor): launch failed: %s", hipGetErrorString(e));
        return SFM_ERR_HIP;
    }
    return SFM_OK;
}

}  // namespace sfm
