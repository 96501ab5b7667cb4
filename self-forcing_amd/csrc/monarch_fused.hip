// Monarch attention forward as ONE kernel on gfx950 (bf16 / fp16, head_dim 128, b1 <= 32, b2 <= 64, no causal mask): the
// right factor's products Kbar / Y (step 1, _al_cl_y_fwd, wan/modules/monarch_attn.py:109-253) never leave the compute
// unit; the left factor (step 2, _z_fwd, monarch_attn.py:698-842) consumes them from LDS.
//
// A workgroup of 8 waves owns a group of up to 12 (a, j) columns of one (batch, head) unit and walks a contiguous range
// of that unit's K/V tiles (f, k), k-major.  The waves have fixed roles:
//   * waves 6, 7 (right factor): per tile the logits S^T[l, c] = K[f,k,l,:] . Q[a_c,k,j_c,:] (16x16x32 MFMA; the K rows
//     and the 16 columns' query rows come straight from global memory into registers, two steps ahead), the block
//     softmax over l, sum_l R log2 R, and R^T (16 bit) into LDS.  They alternate tiles and have two steps per tile.
//   * waves 0..5 (owners): per tile they bring the K and V rows into LDS (global_load_lds_dwordx4, three buffers, two
//     tiles ahead, plus one dword load per cache line six tiles ahead that only warms the L2), contract the tile with
//     its R^T: Kbar^T = K^T R^T, Y^T = V^T R^T (A operands are transposing LDS reads of the row-major tiles), and park
//     the columns' Kbar / Y rows in LDS.  Every `rc` tiles each owner runs the left factor for its own two columns on
//     the parked rows: S2^T[r, i] = Kbar[r,:] . Q[a,i,j,:] - cl[r] (16x16x32 MFMA), online softmax over r,
//     O^T[d, i] += Y^T[d, r] P^T[r, i] (32x32x16 MFMA, fp32 accumulators for the whole range).  The accumulators (64
//     registers per column) and the columns' query rows (32 registers per column) stay in registers, which is what
//     limits a workgroup to 12 columns.
// LDS rows are 256 bytes; their 16-byte pieces are XOR-swizzled by two or three low bits of the row (tiles) or of the
// row and the column (parked rows), chosen so that every access pattern above spreads evenly over the banks while the
// offsets between the reads of one operand stay instruction immediates.
//
// Work distribution: the tile list of all units of a pass is cut into `nstreams` equal contiguous ranges; workgroup
// (stream, group) handles the group's columns over the stream's range, so that the workgroups of one stream read the
// same K/V tiles at the same time (they are given consecutive positions on one XCD and share its L2).  A stream's
// range may cross unit boundaries and a unit may be covered by several streams: each (unit, stream) segment writes
// its normalised output and its log-sum-exp to a scratch slot, and a small second kernel merges the slots of a row
// (the merge _z_fwd does between KV chunks, monarch_attn.py:790-797, 840-842).  A segment that covers a whole unit
// writes the final output directly.

#include <string.h>

#include "sfm_common.hpp"

namespace sfm {

namespace {

constexpr int kFD = 128;           // head_dim
constexpr int kPitch = 2 * kFD;    // bytes per row
constexpr int kOwners = 6;         // waves that own columns; two more waves compute the right factor's logits
constexpr int kCPW = 2;            // columns per owner wave
constexpr int kMaxNJ = kOwners * kCPW;
constexpr int kBufs = 3;           // K/V tile buffers
constexpr int kLdsMax = 160 * 1024;
constexpr int kRtBytes = 3 * 2048, kClBytes = 2 * 1024;

struct FusedArgs {
    const void* q;
    const void* k;
    const void* v;
    void* out;
    void* part_o;        // [units][nslots][ncols][b1][D], tensor dtype
    float* part_lse;     // [units][nslots][ncols][32], log2 units
    float* stats;        // optional: merged log2-sum-exp per query row
    uint32_t stats_ld;
    int H, na, nf, b1, b2, b2p;
    int unit0, nunits;
    int ncols, nj, ngroups;
    int rc;              // parked rows per left-factor pass (8..16)
    int lds_bytes;
    int tpu, total, tps, nstreams, nslots;
    // token row of K[f, k, 0, :] = frow(f) + krow(k); frow advances by step_e per block-frame, by step_c instead every
    // wrap_e-th and by step_a instead every (wrap_e * wrap_c)-th (the tiling's column / row tiles of a frame group)
    int step_e, step_c, step_a, wrap_e, wrap_c;
    float scale;
    TokMap qmap, kmap;
    int64_t qs[3], ks[3], vs[3], os[3];
};

__device__ __forceinline__ float xg_max(float x) {      // over the four 16-lane rows of a wave
    auto a = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    x = fmaxf(__uint_as_float(a[0]), __uint_as_float(a[1]));
    auto b = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return fmaxf(__uint_as_float(b[0]), __uint_as_float(b[1]));
}
__device__ __forceinline__ float xg_sum(float x) {
    auto a = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    x = __uint_as_float(a[0]) + __uint_as_float(a[1]);
    auto b = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return __uint_as_float(b[0]) + __uint_as_float(b[1]);
}

typedef short fz_s16x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ u32x2 fz_read_tr(const char* lds) {
    fz_s16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((fz_s16x4 __attribute__((address_space(3)))*)lds);
    return __builtin_bit_cast(u32x2, v);
}
__device__ __forceinline__ void fz_load_lds16(const char* base, uint32_t off, uint32_t lds_addr) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_addr), "v"(off), "s"(base) : "memory", "m0");
}
// Walks a unit's tiles (f, k) in the order k-major, f-minor and keeps the token row of K[f, k, 0, :] without divisions.
struct TileWalk {
    int tt, f, k, e, c;
    uint32_t frow, krow;
    __device__ __forceinline__ void init(const FusedArgs& p, int tt_) {
        tt = tt_;
        k = tt / p.nf;
        f = tt - k * p.nf;
        frow = (uint32_t)p.kmap.row(f, 0);
        krow = (uint32_t)p.kmap.row_delta(k);
        e = f % p.wrap_e;
        c = (f / p.wrap_e) % p.wrap_c;
    }
    __device__ __forceinline__ uint32_t row() const { return frow + krow; }
    // next tile; stays on the unit's last tile
    __device__ __forceinline__ void next(const FusedArgs& p) {
        if (tt >= p.tpu - 1) return;
        ++tt;
        if (++f == p.nf) {
            f = 0; e = 0; c = 0; frow = 0;
            krow = (uint32_t)p.kmap.row_delta(++k);
        } else if (++e < p.wrap_e) {
            frow += (uint32_t)p.step_e;
        } else {
            e = 0;
            if (++c < p.wrap_c) {
                frow += (uint32_t)p.step_c;
            } else {
                c = 0;
                frow += (uint32_t)p.step_a;
            }
        }
    }
};

}  // namespace

template <class E>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2))) void monarch_fused_kernel(FusedArgs p) {
    extern __shared__ __attribute__((aligned(256))) char lds[];
    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lane = tid & 63;
    const int c16 = lane & 15, g = lane >> 4;          // 16x16x32 layouts: column / row group
    const int m32 = lane & 31, hf = lane >> 5;         // 32x32x16 layouts

    // Workgroups are dealt to the XCDs round-robin; v is a position such that the workgroups of one XCD are consecutive.
    const int G = gridDim.x;
    const int xcd = blockIdx.x & 7, idx = blockIdx.x >> 3;
    int pre = 0;
    for (int y = 0; y < xcd; ++y) pre += (G - y + 7) >> 3;
    const int v = pre + idx;
    const int stream = v / p.ngroups, group = v - stream * p.ngroups;
    if (stream >= p.nstreams) return;
    const int c0 = group * p.nj;
    const int ncg = min(p.nj, p.ncols - c0);           // columns of this group
    const int T0 = stream * p.tps, T1 = min(T0 + p.tps, p.total);

    const int b2 = p.b2, nj = p.nj, rc = p.rc;
    const int TB = p.b2p * kPitch;                     // bytes of one K or V tile; buffer b holds K at 2 b TB, V behind it
    const int P0 = 2 * kBufs * TB;                     // Kbar park [nj][rc rows][256 B]
    const int PC = rc * kPitch;                        // one column's parked rows
    const int PY = nj * PC;                            // the Y park follows the Kbar park
    const int R0 = P0 + 2 * PY;                        // R^T: [3][16 columns][64 l] 16 bit
    const int C0 = R0 + kRtBytes;                      // cl: [2][16 columns][16 rows] float
    const uint32_t lds0 = (uint32_t)(size_t)(__attribute__((address_space(3))) char*)lds;

    // All of LDS starts finite: operands are read a few rows past the end of a tile (to a multiple of 32 rows) and of a
    // column's parked rows (to 16); those rows carry weight 0, and 0 * NaN would be NaN.
    for (int o = tid * 16; o < p.lds_bytes; o += 512 * 16) *(u32x4*)(lds + o) = u32x4{0u, 0u, 0u, 0u};

    const uint32_t qs1 = (uint32_t)p.qs[1], ks1 = (uint32_t)p.ks[1];
    const float sc2 = p.scale * kLog2e;
    const f32x4 kZero4 = {0.f, 0.f, 0.f, 0.f};

    // Every wave runs the same sequence of barriers: per segment one at the top of each step s = -2 .. N-1, one before
    // each left-factor pass (after the steps that fill the last parked row, and after step N-1), one at the segment's end.
    if (wave >= kOwners) {
        // ================= right-factor waves: logits, block softmax over l, R^T and cl to LDS =================
        // Wave kOwners + e takes the tiles n with n % 2 == e: the logits in step n - 2, the softmax in step n - 1.
        const int me = wave - kOwners;
        uint32_t qoff_l;       // byte offset of Q[a, 0, j, 8 g ..] of this lane's column (past the group's last column: that one again)
        {
            const int cg = c0 + min(c16, ncg - 1);
            const int a = cg / b2;
            qoff_l = (uint32_t)(p.qmap.row(a, 0) + (cg - a * b2)) * qs1 * 2 + 16 * g;
        }
        uint32_t koff[4];      // byte offset of key row 16 mt + c16 (head-dim 8 g ..) from the tile's first row
#pragma unroll
        for (int mt = 0; mt < 4; ++mt) koff[mt] = (uint32_t)min(16 * mt + c16, b2 - 1) * ks1 * 2 + 16 * g;
        for (int T = T0; T < T1;) {
            const int ul = T / p.tpu;
            const int tt0 = T - ul * p.tpu;
            const int N = min(p.tpu - tt0, T1 - T);         // tiles of this segment
            T += N;
            const int unit = p.unit0 + ul;
            const int bb = unit / p.H, hh = unit - bb * p.H;
            const char* kg = (const char*)p.k + ((int64_t)bb * p.ks[0] + (int64_t)hh * p.ks[2]) * 2;
            const char* qg = (const char*)p.q + ((int64_t)bb * p.qs[0] + (int64_t)hh * p.qs[2]) * 2;

            u32x4 kr[4][4], qB[4];      // K rows 16 mt + c16 (A) and the 16 columns' query rows of block row k (B), 16 bytes per step
            TileWalk tw;                // the tile this wave fetches next: me, me + 2, ...
            tw.init(p, min(tt0 + me, p.tpu - 1));
            int qk = -1;
            uint32_t qdelta = 0;
            auto prefetch = [&]() {
                const char* kb = kg + (size_t)tw.row() * ks1 * 2;
#pragma unroll
                for (int mt = 0; mt < 4; ++mt)
#pragma unroll
                    for (int ks = 0; ks < 4; ++ks) kr[mt][ks] = *(const u32x4*)(kb + koff[mt] + 64 * ks);
                if (tw.k != qk) {
                    qk = tw.k;
                    qdelta = (uint32_t)p.qmap.row_delta(qk) * qs1 * 2;
                }
                const char* qb = qg + qdelta;
#pragma unroll
                for (int ks = 0; ks < 4; ++ks) qB[ks] = *(const u32x4*)(qb + qoff_l + 64 * ks);
                tw.next(p);
                tw.next(p);
            };
            f32x4 sa[4] = {kZero4, kZero4, kZero4, kZero4};
            float mx = 0.f;
            if (me < N) prefetch();
            int crow = 0;                           // parked row of tile s (the owners' counter, for the barriers)
            int my_row = me % rc, my_par = (me / rc) & 1;      // parked row and cl buffer of this wave's next softmax tile
            for (int s = -2; s < N; ++s) {
                lds_barrier();
                if (((s + 2) & 1) == me) {
                    if (s + 2 < N) {
                        // logits of tile n = s + 2 and their column maxima
#pragma unroll
                        for (int mt = 0; mt < 4; ++mt) {
                            sa[mt] = kZero4;
#pragma unroll
                            for (int ks = 0; ks < 4; ++ks) sa[mt] = E::mfma16(kr[mt][ks], qB[ks], sa[mt]);
                        }
                        if (s + 4 < N) prefetch();
                        mx = -INFINITY;
#pragma unroll
                        for (int mt = 0; mt < 4; ++mt)
#pragma unroll
                            for (int e = 0; e < 4; ++e) {
                                const int l = 16 * mt + 4 * g + e;
                                const float z = l < b2 ? sa[mt][e] * sc2 : kMaskLogit;
                                sa[mt][e] = z;
                                mx = fmaxf(mx, z);
                            }
                        mx = xg_max(mx);
                    }
                } else if (s + 1 >= 0 && s + 1 < N) {
                    const int n = s + 1;
                    float sum = 0.f, ent = 0.f;
#pragma unroll
                    for (int mt = 0; mt < 4; ++mt)
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            const float z = sa[mt][e];
                            const float ex = fast_exp2(z - mx);       // exactly 0 for rows past the tile
                            sum += ex;
                            ent += ex * z;
                            sa[mt][e] = ex;
                        }
                    sum = xg_sum(sum);
                    ent = xg_sum(ent);
                    const float inv = 1.f / sum;
                    char* rt = lds + R0 + (n % 3) * 2048 + c16 * 128 + 8 * (g & 1);
#pragma unroll
                    for (int mt = 0; mt < 4; ++mt) {
                        u32x2 w;                                       // R rounded to 16 bit once, after its normalisation
                        w.x = pack2<E>(sa[mt][0] * inv, sa[mt][1] * inv);
                        w.y = pack2<E>(sa[mt][2] * inv, sa[mt][3] * inv);
                        *(u32x2*)(rt + (((2 * mt + (g >> 1)) ^ (c16 & 7)) << 4)) = w;
                    }
                    if (g == 0) *(float*)(lds + C0 + my_par * 1024 + c16 * 64 + my_row * 4) = ent * inv - (mx + log2f(sum));
                    my_row += 2;
                    if (my_row >= rc) {
                        my_row -= rc;
                        my_par ^= 1;
                    }
                }
                if (s >= 0) {
                    if (crow == rc - 1 || s == N - 1) lds_barrier();
                    crow = crow == rc - 1 ? 0 : crow + 1;
                }
            }
            lds_barrier();
        }
    } else {
        // ================= owner waves: the tiles into LDS; Kbar^T = K^T R^T, Y^T = V^T R^T per tile; the left factor of their columns =================
        const int rq = (lane >> 2) & 3, cq = lane & 3;
        // A 16-lane block of a transposing read takes 4 rows x 16 values; lane 4 r' + c' supplies row r', values 4 c' .. 4 c' + 3.
        // K / V tile as the A operand of K^T R^T (16 head-dim rows 16 mt .. x 32 key rows per step): row 8 g + r' of the
        // step (+4 for the second half, +32 for the second step: immediates), pieces 2 mt, 2 mt + 1 XOR ((row & 3) << 1).
        const uint32_t trbase = (uint32_t)((8 * g + rq) * kPitch + 8 * (cq & 1) + 16 * (cq >> 1));
        // Parked row written from the accumulators: column c16, head-dim 16 mt + 4 g ..: piece 2 mt + (g >> 1)
        // XOR ((column & 3) << 1) XOR ((row & 1) << 2).
        const uint32_t wbase = (uint32_t)(c16 * PC + 16 * (g >> 1) + 8 * (g & 1));
        // R^T as the B operand: column c16, key rows 32 ks + 8 g ..: piece 4 ks + g XOR (c16 & 7)
        const uint32_t rtb = (uint32_t)(c16 * 128 + ((g ^ (c16 & 7)) << 4));
        // tile loads: instruction i covers rows 4 i .. 4 i + 3 (this lane: row 4 i + g, piece (lane & 15) XOR ((g & 3) << 1));
        // waves 0..2 bring the K tile, waves 3..5 the V tile, instruction i = wave % 3, + 3, ...
        const int ninst = p.b2p / 4;
        const int dfirst = wave % 3;
        const int nmine = dfirst < ninst ? (ninst - dfirst + 2) / 3 : 0;       // 0..6 loads per step
        const uint32_t dlane = (uint32_t)(((lane & 15) ^ ((g & 3) << 1)) * 16);
        uint32_t qoff[2];           // byte offset of query row i = 16 nt + c16 (head-dim 8 g ..) from the column's row 0
#pragma unroll
        for (int nt = 0; nt < 2; ++nt) qoff[nt] = (uint32_t)p.qmap.row_delta(min(16 * nt + c16, p.b1 - 1)) * qs1 * 2 + 16 * g;
        int colx[kCPW];             // column index within the group (clamped)
        uint32_t qcol_x[kCPW];      // token row of Q[a, 0, j] of the column
#pragma unroll
        for (int x = 0; x < kCPW; ++x) {
            colx[x] = min(wave * kCPW + x, ncg - 1);
            const int cg = c0 + colx[x];
            const int a = cg / b2;
            qcol_x[x] = (uint32_t)(p.qmap.row(a, 0) + (cg - a * b2));
        }

        for (int T = T0; T < T1;) {
            const int ul = T / p.tpu;
            const int tt0 = T - ul * p.tpu;
            const int N = min(p.tpu - tt0, T1 - T);         // tiles of this segment
            T += N;
            const int unit = p.unit0 + ul;
            const int bb = unit / p.H, hh = unit - bb * p.H;
            const char* kg = (const char*)p.k + ((int64_t)bb * p.ks[0] + (int64_t)hh * p.ks[2]) * 2;
            const char* vg = (const char*)p.v + ((int64_t)bb * p.vs[0] + (int64_t)hh * p.vs[2]) * 2;
            const char* qg = (const char*)p.q + ((int64_t)bb * p.qs[0] + (int64_t)hh * p.qs[2]) * 2;
            const char* tg = wave < 3 ? kg : vg;
            // Tiles are staged two steps ahead; the walk stays on the unit's last tile once it reaches it (the loads past a
            // segment's end are not used).  A wave issues the same number of loads in every step, which the waits count on.
            TileWalk tw_stage;
            tw_stage.init(p, tt0);
            auto stage = [&](int buf) {
                const char* tb = tg + (size_t)tw_stage.row() * ks1 * 2;
                const uint32_t dst = lds0 + (uint32_t)buf * 2 * TB + (wave < 3 ? 0u : (uint32_t)TB);
                for (int i = dfirst; i < ninst; i += 3)
                    fz_load_lds16(tb, (uint32_t)min(4 * i + g, b2 - 1) * ks1 * 2 + dlane, dst + (uint32_t)i * 1024);
                tw_stage.next(p);
            };

            // Q[a, i, j, :] as B operands of the left factor's logits (i = 16 nt + c16, head-dim 32 ks + 8 g ..): 32 registers
            // per column that this role cannot keep for the whole segment beside the accumulators.  They are fetched for
            // every pass: the first column's at the top of the step that ends with the pass, the second column's as soon as
            // the first column's logits are done.
            u32x4 qS[2][4];
            auto load_q = [&](int x) {
#pragma unroll
                for (int nt = 0; nt < 2; ++nt) {
                    const char* qrow = qg + (size_t)qcol_x[x] * qs1 * 2 + qoff[nt];
#pragma unroll
                    for (int ks = 0; ks < 4; ++ks) qS[nt][ks] = *(const u32x4*)(qrow + 64 * ks);
                }
            };
            f32x16 oacc[kCPW][4];
            float mrun[kCPW][2], lrun[kCPW][2];
#pragma unroll
            for (int x = 0; x < kCPW; ++x) {
#pragma unroll
                for (int nt = 0; nt < 2; ++nt) {
                    mrun[x][nt] = -INFINITY;
                    lrun[x][nt] = 0.f;
                }
#pragma unroll
                for (int dt = 0; dt < 4; ++dt)
#pragma unroll
                    for (int e = 0; e < 16; ++e) oacc[x][dt][e] = 0.f;
            }

            int crow = 0, cpar = 0;       // parked row of tile s and its cl buffer
            int buf = 0;                  // s % 3 for s >= 0
            for (int s = -2; s < N; ++s) {
                // Vector memory operations complete in order and this wave issues `nmine` tile loads per step: when at most
                // that many are outstanding, its loads of tile s (issued two steps ago) have landed.  Then every wave's
                // have, and every wave has finished with the buffers, R^T and parked rows of the step before.
                switch (nmine) {
                    case 6: asm volatile("s_waitcnt vmcnt(6)" ::: "memory"); break;
                    case 5: asm volatile("s_waitcnt vmcnt(5)" ::: "memory"); break;
                    case 4: asm volatile("s_waitcnt vmcnt(4)" ::: "memory"); break;
                    case 3: asm volatile("s_waitcnt vmcnt(3)" ::: "memory"); break;
                    case 2: asm volatile("s_waitcnt vmcnt(2)" ::: "memory"); break;
                    case 1: asm volatile("s_waitcnt vmcnt(1)" ::: "memory"); break;
                    default: asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); break;
                }
                lds_barrier();
                const bool pass = s >= 0 && (crow == rc - 1 || s == N - 1);        // this step ends with a left-factor pass
                if (pass) load_q(0);
                {
                    const int b2n = s < 0 ? s + 2 : (buf == 0 ? 2 : buf - 1);       // (s + 2) % 3
                    stage(b2n);
                }
                if (s >= 0) {
                    const char* rt = lds + R0 + buf * 2048;
                    u32x4 rb[2];
                    rb[0] = *(const u32x4*)(rt + rtb);
                    rb[1] = *(const u32x4*)(rt + (rtb ^ 64u));
                    const uint32_t wrow = wbase + (uint32_t)(P0 + crow * kPitch);
                    const uint32_t rkey = (uint32_t)((crow & 1) << 1);
                    const uint32_t tb0 = (uint32_t)(buf * 2 * TB) + trbase;
                    // 16 units of (matrix, 16 head-dim rows): this wave takes u = wave, wave + 6, wave + 12
#pragma unroll
                    for (int uu = 0; uu < 3; ++uu) {
                        const int u = wave + kOwners * uu;
                        if (u < 16) {
                            const int mat = u >> 3, mt = u & 7;
                            const char* tp = lds + (tb0 + (uint32_t)(mat * TB) + ((((uint32_t)mt) ^ (uint32_t)rq) << 5));
                            const u32x2 l0 = fz_read_tr(tp), h0 = fz_read_tr(tp + 4 * kPitch);
                            const u32x2 l1 = fz_read_tr(tp + 32 * kPitch), h1 = fz_read_tr(tp + 36 * kPitch);
                            f32x4 acc = E::mfma16(u32x4{l0.x, l0.y, h0.x, h0.y}, rb[0], kZero4);
                            acc = E::mfma16(u32x4{l1.x, l1.y, h1.x, h1.y}, rb[1], acc);
                            u32x2 w;
                            w.x = pack2<E>(acc[0], acc[1]);
                            w.y = pack2<E>(acc[2], acc[3]);
                            if (c16 < nj)
                                *(u32x2*)(lds + wrow + (uint32_t)(mat * PY) + (((((uint32_t)mt) ^ rkey) ^ (uint32_t)(c16 & 3)) << 5)) = w;
                        }
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }

                if (pass) {
                    // ---- left factor over the parked rows 0 .. crow
                    lds_barrier();
                    const int nrows = crow + 1;
                    const char* clb = lds + C0 + cpar * 1024;
#pragma unroll
                    for (int x = 0; x < kCPW; ++x) {
                        // a wave with fewer columns than kCPW works on its last column again (nothing of it is written)
                        const int cx = colx[x];
                        // Kbar rows as the A operand: row c16, pieces 4 ks + g; Y rows through transposing reads: rows 8 hf + r'
                        // (+4), pieces 4 dt + 2 (g & 1) + (c' >> 1); the piece XOR puts ks / dt odd 64 bytes from ks / dt even
                        const uint32_t a0 = (uint32_t)(P0 + cx * PC + c16 * kPitch + (((((cx >> 1) ^ c16) & 1)) << 6) + ((g ^ ((cx & 1) << 1)) << 4));
                        const uint32_t y0 = (uint32_t)(P0 + PY + cx * PC + (8 * hf + rq) * kPitch + 8 * (cq & 1) + 16 * (cq >> 1) +
                                                       (((g ^ cx) & 1) << 5) + ((((cx >> 1) ^ rq) & 1) << 6));
                        const char* pa0 = lds + a0;
                        const char* pa1 = lds + (a0 ^ 64u);
                        f32x4 S[2] = {kZero4, kZero4};
#pragma unroll
                        for (int ks = 0; ks < 4; ++ks) {
                            const u32x4 a = *(const u32x4*)(((ks & 1) ? pa1 : pa0) + 128 * (ks >> 1));
                            S[0] = E::mfma16(a, qS[0][ks], S[0]);
                            S[1] = E::mfma16(a, qS[1][ks], S[1]);
                        }
                        if (x + 1 < kCPW) load_q(x + 1);
                        const f32x4 cl4 = *(const f32x4*)(clb + cx * 64 + 16 * g);
                        __builtin_amdgcn_sched_barrier(0);
                        float mxc[2] = {-INFINITY, -INFINITY};
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            const int r = 4 * g + e;
#pragma unroll
                            for (int nt = 0; nt < 2; ++nt) {
                                float z = S[nt][e] * sc2 - cl4[e];
                                z = r < nrows ? z : -INFINITY;
                                S[nt][e] = z;
                                mxc[nt] = fmaxf(mxc[nt], z);
                            }
                        }
                        float alpha[2];
                        uint32_t pk2[2][2];
                        bool moved = false;
#pragma unroll
                        for (int nt = 0; nt < 2; ++nt) {
                            const float mnew = fmaxf(mrun[x][nt], xg_max(mxc[nt]));       // finite: row 0 of a pass is always there
                            moved = moved || mnew > mrun[x][nt];
                            alpha[nt] = fast_exp2(mrun[x][nt] - mnew);
                            float ps = 0.f;
#pragma unroll
                            for (int e = 0; e < 4; ++e) {
                                const float ex = fast_exp2(S[nt][e] - mnew);
                                ps += ex;
                                S[nt][e] = ex;
                            }
                            lrun[x][nt] = lrun[x][nt] * alpha[nt] + ps;      // this lane's rows only; summed over the row groups at the end
                            mrun[x][nt] = mnew;
                            pk2[nt][0] = pack2<E>(S[nt][0], S[nt][1]);
                            pk2[nt][1] = pack2<E>(S[nt][2], S[nt][3]);
                        }
                        // P^T as the B operand of the 32x32x16 product: lane i + 32 h needs rows 8 h .. 8 h + 7 of column i
                        const auto sx = __builtin_amdgcn_permlane16_swap(pk2[0][0], pk2[1][0], false, false);
                        const auto sy = __builtin_amdgcn_permlane16_swap(pk2[0][1], pk2[1][1], false, false);
                        const u32x4 pb = {(uint32_t)sx[0], (uint32_t)sy[0], (uint32_t)sx[1], (uint32_t)sy[1]};
                        // the running output is rescaled only when some row's maximum moved (after the first passes it rarely does)
                        if (__builtin_amdgcn_ballot_w64(moved) != 0) {
                            const float asel = (lane & 16) ? alpha[1] : alpha[0];
#pragma unroll
                            for (int dt = 0; dt < 4; ++dt)
#pragma unroll
                                for (int e = 0; e < 16; ++e) oacc[x][dt][e] *= asel;
                        }
                        const char* py0 = lds + y0;
                        const char* py1 = lds + (y0 ^ 64u);
                        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                        for (int dt = 0; dt < 4; ++dt) {
                            const char* py = ((dt & 1) ? py1 : py0) + 128 * (dt >> 1);
                            const u32x2 lo = fz_read_tr(py), hi = fz_read_tr(py + 4 * kPitch);
                            oacc[x][dt] = E::mfma32(u32x4{lo.x, lo.y, hi.x, hi.y}, pb, oacc[x][dt]);
                            if (dt == 1) __builtin_amdgcn_sched_barrier(0);
                        }
                        __builtin_amdgcn_sched_barrier(0);
                    }
                }
                if (s >= 0) {
                    if (crow == rc - 1) {
                        crow = 0;
                        cpar ^= 1;
                    } else {
                        ++crow;
                    }
                    buf = buf == 2 ? 0 : buf + 1;
                }
            }

            // ---- end of the segment: O = O^T / l through the wave's 8 KB of LDS, to the output or to this segment's slot
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");       // the tile loads issued past the segment's end have landed
            lds_barrier();                                          // every wave is done with the tiles and the parked rows
            const bool whole = N == p.tpu;
            const int s_first = (int)(((int64_t)ul * p.tpu) / p.tps);
            const int slot = stream - s_first;
            char* wl = lds + wave * (32 * kPitch);
#pragma unroll
            for (int x = 0; x < kCPW; ++x) {
                if (wave * kCPW + x < ncg) {
                    const int cg = c0 + colx[x];
                    float lse2[2], inv[2];
#pragma unroll
                    for (int nt = 0; nt < 2; ++nt) {
                        const float lt = xg_sum(lrun[x][nt]);
                        lse2[nt] = mrun[x][nt] + log2f(lt);
                        inv[nt] = 1.f / lt;
                    }
                    const float isel = (lane & 16) ? inv[1] : inv[0];
                    const float lsel = (lane & 16) ? lse2[1] : lse2[0];
#pragma unroll
                    for (int dt = 0; dt < 4; ++dt)
#pragma unroll
                        for (int q4 = 0; q4 < 4; ++q4) {
                            u32x2 w;
                            w.x = pack2<E>(oacc[x][dt][4 * q4 + 0] * isel, oacc[x][dt][4 * q4 + 1] * isel);
                            w.y = pack2<E>(oacc[x][dt][4 * q4 + 2] * isel, oacc[x][dt][4 * q4 + 3] * isel);
                            *(u32x2*)(wl + m32 * kPitch + (32 * dt + 8 * q4 + 4 * hf) * 2) = w;
                        }
                    lds_wave_sync();
                    if (whole) {
                        char* og = (char*)p.out + ((int64_t)bb * p.os[0] + (int64_t)hh * p.os[2]) * 2;
                        for (int c = lane; c < 32 * 16; c += 64) {
                            const int r = c >> 4, ch = c & 15;
                            if (r < p.b1) {
                                const u32x4 w = *(const u32x4*)(wl + r * kPitch + ch * 16);
                                *(u32x4*)(og + (size_t)(qcol_x[x] + (uint32_t)p.qmap.row_delta(r)) * (size_t)p.os[1] * 2 + ch * 16) = w;
                            }
                        }
                        if (p.stats != nullptr && hf == 0 && m32 < p.b1) p.stats[((int64_t)unit * p.ncols + cg) * p.stats_ld + m32] = lsel;
                    } else {
                        const size_t blk = ((size_t)ul * p.nslots + slot) * p.ncols + cg;
                        char* pg = (char*)p.part_o + blk * (size_t)p.b1 * kPitch;
                        for (int c = lane; c < 32 * 16; c += 64) {
                            const int r = c >> 4, ch = c & 15;
                            if (r < p.b1) *(u32x4*)(pg + r * kPitch + ch * 16) = *(const u32x4*)(wl + r * kPitch + ch * 16);
                        }
                        if (hf == 0) p.part_lse[blk * 32 + m32] = lsel;
                    }
                    lds_wave_sync();
                }
            }
        }
    }
}

// Merges the slots of a unit that several streams covered: out = sum_s w_s O_s / sum_s w_s with w_s = 2^(lse_s - max).
// One workgroup per (unit, column); thread = (query row i, 16-byte piece of the row).
template <class E>
__global__ __launch_bounds__(256) void monarch_fused_merge_kernel(FusedArgs p) {
    const int ul = blockIdx.y, cg = blockIdx.x;
    const int s0 = (int)(((int64_t)ul * p.tpu) / p.tps);
    const int s1 = (int)(((int64_t)(ul + 1) * p.tpu - 1) / p.tps);
    const int ns = s1 - s0 + 1;
    if (ns == 1) return;          // one segment covered the whole unit and wrote the output itself
    const int unit = p.unit0 + ul;
    const int bb = unit / p.H, hh = unit - bb * p.H;
    const int a = cg / p.b2, j = cg - a * p.b2;
    for (int w = threadIdx.x; w < p.b1 * 16; w += 256) {
        const int i = w >> 4, ch = w & 15;
        float mx = -INFINITY;
        for (int s = 0; s < ns; ++s) mx = fmaxf(mx, p.part_lse[(((size_t)ul * p.nslots + s) * p.ncols + cg) * 32 + i]);
        float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        float wsum = 0.f;
        for (int s = 0; s < ns; ++s) {
            const size_t blk = ((size_t)ul * p.nslots + s) * p.ncols + cg;
            const float wgt = exp2f(p.part_lse[blk * 32 + i] - mx);
            wsum += wgt;
            const u32x4 o = *(const u32x4*)((const char*)p.part_o + (blk * p.b1 + i) * kPitch + ch * 16);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                acc[2 * e] += wgt * E::to_float((uint16_t)(o[e] & 0xffffu));
                acc[2 * e + 1] += wgt * E::to_float((uint16_t)(o[e] >> 16));
            }
        }
        const float inv = 1.f / wsum;
        u32x4 r;
#pragma unroll
        for (int e = 0; e < 4; ++e) r[e] = pack2<E>(acc[2 * e] * inv, acc[2 * e + 1] * inv);
        char* og = (char*)p.out + ((int64_t)bb * p.os[0] + (int64_t)hh * p.os[2]) * 2;
        *(u32x4*)(og + (size_t)(p.qmap.row(a, i) + j) * (size_t)p.os[1] * 2 + ch * 16) = r;
        if (p.stats != nullptr && ch == 0) p.stats[((int64_t)unit * p.ncols + cg) * p.stats_ld + i] = mx + log2f(wsum);
    }
}

// ------------------------------------------------------------------------------------------------
// host side
// ------------------------------------------------------------------------------------------------
struct FusedPlan {
    int nj, ngroups, nstreams, tps, nslots, b2p, rc;
    size_t lds;
};

static FusedPlan fused_plan(int na, int nf, int b1, int b2, int nunits, int cus) {
    FusedPlan pl;
    pl.b2p = (b2 + 3) / 4 * 4;
    const int ncols = na * b2;
    int nj = kMaxNJ < ncols ? kMaxNJ : ncols;
    // three K/V tile buffers, R^T and cl; the rest of LDS parks nj columns x rc rows of Kbar and of Y
    const int avail = kLdsMax - 2 * kBufs * pl.b2p * kPitch - kRtBytes - kClBytes;
    int rc = avail / (2 * nj * kPitch);
    if (rc > 16) rc = 16;
    pl.rc = rc;                                            // >= 8 for b2 <= 64
    pl.ngroups = (ncols + nj - 1) / nj;
    pl.nj = (ncols + pl.ngroups - 1) / pl.ngroups;         // even groups
    const int64_t tpu = (int64_t)nf * b1, total = tpu * nunits;
    int64_t ns = cus / pl.ngroups;
    if (ns < 1) ns = 1;
    if (ns > total) ns = total;
    pl.tps = (int)((total + ns - 1) / ns);
    pl.nstreams = (int)((total + pl.tps - 1) / pl.tps);
    int64_t slots = (tpu - 1) / pl.tps + 2;                // a unit touches at most this many consecutive streams
    if (slots > pl.nstreams) slots = pl.nstreams;
    pl.nslots = (int)slots;
    size_t lds = (size_t)2 * kBufs * pl.b2p * kPitch + (size_t)2 * pl.nj * pl.rc * kPitch + kRtBytes + kClBytes;
    if (lds < kOwners * 32 * kPitch) lds = kOwners * 32 * kPitch;      // the output turn needs 8 KB per owner wave
    pl.lds = lds;
    return pl;
}

// Block-causal masking (the no-cache training operator) stays on the two-kernel forward.
bool monarch_fused_supported(int dtype, int D, int b1, int b2, int causal) {
    return (dtype == SFM_BF16 || dtype == SFM_F16) && D == kFD && b1 >= 1 && b1 <= 32 && b2 >= 1 && b2 <= 64 && causal == 0;
}

// Scratch of a pass over `nunits` units: the segments' outputs and log-sum-exps.
size_t monarch_fused_bytes(int na, int nf, int b1, int b2, int nunits) {
    const FusedPlan pl = fused_plan(na, nf, b1, b2, nunits, cu_count());
    const size_t blocks = (size_t)nunits * pl.nslots * na * b2;
    size_t bytes = blocks * b1 * kPitch;
    bytes = (bytes + 255) / 256 * 256;
    bytes += blocks * 32 * sizeof(float);
    return (bytes + 255) / 256 * 256;
}

template <class E>
static int launch_fused_t(const MonarchArgs& a, int nunits, void* ws, size_t ws_bytes, hipStream_t stream, const StepEvents* ev) {
    const FusedPlan pl = fused_plan(a.na, a.nf, a.b1, a.b2, nunits, cu_count());
    FusedArgs f;
    memset(&f, 0, sizeof(f));
    f.q = a.q; f.k = a.k; f.v = a.v; f.out = a.out;
    f.stats = a.stats; f.stats_ld = a.stats_ld;
    f.H = a.H; f.na = a.na; f.nf = a.nf; f.b1 = a.b1; f.b2 = a.b2; f.b2p = pl.b2p;
    f.unit0 = a.unit0; f.nunits = nunits;
    f.ncols = a.na * a.b2; f.nj = pl.nj; f.ngroups = pl.ngroups;
    f.rc = pl.rc; f.lds_bytes = (int)pl.lds;
    f.tpu = a.nf * a.b1; f.total = f.tpu * nunits; f.tps = pl.tps; f.nstreams = pl.nstreams; f.nslots = pl.nslots;
    f.scale = a.scale;
    f.qmap = a.qmap; f.kmap = a.kmap;
    if (a.kmap.natural) {
        const TokMap& m = a.kmap;
        f.wrap_e = m.w_reduce; f.wrap_c = m.h_reduce;
        f.step_e = m.ww;
        f.step_c = m.hh * m.w - (m.w_reduce - 1) * m.ww;
        f.step_a = m.f_tied * m.h * m.w - (m.h_reduce - 1) * m.hh * m.w - (m.w_reduce - 1) * m.ww;
    } else {
        f.wrap_e = 0x7fffffff; f.wrap_c = 1;
        f.step_e = f.step_c = f.step_a = a.b1 * a.b2;
    }
    for (int i = 0; i < 3; ++i) { f.qs[i] = a.qs[i]; f.ks[i] = a.ks[i]; f.vs[i] = a.vs[i]; f.os[i] = a.os[i]; }
    const size_t blocks = (size_t)nunits * pl.nslots * f.ncols;
    f.part_o = ws;
    f.part_lse = (float*)((char*)ws + (blocks * a.b1 * kPitch + 255) / 256 * 256);
    if (monarch_fused_bytes(a.na, a.nf, a.b1, a.b2, nunits) > ws_bytes) {
        set_error("internal: the one-kernel forward's pass of %d units does not fit the workspace", nunits);
        return SFM_ERR_WORKSPACE;
    }
    if ((int64_t)a.nf * a.b1 * nunits >= ((int64_t)1 << 31) || pl.lds > (size_t)kLdsMax || pl.rc < 8) {
        set_error("internal: fused Monarch launch shape");
        return SFM_ERR_UNSUPPORTED;
    }
    hipError_t e = hipFuncSetAttribute((const void*)monarch_fused_kernel<E>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)pl.lds);
    if (e != hipSuccess) {
        set_error("hipFuncSetAttribute failed: %s", hipGetErrorString(e));
        return SFM_ERR_HIP;
    }
    if (ev) (void)hipEventRecord(ev->ev[0], stream);
    hipLaunchKernelGGL((monarch_fused_kernel<E>), dim3(pl.nstreams * pl.ngroups), dim3(512), pl.lds, stream, f);
    if (ev) (void)hipEventRecord(ev->ev[1], stream);
    hipLaunchKernelGGL((monarch_fused_merge_kernel<E>), dim3(f.ncols, nunits), dim3(256), 0, stream, f);
    if (ev) (void)hipEventRecord(ev->ev[2], stream);
    e = hipGetLastError();
    if (e != hipSuccess) {
        set_error("hip launch failed: %s", hipGetErrorString(e));
        return SFM_ERR_HIP;
    }
    return SFM_OK;
}

int launch_monarch_fused(const MonarchArgs& a, int dtype, int nunits, void* ws, size_t ws_bytes, hipStream_t stream, const StepEvents* ev) {
    return dtype == SFM_BF16 ? launch_fused_t<BF16>(a, nunits, ws, ws_bytes, stream, ev) : launch_fused_t<F16>(a, nunits, ws, ws_bytes, stream, ev);
}

}  // namespace sfm
