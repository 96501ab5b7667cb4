// Monarch attention forward on gfx950 MFMA (bf16 / fp16, head_dim 64 or 128, block cols b2 <= 128).
//
// Two kernels per pass over a group of (batch x head) units:
//
//  step 1 (right factor; replaces _al_cl_y_fwd, wan/modules/monarch_attn.py:109-253)
//      work item = tile (unit, key block row k, kv block-frame f) against all (a, j) columns of a chunk of query
//      block-frames; one workgroup per CU, each taking an equal contiguous share of the tile list.
//      per tile: K[f,k,:,:], V[f,k,:,:] go row-major into LDS once, straight from global memory (the contractions
//      take K^T / V^T from transposing LDS reads), and for ALL columns of the chunk
//          S^T[l,(a,j)] = K[f,k,l,:] . Q[a,k,j,:]           (MFMA, wave = 32 (a,j) columns)
//          R = softmax_l(s S)       cl = sum_l R log2 R      (registers + one cross-half shuffle)
//          Kbar^T = K^T R^T,  Y^T = V^T R^T                  (MFMA; R^T is fed straight from the
//                                                             accumulator layout, see perm_row)
//      rows Kbar[a,j,(f,k),:], Y[a,j,(f,k),:] go to the workspace straight from the accumulators: one
//      v_permlane32_swap per dword pair leaves 8 consecutive head-dim elements per lane (16-byte stores).
//
//  step 2 (left factor; replaces _z_fwd, monarch_attn.py:698-842)
//      wave = (unit, a, j): streams its contiguous Kbar / Y rows once, 32 rows at a time, through its own part of
//      LDS (global_load_lds_dwordx4, one chunk ahead; no barriers: a wave waits for its own loads only),
//          S2^T[(f,k), i] = Kbar[(f,k),:] . Q[a,i,j,:]  - cl       online softmax over (f,k)
//          O^T[d, i]     += Y^T[d,(f,k)] P^T[(f,k), i]
//      with the Y^T operands from transposing LDS reads and the query rows in registers.
//
// The running output stays in fp32 for the whole KV range (the reference rounds it to 16 bit
// between KV chunks, monarch_attn.py:795,838).

#include "sfm_common.hpp"

namespace sfm {

// ------------------------------------------------------------------------------------------------
// step 1
// ------------------------------------------------------------------------------------------------
// The K and V tiles are staged row-major (64 rows of 2 D bytes, 16-byte chunks XOR-swizzled per row) straight
// from global memory into LDS (global_load_lds_dwordx4, two buffers per wave group) and the K^T / V^T operands of the
// contractions are transposing LDS reads (ds_read_tr16_b64): no staging registers, no transposes written to LDS,
// one barrier per tile.
typedef short s1_s16x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ u32x2 s1_read_tr(const char* lds, uint32_t off) {
    s1_s16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s1_s16x4 __attribute__((address_space(3)))*)(lds + off));
    return __builtin_bit_cast(u32x2, v);
}
__device__ __forceinline__ void s1_load_lds16(const char* base, uint32_t off, uint32_t lds_addr) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_addr), "v"(off), "s"(base) : "memory", "m0");
}
template <int CPR>
__device__ __forceinline__ int s1_swz(int r) {
    return CPR >= 16 ? (((r & 3) << 2) | ((r >> 2) & 3)) : ((((r >> 1) & 1) << 2) | ((r >> 2) & 3));
}
template <int D, int NT>
struct S1Lds {
    static constexpr int kRows = NT <= 2 ? 64 : 32 * NT;     // rows of a K / V tile
    static constexpr int kPitch = 2 * D, kTile = kRows * kPitch;
    static constexpr int kGroup = 4 * kTile;                 // [buffer][K tile | V tile]
    static __host__ __device__ constexpr size_t bytes() { return (size_t)kGroup; }
};

// NT: 32-row tiles of the key axis l (b2 <= 32 NT).  Up to two tiles a workgroup is two wave groups of at most 5 waves
//     (170 registers per wave); three and four tiles (b2 up to 128: the 720p and 1080p grids) run one group of up to 8
//     waves with 256 registers, whose tile buffers take 96 / 128 KB of LDS.
// WR: also write the right factor R (16 bit, 64 values per scratch row) to p.rb; the backward uses it.
// IT: a pass of the iterated refinement (wan/modules/monarch_attn.py:1716-1722): the logits are scaled per (a, f, k, j)
//     column and, after the first pass, the query operand of tile (f, k) is the column's representative p.rep[a, j, (f, k)]
//     instead of Q[a, k, j]; the operand is then fetched for every tile.
template <class E, int D, int NT, bool WR = false, bool IT = false>
__global__ __launch_bounds__(NT > 2 ? 512 : 640) __attribute__((amdgpu_waves_per_eu(NT > 2 ? 2 : 3, NT > 2 ? 2 : 3)))
void monarch_step1_kernel(MonarchArgs p) {
    using L = S1Lds<D, NT>;
    constexpr int CPR = D / 8;   // 16-byte chunks of a K/V row
    constexpr int DS = D / 16;   // contraction steps of the logits
    extern __shared__ __attribute__((aligned(256))) char lds_s1[];

    // A workgroup is `p.s1_groups` independent wave groups that share nothing but the barriers, each with
    // its own LDS tiles.  Two groups of 5 waves put 3,3,2,2 waves on the four SIMDs, which one group of 5
    // cannot (waves go to SIMDs round-robin).
    const int G = p.s1_groups;
    const int nthreads = blockDim.x / G;                  // threads of one group
    const int nwaves = nthreads >> 6;
    const int grp = __builtin_amdgcn_readfirstlane(threadIdx.x / nthreads);
    const int tid = threadIdx.x - grp * nthreads;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lane = tid & 63;
    const int m = lane & 31;
    const int hf = lane >> 5;
    const uint32_t piece = (uint32_t)(4 * ((m >> 3) & 1) + 2 * ((m >> 4) & 1) + hf) * 16;   // see the output stores below

    char* const lds = lds_s1 + grp * L::kGroup;
    const uint32_t lds0 = (uint32_t)(size_t)(__attribute__((address_space(3))) char*)lds;

    // Work items are K/V tiles t = ((ul * b1 + k) * n_achunks + ac) * nf + f, i.e. one kv block row (f, k) of
    // one unit against the query rows Q[a, k, :, :] of one chunk of query block-frames.  The launch has one
    // workgroup per CU and every workgroup takes an equal contiguous share of the tile list (its groups
    // alternate within the share), so no round of workgroups is left partly filled.  The query operands
    // stay in registers while consecutive tiles differ in f only.
    const int T = p.s1_total;
    const int t0 = (int)((int64_t)blockIdx.x * T / gridDim.x);
    const int t1 = (int)((int64_t)(blockIdx.x + 1) * T / gridDim.x);
    const int rounds = (t1 - t0 + G - 1) / G;
    const int mine = (t1 - t0 - grp + G - 1) / G;         // tiles of this group: t0 + grp, t0 + grp + G, ...
    if (mine <= 0) {                                      // still joins the barriers of the other group
        for (int r = 0; r < rounds; ++r) lds_barrier();
        return;
    }

    const int b2 = p.b2;
    const uint32_t qs1 = (uint32_t)p.qs[1], ks1 = (uint32_t)p.ks[1];
    const uint32_t fstep = p.ws_f ? p.ws_f : (uint32_t)p.b1 * p.ws_row;     // scratch rows between consecutive f

    struct Tile {
        int f, k, ul, ac, a0, ncols;
    };
    auto decode = [&](int t) {
        Tile x;
        x.f = t % p.nf;
        int r = t / p.nf;
        const int ac = r % p.n_achunks;
        r /= p.n_achunks;
        x.k = r % p.b1;
        x.ul = r / p.b1;
        x.ac = ac;
        x.a0 = ac * p.a_chunk;
        x.ncols = min(p.a_chunk, p.na - x.a0) * b2;
        return x;
    };

    // Tile x into buffer `buf`: LDS position P (in 16-byte units) holds chunk (P % CPR) ^ swz(row) of row P / CPR.
    // Rows past the end of a short tile (l >= b2) load row b2 - 1 again; their logits are masked below.  Every wave
    // issues the same number of loads for every tile, which the partial wait at the top of a round relies on.
    auto stage = [&](const Tile& x, int buf) {
        const int unit = p.unit0 + x.ul;
        const int b = unit / p.H, h = unit % p.H;
        const char* kg = (const char*)p.k + ((int64_t)b * p.ks[0] + (int64_t)h * p.ks[2]) * 2;
        const char* vg = (const char*)p.v + ((int64_t)b * p.vs[0] + (int64_t)h * p.vs[2]) * 2;
        const uint32_t krow0 = (uint32_t)p.kmap.row(x.f, x.k);        // uniform
        const uint32_t dst = lds0 + (uint32_t)buf * 2 * L::kTile;
        for (int g = wave; g < NT * (CPR / 2); g += nwaves) {         // 1 KB (64 / CPR rows) per step
            const int P = g * 64 + lane;
            const int r = P / CPR, c = (P % CPR) ^ s1_swz<CPR>(r);
            const uint32_t off = (krow0 + (uint32_t)min(r, b2 - 1)) * ks1 * 2 + (uint32_t)c * 16;
            s1_load_lds16(kg, off, dst + (uint32_t)g * 1024);
            s1_load_lds16(vg, off, dst + L::kTile + (uint32_t)g * 1024);
        }
    };
    // K rows 32 t + m as the logits' A operand
    const uint32_t a_off = (uint32_t)m * L::kPitch + (uint32_t)((hf ^ s1_swz<CPR>(m)) << 4);
    // K^T / V^T as the contractions' A operand: rows = head-dim 32 dt + m, 16 key rows per step in the order the
    // logits' accumulators hold them (two transposing reads of 4 x 4 blocks each)
    uint32_t tr[D / 32][2];
    {
        const int s16 = lane & 15, g16 = lane >> 4;
        const int rl = 4 * hf + (s16 >> 2);
        const int cl = 2 * (g16 & 1) + ((s16 & 3) >> 1);
#pragma unroll
        for (int dt = 0; dt < D / 32; ++dt)
#pragma unroll
            for (int half = 0; half < 2; ++half) {
                const int r = rl + 8 * half;
                tr[dt][half] = (uint32_t)(r * L::kPitch + (((4 * dt + cl) ^ s1_swz<CPR>(r)) << 4) + (s16 & 1) * 8);
            }
    }

    const float sc2 = p.scale * kLog2e;
    const f32x16 kZero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};

    // Everything from the logits to the output stores runs without a branch, and a lane whose column
    // index is past the chunk's last column works on that last column again (same values to the same
    // addresses).  The number of stores after a tile's loads is then the same on every path, so that the
    // wait for the loads can leave those stores in flight instead of draining them.
    u32x4 qb[DS];                                          // logits operand (B): this lane's query row
    uint32_t crow[4] = {0, 0, 0, 0};                       // byte offsets in the (f, k) slab of the four scratch rows this lane stores to
    uint32_t cloff = 0;                                    // same for cl
    int qkey = -1;
    float wsc = 1.f;                                       // IT: the column's logits factor

    Tile cur = decode(t0 + grp), nxt = cur;
    stage(cur, 0);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    for (int r = 0; r < rounds; ++r) {
        const bool fresh = r < mine;     // in its last round a group may have no tile left: it repeats its previous one
        // Vector memory operations complete in order: this wave's part of tile r has landed when only the Kbar / Y
        // stores of the round before (the last 8 * D / 64 operations it issued) are outstanding.
        if (D == 128) asm volatile("s_waitcnt vmcnt(16)" ::: "memory");
        else asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
        lds_barrier();                   // tile r is in LDS; every wave has finished reading the tile before it
        if (fresh) cur = nxt;
        const char* kt = lds + (r & 1) * 2 * L::kTile;
        const char* vt = kt + L::kTile;
        const int key = (cur.ul * p.b1 + cur.k) * p.n_achunks + cur.ac;       // one value per (unit, k, query chunk)
        const uint32_t srow = (uint32_t)cur.ul * p.ws_unit + (uint32_t)cur.k * p.ws_row + (uint32_t)cur.f * fstep;
        if ((IT && p.iter_mode == 2) || key != qkey) {
            qkey = key;
            const int unit = p.unit0 + cur.ul;
            const int b = unit / p.H, h = unit % p.H;
            const uint16_t* qg = (const uint16_t*)p.q + (int64_t)b * p.qs[0] + (int64_t)h * p.qs[2];
            const int cg = min(wave * 32 + m, cur.ncols - 1);
            const int cl_a = cg / b2;
            const int cj = cg - cl_a * b2;
            const int ca = cur.a0 + cl_a;
            const uint16_t* qrow = qg + ((uint32_t)(p.qmap.row(ca, cur.k) + cj) * qs1 + 8 * hf);
            if (IT) {
                wsc = 1.0f / (1.0f + 1e-6f);
                if (p.iter_mode == 2) {
                    const size_t rrow = (size_t)srow + (size_t)(ca * b2 + cj) * p.ws_aj;
                    qrow = (const uint16_t*)p.rep + rrow * D + 8 * hf;
                    wsc = fminf(1.0f / (p.wgt[rrow] + 1e-6f), 1e4f);
                }
            }
#pragma unroll
            for (int ds = 0; ds < DS; ++ds) qb[ds] = *(const u32x4*)(qrow + 16 * ds);
#pragma unroll
            for (int ds = 0; ds < DS; ++ds) asm volatile("" : "+v"(qb[ds]));      // waited for here, before the tile loads below
            cloff = (uint32_t)(ca * b2 + cj) * p.cl_aj * 4;
#pragma unroll
            for (int rb = 0; rb < 4; ++rb) {
                const int sg = min(wave * 32 + (m & 7) + 8 * rb, cur.ncols - 1);
                const int sa = sg / b2;
                crow[rb] = (uint32_t)((cur.a0 + sa) * b2 + (sg - sa * b2)) * p.ws_aj * (D * 2) + piece;
            }
        }
        if (r + 1 < rounds) {
            // the tile after this one; past the end of the share the current tile is loaded again and dropped
            const int tn = t0 + grp + (r + 1) * G;
            nxt = decode(tn < t1 ? tn : t0 + grp + (mine - 1) * G);
            stage(nxt, (r + 1) & 1);
        }

        u32x4 pb[2 * NT];                // R^T as B operands, 16 contraction rows per step
        {
            f32x16 s[NT];
#pragma unroll
            for (int t = 0; t < NT; ++t)
#pragma unroll
                for (int ds = 0; ds < DS; ++ds) {
                    const u32x4 a = *(const u32x4*)(kt + 32 * t * L::kPitch + (a_off ^ (uint32_t)(ds << 5)));
                    s[t] = E::mfma32(a, qb[ds], ds ? s[t] : kZero);
                }
            // block softmax over l (rows of S^T): 16 NT values here, the rest in lane ^ 32
            float mx = -INFINITY;
#pragma unroll
            for (int t = 0; t < NT; ++t)
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    int l = 32 * t + 8 * (v >> 2) + 4 * hf + (v & 3);
                    float zz = l < b2 ? (IT ? s[t][v] * sc2 * wsc : s[t][v] * sc2) : kMaskLogit;
                    s[t][v] = zz;
                    mx = fmaxf(mx, zz);
                }
            mx = xhalf_max(mx);
            float sum = 0.f, ent = 0.f;
#pragma unroll
            for (int t = 0; t < NT; ++t)
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    float zz = s[t][v];
                    float e = fast_exp2(zz - mx);        // exactly 0 for masked rows
                    sum += e;
                    ent += e * zz;
                    s[t][v] = e;
                }
            sum = xhalf_sum(sum);
            ent = xhalf_sum(ent);
            const float inv_l = 1.f / sum;
            // R = e / sum is rounded to 16 bit once, as the reference's right factor is
#pragma unroll
            for (int st = 0; st < 2 * NT; ++st) {
                const int t = st >> 1, v0 = 8 * (st & 1);
                pb[st].x = pack2<E>(s[t][v0 + 0] * inv_l, s[t][v0 + 1] * inv_l);
                pb[st].y = pack2<E>(s[t][v0 + 2] * inv_l, s[t][v0 + 3] * inv_l);
                pb[st].z = pack2<E>(s[t][v0 + 4] * inv_l, s[t][v0 + 5] * inv_l);
                pb[st].w = pack2<E>(s[t][v0 + 6] * inv_l, s[t][v0 + 7] * inv_l);
            }
            // sum_l R log2 R (both halves of a column hold, and store, the same value)
            {
                const size_t clrow = (size_t)cur.ul * p.cl_unit + (size_t)((uint32_t)cur.k * p.ws_row + (uint32_t)cur.f * fstep) * p.cl_row;
                *(float*)((char*)p.cl + clrow * 4 + cloff) = ent * inv_l - (mx + log2f(sum));
            }
            if (WR) {
                // R[l] for l = 16 st + 0..15: the lower half of the wave holds 0..3 and 8..11, the upper half 4..7 and
                // 12..15; exchanging the lower half's second pair with the upper half's first leaves 8 consecutive values
                char* rrow = (char*)p.rb + ((size_t)srow + cloff / 4) * 128 + 16 * hf;
#pragma unroll
                for (int st = 0; st < 2 * NT; ++st) {
                    auto rx = __builtin_amdgcn_permlane32_swap(pb[st].x, pb[st].z, false, false);
                    auto ry = __builtin_amdgcn_permlane32_swap(pb[st].y, pb[st].w, false, false);
                    const u32x4 w = {(uint32_t)rx[0], (uint32_t)ry[0], (uint32_t)rx[1], (uint32_t)ry[1]};
                    *(u32x4*)(rrow + 32 * st) = w;
                }
            }
        }
        // contractions with K^T then V^T, 32 head-dim columns at a time.  A 32 x 32 accumulator tile holds,
        // per lane (column c, half hf), head-dim 8g + 4hf + 0..3 for g = 0..3; swapping the g-odd dwords of the
        // lower half with the g-even dwords of the upper half (v_permlane32_swap) leaves 8 consecutive
        // elements per lane: the 16-byte piece 4 dt + 2 gp + hf of column c's 2D-byte scratch row.  Two more
        // exchanges, over a pair of head-dim blocks, trade lane bit 4 for gp (v_permlane16_swap) and lane
        // bit 3 for the block within the pair (a rotation by 8 within rows of 16 lanes).  Afterwards a lane
        // holds, for each of the four row groups rb, the piece 4 (dt0 + bit 3) + 2 bit 4 + hf of column
        // (c & 7) + 8 rb, so that one store instruction writes 128 contiguous bytes of each of 8 rows.
#pragma unroll
        for (int which = 0; which < 2; ++which) {
            const char* tbase = which == 0 ? kt : vt;
            char* og = (char*)(which == 0 ? p.kbar : p.y) + (size_t)srow * (D * 2);
#pragma unroll
            for (int dp = 0; dp < D / 64; ++dp) {
                uint32_t w[2][2][4];             // [block in pair][gp][dword]
#pragma unroll
                for (int dl = 0; dl < 2; ++dl) {
                    const int dt = 2 * dp + dl;
                    f32x16 acc;
#pragma unroll
                    for (int st = 0; st < 2 * NT; ++st) {
                        const u32x2 lo = s1_read_tr(tbase, tr[dt][0] + st * 16 * L::kPitch);
                        const u32x2 hi = s1_read_tr(tbase, tr[dt][1] + st * 16 * L::kPitch);
                        const u32x4 a = {lo.x, lo.y, hi.x, hi.y};
                        acc = E::mfma32(a, pb[st], st ? acc : kZero);
                    }
#pragma unroll
                    for (int gp = 0; gp < 2; ++gp) {
                        const int g0 = 2 * gp, g1 = 2 * gp + 1;
                        auto rx = __builtin_amdgcn_permlane32_swap(pack2<E>(acc[4 * g0 + 0], acc[4 * g0 + 1]),
                                                                   pack2<E>(acc[4 * g1 + 0], acc[4 * g1 + 1]), false, false);
                        auto ry = __builtin_amdgcn_permlane32_swap(pack2<E>(acc[4 * g0 + 2], acc[4 * g0 + 3]),
                                                                   pack2<E>(acc[4 * g1 + 2], acc[4 * g1 + 3]), false, false);
                        w[dl][gp][0] = rx[0]; w[dl][gp][1] = ry[0]; w[dl][gp][2] = rx[1]; w[dl][gp][3] = ry[1];
                    }
                    // lane bit 4 <-> gp: slot 0 then holds rows (c & 15), slot 1 rows (c & 15) + 16
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        auto x = __builtin_amdgcn_permlane16_swap(w[dl][0][q], w[dl][1][q], false, false);
                        w[dl][0][q] = x[0]; w[dl][1][q] = x[1];
                    }
                }
                // lane bit 3 <-> block within the pair
#pragma unroll
                for (int r4 = 0; r4 < 2; ++r4) {
                    u32x4 lo, hi;
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        const uint32_t a = w[0][r4][q], b = w[1][r4][q];
                        // row_ror:8 within 16 lanes; bank mask 0xc writes lanes 8..15 of a row, 0x3 lanes 0..7
                        lo[q] = (uint32_t)__builtin_amdgcn_update_dpp((int)a, (int)b, 0x128, 0xf, 0xc, false);
                        hi[q] = (uint32_t)__builtin_amdgcn_update_dpp((int)b, (int)a, 0x128, 0xf, 0x3, false);
                    }
                    // Non-temporal: the rows are read exactly once, by step 2, after the whole grid has finished.
                    // Ordinary stores leave them dirty in the caches and their write-back then competes with
                    // step 2's reads (measured at 4680 x 32760, 12 heads: step 1 +15 us, step 2 -45 us).
                    __builtin_nontemporal_store(lo, (u32x4*)(og + crow[2 * r4 + 0] + 128 * dp));
                    __builtin_nontemporal_store(hi, (u32x4*)(og + crow[2 * r4 + 1] + 128 * dp));
                }
            }
        }
    }
}

// ------------------------------------------------------------------------------------------------
// step 2
// ------------------------------------------------------------------------------------------------
// Per wave: [Kbar chunk | Y chunk | cl values, two buffers of 256 bytes], a chunk being 32 scratch rows of 2 D bytes,
// row-major with the 16-byte pieces XOR-swizzled per row as in step 1.  One buffer per matrix: the next chunk's Kbar rows
// are requested as soon as the logits have read the current ones, its Y rows as soon as the output products have, which
// keeps a chunk in flight with 17 KB of LDS per wave instead of 33 KB, so that two workgroups share a compute unit
// (two waves per SIMD, and the 1872 waves of the 480p chunk shape in one round instead of two).
template <int D>
struct S2Lds {
    static constexpr int kPitch = 2 * D, kTile = 32 * kPitch;
    static constexpr int kWave = 2 * kTile + 512;
    static __host__ __device__ constexpr size_t bytes() { return 4 * (size_t)kWave; }
};

__device__ __forceinline__ void s2_load_lds4(const char* base, uint32_t off, uint32_t lds_addr) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2" ::"s"(lds_addr), "v"(off), "s"(base) : "memory", "m0");
}

// The four waves of a workgroup share nothing: each streams the rows of its own (a, j) through its own part of LDS
// (global_load_lds_dwordx4, 1 KB contiguous per instruction, requested as soon as the buffer's last reader is done) and
// synchronises with its own loads only (vector memory operations complete in order, so waiting until only the loads
// issued after a tile's are outstanding means that tile has landed).
template <class E, int D>
__global__ __launch_bounds__(256) void monarch_step2_kernel(MonarchArgs p) {
    using L = S2Lds<D>;
    constexpr int DS = D / 16, DT = D / 32, CPR = D / 8;
    extern __shared__ __attribute__((aligned(256))) char lds_s2[];

    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lane = tid & 63;
    const int m = lane & 31;
    const int hf = lane >> 5;

    const int b2 = p.b2;
    const int njg = (b2 + 3) / 4;
    const int a = blockIdx.x / njg;
    const int jraw = (blockIdx.x % njg) * 4 + wave;
    const bool j_ok = jraw < b2;
    const int j = j_ok ? jraw : b2 - 1;
    const int ul = blockIdx.y;
    const int unit = p.unit0 + ul;
    const int b = unit / p.H, h = unit % p.H;
    const int i0 = blockIdx.z * 32;

    const int f_lim = p.causal ? min(p.nf, (a / p.causal + 1) * p.causal) : p.nf;
    const int r_lim = f_lim * p.b1;
    const int nch = (r_lim + 31) / 32;

    const int64_t blk = (int64_t)ul * p.ws_unit + (int64_t)(a * b2 + j) * p.ws_aj;   // in rows; the rows of one (a, j) are consecutive
    const char* kb = (const char*)p.kbar + blk * (2 * D);
    const char* yb = (const char*)p.y + blk * (2 * D);
    const char* clp = (const char*)(p.cl + (int64_t)ul * p.cl_unit + (int64_t)(a * b2 + j) * p.cl_aj);
    const uint32_t cl_ld = p.cl_row * 4;                  // bytes between the cl values of consecutive rows

    char* const wl = lds_s2 + wave * L::kWave;
    const uint32_t lds0 = (uint32_t)(size_t)(__attribute__((address_space(3))) char*)wl;

    // logits operand (B): this lane's query row Q[a, i0 + m, j, :] (zero past b1)
    u32x4 qb[DS];
    {
        const uint16_t* qg = (const uint16_t*)p.q + (int64_t)b * p.qs[0] + (int64_t)h * p.qs[2];
        const int i = min(i0 + m, p.b1 - 1);
        const uint16_t* qrow = qg + (p.qmap.row(a, i) + j) * p.qs[1] + 8 * hf;
#pragma unroll
        for (int ds = 0; ds < DS; ++ds) qb[ds] = *(const u32x4*)(qrow + 16 * ds);
#pragma unroll
        for (int ds = 0; ds < DS; ++ds) asm volatile("" : "+v"(qb[ds]));       // waited for here, before the first chunk's loads
        if (i0 + m >= p.b1) {
#pragma unroll
            for (int ds = 0; ds < DS; ++ds) qb[ds] = u32x4{0u, 0u, 0u, 0u};
        }
    }

    const uint32_t a_off = (uint32_t)m * L::kPitch + (uint32_t)((hf ^ s1_swz<CPR>(m)) << 4);   // Kbar row m as the logits' A operand
    uint32_t tr[DT][2];            // Y^T as the output's A operand: transposing reads, as in step 1
    {
        const int s16 = lane & 15, g16 = lane >> 4;
        const int rl = 4 * hf + (s16 >> 2);
        const int cl = 2 * (g16 & 1) + ((s16 & 3) >> 1);
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int half = 0; half < 2; ++half) {
                const int r = rl + 8 * half;
                tr[dt][half] = (uint32_t)(r * L::kPitch + (((4 * dt + cl) ^ s1_swz<CPR>(r)) << 4) + (s16 & 1) * 8);
            }
    }

    const float sc2 = p.scale * kLog2e;
    const f32x16 kZero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    f32x16 oacc[DT];               // O^T[d = 32 dt + 8 g + 4 hf + e, i = m]
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) oacc[dt] = kZero;
    float mrun = -INFINITY, lrun = 0.f;

    auto issue_k = [&](int n) {
#pragma unroll
        for (int g = 0; g < CPR / 2; ++g) {
            const int P = g * 64 + lane;
            const int r = P / CPR, c = (P % CPR) ^ s1_swz<CPR>(r);
            const uint32_t off = (uint32_t)min(32 * n + r, r_lim - 1) * (2 * D) + (uint32_t)c * 16;
            s1_load_lds16(kb, off, lds0 + (uint32_t)g * 1024);
        }
        s2_load_lds4(clp, (uint32_t)(32 * n + m) * cl_ld, lds0 + 2 * L::kTile + (uint32_t)(n & 1) * 256);   // lanes >= 32 repeat
    };
    auto issue_y = [&](int n) {
#pragma unroll
        for (int g = 0; g < CPR / 2; ++g) {
            const int P = g * 64 + lane;
            const int r = P / CPR, c = (P % CPR) ^ s1_swz<CPR>(r);
            const uint32_t off = (uint32_t)min(32 * n + r, r_lim - 1) * (2 * D) + (uint32_t)c * 16;
            s1_load_lds16(yb, off, lds0 + L::kTile + (uint32_t)g * 1024);
        }
    };
    issue_k(0);
    issue_y(0);
    for (int n = 0; n < nch; ++n) {
        // Kbar and cl of chunk n have landed when only the Y loads issued after them are outstanding
        if (D == 128) asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
        else asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
        const char* kt = wl;
        const char* yt = wl + L::kTile;
        const char* clt = wl + 2 * L::kTile + (n & 1) * 256;

        f32x16 s;
#pragma unroll
        for (int ds = 0; ds < DS; ++ds) {
            const u32x4 ak = *(const u32x4*)(kt + (a_off ^ (uint32_t)(ds << 5)));
            s = E::mfma32(ak, qb[ds], ds ? s : kZero);
        }
        f32x4 cc[4];
#pragma unroll
        for (int g = 0; g < 4; ++g) cc[g] = *(const f32x4*)(clt + (8 * g + 4 * hf) * 4);
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");       // the Kbar tile has been read: the next chunk's may land on it
        if (n + 1 < nch) issue_k(n + 1);

        float mx = -INFINITY;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            int r = 32 * n + 8 * (v >> 2) + 4 * hf + (v & 3);
            float z = r < r_lim ? s[v] * sc2 - cc[v >> 2][v & 3] : -INFINITY;
            s[v] = z;
            mx = fmaxf(mx, z);
        }
        mx = xhalf_max(mx);
        const float mnew = fmaxf(mrun, mx);        // finite: chunk n has at least one valid row
        const float alpha = exp2f(mrun - mnew);
        float psum = 0.f;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            float e = exp2f(s[v] - mnew);
            psum += e;
            s[v] = e;
        }
        lrun = lrun * alpha + psum;
        mrun = mnew;
        u32x4 pb[2];
#pragma unroll
        for (int st = 0; st < 2; ++st) {
            pb[st].x = pack2<E>(s[8 * st + 0], s[8 * st + 1]);
            pb[st].y = pack2<E>(s[8 * st + 2], s[8 * st + 3]);
            pb[st].z = pack2<E>(s[8 * st + 4], s[8 * st + 5]);
            pb[st].w = pack2<E>(s[8 * st + 6], s[8 * st + 7]);
        }
        // Y of chunk n has landed when only the Kbar / cl loads of chunk n + 1 are outstanding
        if (n + 1 < nch) {
            if (D == 128) asm volatile("s_waitcnt vmcnt(9)" ::: "memory");
            else asm volatile("s_waitcnt vmcnt(5)" ::: "memory");
        } else {
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        }
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
#pragma unroll
            for (int v = 0; v < 16; ++v) oacc[dt][v] *= alpha;
#pragma unroll
            for (int st = 0; st < 2; ++st) {
                const u32x2 lo = s1_read_tr(yt, tr[dt][0] + st * 16 * L::kPitch);
                const u32x2 hi = s1_read_tr(yt, tr[dt][1] + st * 16 * L::kPitch);
                const u32x4 ay = {lo.x, lo.y, hi.x, hi.y};
                oacc[dt] = E::mfma32(ay, pb[st], oacc[dt]);
            }
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");       // the Y tile has been read
        if (n + 1 < nch) issue_y(n + 1);
    }

    // epilogue: O[i, d] = O^T / l, turned through the wave's LDS (the operand buffers are dead: every load has landed)
    const float ltot = xhalf_sum(lrun);
    const float inv = 1.f / ltot;
    if (p.stats != nullptr && hf == 0 && j_ok && i0 + m < p.b1)
        p.stats[((int64_t)unit * (p.na * b2) + a * b2 + j) * p.stats_ld + i0 + m] = mrun + log2f(ltot);
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            u32x2 w;
            w.x = pack2<E>(oacc[dt][4 * g + 0] * inv, oacc[dt][4 * g + 1] * inv);
            w.y = pack2<E>(oacc[dt][4 * g + 2] * inv, oacc[dt][4 * g + 3] * inv);
            *(u32x2*)(wl + m * L::kPitch + (32 * dt + 8 * g + 4 * hf) * 2) = w;
        }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    {
        uint16_t* og = (uint16_t*)p.out + (int64_t)b * p.os[0] + (int64_t)h * p.os[2];
        for (int c = lane; c < 32 * CPR; c += 64) {
            int r = c / CPR, ch = c % CPR;
            int i = i0 + r;
            if (i < p.b1 && j_ok) {
                u32x4 w = *(const u32x4*)(wl + r * L::kPitch + ch * 16);
                *(u32x4*)(og + (p.qmap.row(a, i) + j) * p.os[1] + ch * 8) = w;
            }
        }
    }
}

// ------------------------------------------------------------------------------------------------
// iterated refinement: the next pass's query representatives (wan/modules/monarch_attn.py:1741-1744)
//   rep[a, j, r, :] = sum_i L[i, r] Q[a, i, j, :],   wgt[a, j, r] = sum_i L[i, r],   r = (f, k)
// with L[i, r] = exp2(s log2e <Q_i, Kbar_r> - cl_r - stats_i), stats = the left factor's row statistics that step 2 wrote.
// Step 2 with the operands' roles exchanged: one wave per (a, j) streams the column's Kbar rows 32 at a time through its
// LDS; the logits come out as S[i, r] (A = query rows, B = Kbar rows), so that a lane holds a column r, and
// rep^T[d, r] = sum_i Q^T[d, i] L[i, r] takes Q^T from transposing reads of the column's query rows, which sit in the
// wave's LDS for the whole kernel.  NQ = 32-row tiles of the query rows i (b1 <= 32 NQ <= 128: three frames tied per
// block give b1 = 90); with one tile the logits' A operand stays in registers, with more it is read from the LDS rows.
// A workgroup is 4 waves (NQ <= 2) or 3 (more LDS per wave).
// ------------------------------------------------------------------------------------------------
template <int D, int NQ>
struct RepLds {
    static constexpr int kPitch = 2 * D, kTile = 32 * kPitch;
    static constexpr int kBuf = kTile + 256;               // [Kbar chunk | cl values]
    static constexpr int kQ = 2 * kBuf;                    // offset of the query rows
    static constexpr int kWave = 2 * kBuf + NQ * kTile;
    static constexpr int kWaves = NQ <= 2 ? 4 : 3;
    static __host__ __device__ constexpr size_t bytes() { return (size_t)kWaves * kWave; }
};

template <class E, int D, int NQ>
__global__ __launch_bounds__(256) void monarch_rep_kernel(MonarchArgs p) {
    using L = RepLds<D, NQ>;
    constexpr int DS = D / 16, DT = D / 32, CPR = D / 8;
    extern __shared__ __attribute__((aligned(256))) char lds_s2[];

    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lane = tid & 63;
    const int m = lane & 31;
    const int hf = lane >> 5;

    const int b2 = p.b2;
    const int njg = (b2 + L::kWaves - 1) / L::kWaves;
    const int a = blockIdx.x / njg;
    const int jraw = (blockIdx.x % njg) * L::kWaves + wave;
    if (jraw >= b2) return;                               // the waves of a workgroup share nothing
    const int j = jraw;
    const int ul = blockIdx.y;
    const int unit = p.unit0 + ul;
    const int b = unit / p.H, h = unit % p.H;

    const int r_lim = p.nf * p.b1;
    const int nch = (r_lim + 31) / 32;
    const int64_t blk = (int64_t)ul * p.ws_unit + (int64_t)(a * b2 + j) * p.ws_aj;
    const char* kb = (const char*)p.kbar + blk * (2 * D);
    const char* clp = (const char*)(p.cl + (int64_t)ul * p.cl_unit + (int64_t)(a * b2 + j) * p.cl_aj);
    const uint32_t cl_ld = p.cl_row * 4;
    char* repb = (char*)p.rep + blk * (2 * D);
    float* wgt = p.wgt + blk;

    char* const wl = lds_s2 + wave * L::kWave;
    const uint32_t lds0 = (uint32_t)(size_t)(__attribute__((address_space(3))) char*)wl;
    char* const qt = wl + L::kQ;                          // the column's query rows, laid out like chunks of scratch rows

    const uint16_t* qg = (const uint16_t*)p.q + (int64_t)b * p.qs[0] + (int64_t)h * p.qs[2];
    // query rows into LDS (rows past b1 repeat the last one; their weights are zero)
#pragma unroll
    for (int g = 0; g < NQ * (CPR / 2); ++g) {
        const int P = g * 64 + lane;
        const int r = P / CPR, c = (P % CPR) ^ s1_swz<CPR>(r);
        const uint32_t off = (uint32_t)((p.qmap.row(a, min(r, p.b1 - 1)) + j) * p.qs[1] * 2) + (uint32_t)c * 16;
        s1_load_lds16((const char*)qg, off, lds0 + L::kQ + (uint32_t)g * 1024);
    }
    // one tile: the logits operand (A) is this lane's query row Q[a, m, j, :] (zero past b1), kept in registers
    u32x4 qa[DS];
    if constexpr (NQ == 1) {
        const uint16_t* qrow = qg + (p.qmap.row(a, min(m, p.b1 - 1)) + j) * p.qs[1] + 8 * hf;
#pragma unroll
        for (int ds = 0; ds < DS; ++ds) qa[ds] = *(const u32x4*)(qrow + 16 * ds);
#pragma unroll
        for (int ds = 0; ds < DS; ++ds) asm volatile("" : "+v"(qa[ds]));
        if (m >= p.b1) {
#pragma unroll
            for (int ds = 0; ds < DS; ++ds) qa[ds] = u32x4{0u, 0u, 0u, 0u};
        }
    }
    // the statistics of the 16 NQ rows whose logits this lane will hold
    float st[NQ][16];
    {
        const float* sp = p.stats + ((int64_t)unit * (p.na * b2) + a * b2 + j) * p.stats_ld;
#pragma unroll
        for (int qi = 0; qi < NQ; ++qi)
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int i = 32 * qi + 8 * (v >> 2) + 4 * hf + (v & 3);
                st[qi][v] = i < p.b1 ? sp[i] : 0.f;
            }
#pragma unroll
        for (int qi = 0; qi < NQ; ++qi)
#pragma unroll
            for (int v = 0; v < 16; ++v) asm volatile("" : "+v"(st[qi][v]));
    }

    // chunk n of the Kbar rows (and their cl values) into buffer `buf`
    auto issue = [&](int n, int buf) {
        const uint32_t dst = lds0 + (uint32_t)buf * L::kBuf;
#pragma unroll
        for (int g = 0; g < CPR / 2; ++g) {
            const int P = g * 64 + lane;
            const int r = P / CPR, c = (P % CPR) ^ s1_swz<CPR>(r);
            const uint32_t off = (uint32_t)min(32 * n + r, r_lim - 1) * (2 * D) + (uint32_t)c * 16;
            s1_load_lds16(kb, off, dst + (uint32_t)g * 1024);
        }
        s2_load_lds4(clp, (uint32_t)(32 * n + m) * cl_ld, dst + L::kTile);
    };
    const uint32_t b_off = (uint32_t)m * L::kPitch + (uint32_t)((hf ^ s1_swz<CPR>(m)) << 4);   // row m of a 32-row tile as an MFMA operand
    uint32_t tr[DT][2];            // Q^T as the representatives' A operand: transposing reads, as step 2 reads Y^T
    {
        const int s16 = lane & 15, g16 = lane >> 4;
        const int rl = 4 * hf + (s16 >> 2);
        const int cl = 2 * (g16 & 1) + ((s16 & 3) >> 1);
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int half = 0; half < 2; ++half) {
                const int r = rl + 8 * half;
                tr[dt][half] = (uint32_t)(r * L::kPitch + (((4 * dt + cl) ^ s1_swz<CPR>(r)) << 4) + (s16 & 1) * 8);
            }
    }

    const float sc2 = p.scale * kLog2e;
    const f32x16 kZero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};

    issue(0, 0);
    for (int n = 0; n < nch; ++n) {
        // everything older than the chunk requested last (the stores of the chunk before included) is waited for
        if (n + 1 < nch) {
            issue(n + 1, (n + 1) & 1);
            if (D == 128) asm volatile("s_waitcnt vmcnt(9)" ::: "memory");
            else asm volatile("s_waitcnt vmcnt(5)" ::: "memory");
        } else {
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        }
        const char* kt = wl + (n & 1) * L::kBuf;
        const float cc = *(const float*)(kt + L::kTile + m * 4);
        const bool rok = 32 * n + m < r_lim;
        float wsum = 0.f;
        u32x4 pb[NQ][2];
#pragma unroll
        for (int qi = 0; qi < NQ; ++qi) {
            f32x16 s;              // S[i = 32 qi + 8 g + 4 hf + e, r = 32 n + m]
#pragma unroll
            for (int ds = 0; ds < DS; ++ds) {
                const u32x4 bk = *(const u32x4*)(kt + (b_off ^ (uint32_t)(ds << 5)));
                u32x4 aq;
                if constexpr (NQ == 1) aq = qa[ds];
                else aq = *(const u32x4*)(qt + qi * L::kTile + (b_off ^ (uint32_t)(ds << 5)));
                s = E::mfma32(aq, bk, ds ? s : kZero);
            }
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int i = 32 * qi + 8 * (v >> 2) + 4 * hf + (v & 3);
                const float e = (rok && i < p.b1) ? exp2f(s[v] * sc2 - cc - st[qi][v]) : 0.f;
                s[v] = e;
                wsum += e;
            }
#pragma unroll
            for (int q = 0; q < 2; ++q) {
                pb[qi][q].x = pack2<E>(s[8 * q + 0], s[8 * q + 1]);
                pb[qi][q].y = pack2<E>(s[8 * q + 2], s[8 * q + 3]);
                pb[qi][q].z = pack2<E>(s[8 * q + 4], s[8 * q + 5]);
                pb[qi][q].w = pack2<E>(s[8 * q + 6], s[8 * q + 7]);
            }
        }
        wsum = xhalf_sum(wsum);
        if (hf == 0) wgt[32 * n + m] = wsum;
        char* rrow = repb + (size_t)(32 * n + m) * (2 * D);
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
            f32x16 acc;
#pragma unroll
            for (int qi = 0; qi < NQ; ++qi)
#pragma unroll
                for (int q = 0; q < 2; ++q) {
                    const u32x2 lo = s1_read_tr(qt + qi * L::kTile, tr[dt][0] + q * 16 * L::kPitch);
                    const u32x2 hi = s1_read_tr(qt + qi * L::kTile, tr[dt][1] + q * 16 * L::kPitch);
                    const u32x4 aq = {lo.x, lo.y, hi.x, hi.y};
                    acc = E::mfma32(aq, pb[qi][q], (qi | q) ? acc : kZero);
                }
            // rep^T[d = 32 dt + 8 g + 4 hf + e, r]: the half-swap leaves 8 consecutive d per lane
#pragma unroll
            for (int gp = 0; gp < 2; ++gp) {
                const int g0 = 2 * gp, g1 = 2 * gp + 1;
                auto rx = __builtin_amdgcn_permlane32_swap(pack2<E>(acc[4 * g0 + 0], acc[4 * g0 + 1]),
                                                           pack2<E>(acc[4 * g1 + 0], acc[4 * g1 + 1]), false, false);
                auto ry = __builtin_amdgcn_permlane32_swap(pack2<E>(acc[4 * g0 + 2], acc[4 * g0 + 3]),
                                                           pack2<E>(acc[4 * g1 + 2], acc[4 * g1 + 3]), false, false);
                const u32x4 o = {(uint32_t)rx[0], (uint32_t)ry[0], (uint32_t)rx[1], (uint32_t)ry[1]};
                *(u32x4*)(rrow + (32 * dt + 16 * gp + 8 * hf) * 2) = o;
            }
        }
    }
}

// ------------------------------------------------------------------------------------------------
// host launch
// ------------------------------------------------------------------------------------------------
bool monarch_mfma_supported(int dtype, int D, int b2) {
    return (dtype == SFM_BF16 || dtype == SFM_F16) && (D == 64 || D == 128) && b2 >= 1 && b2 <= 128;
}

int cu_count() {
    static thread_local int cached_dev = -1, cached = 0;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return 256;
    if (dev != cached_dev) {
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
        cached = n;
        cached_dev = dev;
    }
    return cached;
}

// Enqueues step 1 (with the right factor written too when a.rb is set).
template <class E, int D>
static int enqueue_step1(const MonarchArgs& a, int nunits, hipStream_t stream, const void* fn_override = nullptr) {
    const int ncols = a.a_chunk * a.b2;
    const int ntiles = (ncols + 31) / 32;
    const int nwaves = ntiles < 4 ? 4 : ntiles;   // a wave per 32 (a, j) columns, at least 4 to share the tile loads
    if (ntiles < 1 || nwaves > 8) {
        set_error("internal: step-1 launch shape (a_chunk=%d, b2=%d)", a.a_chunk, a.b2);
        return SFM_ERR_UNSUPPORTED;
    }
    const int nt = (a.b2 + 31) / 32;
    const int groups = nwaves <= 5 && nt <= 2 ? 2 : 1;  // wave groups per workgroup (<= 10 waves in all)
    const size_t lds1 = (nt == 4 ? S1Lds<D, 4>::bytes() : nt == 3 ? S1Lds<D, 3>::bytes() : S1Lds<D, 2>::bytes()) * groups;
    if (nt > 2 && a.rb) {
        set_error("internal: the right factor is written for b2 <= 64 only");
        return SFM_ERR_UNSUPPORTED;
    }
    const void* fn = fn_override ? fn_override
                     : nt == 4 ? (const void*)monarch_step1_kernel<E, D, 4, false>
                     : nt == 3 ? (const void*)monarch_step1_kernel<E, D, 3, false>
                     : nt == 2 ? (a.rb ? (const void*)monarch_step1_kernel<E, D, 2, true> : (const void*)monarch_step1_kernel<E, D, 2, false>)
                               : (a.rb ? (const void*)monarch_step1_kernel<E, D, 1, true> : (const void*)monarch_step1_kernel<E, D, 1, false>);
    if (lds1 > 64 * 1024) {
        hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds1);
        if (e != hipSuccess) {
            set_error("hipFuncSetAttribute failed: %s", hipGetErrorString(e));
            return SFM_ERR_HIP;
        }
    }
    MonarchArgs a1 = a;
    a1.s1_total = a.nf * a.b1 * nunits * a.n_achunks;
    a1.s1_groups = groups;
    // one workgroup per CU (a CU holds one: 3 waves per SIMD), fewer when there are not two tiles for each
    int wgs = a.s1_wgs > 0 ? a.s1_wgs : cu_count();
    if (wgs > (a1.s1_total + groups - 1) / groups) wgs = (a1.s1_total + groups - 1) / groups;
    void* args[] = {&a1};
    hipError_t e = hipLaunchKernel(fn, dim3(wgs), dim3(nwaves * 64 * groups), args, lds1, stream);
    if (e != hipSuccess) {
        set_error("hip launch failed: %s", hipGetErrorString(e));
        return SFM_ERR_HIP;
    }
    return SFM_OK;
}

template <class E, int D>
static int launch_t(const MonarchArgs& a, int nunits, hipStream_t stream, const StepEvents* ev) {
    if (ev) (void)hipEventRecord(ev->ev[0], stream);
    MonarchArgs a0 = a;
    a0.rb = nullptr;
    if (int rc = enqueue_step1<E, D>(a0, nunits, stream)) return rc;
    if (ev) (void)hipEventRecord(ev->ev[1], stream);
    const int njg = (a.b2 + 3) / 4;
    dim3 g2(a.na * njg, nunits, (a.b1 + 31) / 32);
    {
        hipError_t e = hipFuncSetAttribute((const void*)monarch_step2_kernel<E, D>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                           (int)S2Lds<D>::bytes());
        if (e != hipSuccess) {
            set_error("hipFuncSetAttribute failed: %s", hipGetErrorString(e));
            return SFM_ERR_HIP;
        }
    }
    hipLaunchKernelGGL((monarch_step2_kernel<E, D>), g2, dim3(256), S2Lds<D>::bytes(), stream, a);
    if (ev) (void)hipEventRecord(ev->ev[2], stream);
    hipError_t err = hipGetLastError();
    if (err != hipSuccess) {
        set_error("hip launch failed: %s", hipGetErrorString(err));
        return SFM_ERR_HIP;
    }
    return SFM_OK;
}

template <class E, int D>
static int launch_step1_t(const MonarchArgs& a, int nunits, hipStream_t stream) {
    return enqueue_step1<E, D>(a, nunits, stream);
}

int launch_monarch_step1(const MonarchArgs& a, int dtype, int nunits, hipStream_t stream) {
    if (dtype == SFM_BF16)
        return a.D == 128 ? launch_step1_t<BF16, 128>(a, nunits, stream) : launch_step1_t<BF16, 64>(a, nunits, stream);
    return a.D == 128 ? launch_step1_t<F16, 128>(a, nunits, stream) : launch_step1_t<F16, 64>(a, nunits, stream);
}

bool monarch_iter_mfma_supported(int dtype, int D, int b1, int b2) {
    return monarch_mfma_supported(dtype, D, b2) && b1 >= 1 && b1 <= 128;
}

template <class E, int D, int NQ>
static int launch_rep_t(const MonarchArgs& a, int nunits, hipStream_t stream) {
    using L = RepLds<D, NQ>;
    hipError_t e = hipFuncSetAttribute((const void*)monarch_rep_kernel<E, D, NQ>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)L::bytes());
    if (e != hipSuccess) {
        set_error("hipFuncSetAttribute failed: %s", hipGetErrorString(e));
        return SFM_ERR_HIP;
    }
    const int njg = (a.b2 + L::kWaves - 1) / L::kWaves;
    hipLaunchKernelGGL((monarch_rep_kernel<E, D, NQ>), dim3(a.na * njg, nunits), dim3(64 * L::kWaves), L::bytes(), stream, a);
    return SFM_OK;
}

// num_iters passes of [step 1 with the pass's query operands | step 2 | representatives for the next pass]; the last
// pass's step 2 writes the output (the earlier ones write it too: it is overwritten).
template <class E, int D>
static int launch_iter_t(const MonarchArgs& a, int nunits, int num_iters, hipStream_t stream) {
    const int njg = (a.b2 + 3) / 4;
    const int nq = (a.b1 + 31) / 32;
    const dim3 g2(a.na * njg, nunits, nq);
    const int nt = (a.b2 + 31) / 32;
    const void* fn1 = nt == 4 ? (const void*)monarch_step1_kernel<E, D, 4, false, true>
                    : nt == 3 ? (const void*)monarch_step1_kernel<E, D, 3, false, true>
                    : nt == 2 ? (const void*)monarch_step1_kernel<E, D, 2, false, true>
                              : (const void*)monarch_step1_kernel<E, D, 1, false, true>;
    hipError_t e = hipFuncSetAttribute((const void*)monarch_step2_kernel<E, D>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)S2Lds<D>::bytes());
    if (e != hipSuccess) {
        set_error("hipFuncSetAttribute failed: %s", hipGetErrorString(e));
        return SFM_ERR_HIP;
    }
    for (int it = 0; it < num_iters; ++it) {
        const bool last = it + 1 == num_iters;
        MonarchArgs a1 = a;
        a1.rb = nullptr;
        a1.iter_mode = it == 0 ? 1 : 2;
        if (int rc = enqueue_step1<E, D>(a1, nunits, stream, fn1)) return rc;
        MonarchArgs a2 = a;
        if (last) a2.stats = nullptr;
        hipLaunchKernelGGL((monarch_step2_kernel<E, D>), g2, dim3(256), S2Lds<D>::bytes(), stream, a2);
        if (!last) {
            const int rc = nq == 1 ? launch_rep_t<E, D, 1>(a, nunits, stream) : nq == 2 ? launch_rep_t<E, D, 2>(a, nunits, stream)
                         : nq == 3 ? launch_rep_t<E, D, 3>(a, nunits, stream) : launch_rep_t<E, D, 4>(a, nunits, stream);
            if (rc) return rc;
        }
    }
    e = hipGetLastError();
    if (e != hipSuccess) {
        set_error("hip launch failed: %s", hipGetErrorString(e));
        return SFM_ERR_HIP;
    }
    return SFM_OK;
}

int launch_monarch_iter_mfma(const MonarchArgs& a, int dtype, int nunits, int num_iters, hipStream_t stream) {
    if (!monarch_iter_mfma_supported(dtype, a.D, a.b1, a.b2) || a.causal || !a.rep || !a.wgt || !a.stats ||
        (int)a.stats_ld < (a.b1 + 31) / 32 * 32) {
        set_error("internal: iterated MFMA launch");
        return SFM_ERR_UNSUPPORTED;
    }
    if (dtype == SFM_BF16)
        return a.D == 128 ? launch_iter_t<BF16, 128>(a, nunits, num_iters, stream) : launch_iter_t<BF16, 64>(a, nunits, num_iters, stream);
    return a.D == 128 ? launch_iter_t<F16, 128>(a, nunits, num_iters, stream) : launch_iter_t<F16, 64>(a, nunits, num_iters, stream);
}

int launch_monarch_mfma(const MonarchArgs& a, int dtype, int nunits, hipStream_t stream, const StepEvents* ev) {
    if (dtype == SFM_BF16)
        return a.D == 128 ? launch_t<BF16, 128>(a, nunits, stream, ev) : launch_t<BF16, 64>(a, nunits, stream, ev);
    return a.D == 128 ? launch_t<F16, 128>(a, nunits, stream, ev) : launch_t<F16, 64>(a, nunits, stream, ev);
}

}  // namespace sfm
