// Dense (non-causal) softmax attention of a query chunk against a KV-cache prefix, and the cache
// row copy used by the *_with_kv_cache entry points.
//
// Replaces attention() (wan/modules/attention.py:141-187, SDPA branch) and the Triton _attn_fwd
// (wan/modules/attn_patch.py:20-110).
//
// MFMA kernel (bf16 / fp16, head_dim 64 or 128): workgroup = 256 or 128 queries of one (batch, head) in 8 or 4 waves,
// wave = 32 queries; with 8 waves a compute unit holds one workgroup and streams every K / V tile once instead of
// twice (3 % faster at 4680 x 32760 on random operands, 6 % on zeros: the chip's power limit takes the rest).  Per 64-key tile (K and V rows in LDS, row-major, 16-byte chunks XOR-swizzled):
//     S^T[l, q] = K[l,:] . Q[q,:]          online softmax per query column (lane)
//     O^T[d, q] += V^T[d, l] P^T[l, q]     V^T comes from transposing LDS reads (ds_read_tr16_b64), P^T from the
//                                          accumulator layout (perm_row)
// Tiles go from global memory straight into LDS (global_load_lds_dwordx4), two K and two V buffers, one
// barrier per tile.  A wave's matrix and vector work are interleaved in its instruction stream: the logits of
// tile n + 1 are contracted while the exponentials of tile n are taken, and the maximum of tile n + 1 is reduced
// while tile n's P V products run.

#include "sfm_common.hpp"

namespace sfm {

template <int D, int NW = 4>
struct DnLds {
    static constexpr int kCPR = D / 8;                  // 16-byte chunks per row
    static constexpr int kPitch = 2 * D;                // bytes per row
    static constexpr int kMat = 64 * kPitch;            // one 64-row tile
    static constexpr int kK = 0, kV = 2 * kMat;         // K tiles 0/1, then V tiles 0/1
    static constexpr int kStage = NW * 32 * (2 * D + 16);  // output staging, NW waves x 32 rows
    static constexpr int kTotal = 4 * kMat > kStage ? 4 * kMat : kStage;
    // chunk c of row r sits at chunk position c ^ swz(r); depends on r mod 16 only
    static __device__ __forceinline__ int swz(int r) {
        return D >= 128 ? (((r & 3) << 2) | ((r >> 2) & 3)) : ((((r >> 1) & 1) << 2) | ((r >> 2) & 3));
    }
};

typedef short dn_s16x4 __attribute__((ext_vector_type(4)));

// Transposing LDS read: within each group of 16 lanes, lane i receives element i % 4 of the 8 bytes addressed
// by lanes i/4, i/4 + 4, i/4 + 8, i/4 + 12.  With lane s of a group addressing row s / 4, columns
// 4 (s % 4) .. + 3 of a 4 x 16 block, lane i ends up with column i of the four rows.
__device__ __forceinline__ u32x2 dn_read_tr(const char* lds, uint32_t off) {
    dn_s16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((dn_s16x4 __attribute__((address_space(3)))*)(lds + off));
    return __builtin_bit_cast(u32x2, v);
}

// 16 bytes per lane from global memory into LDS without passing through registers: lane i of the wave reads
// base + off (off per lane, unsigned 32 bit) and writes LDS bytes [lds_addr + 16 i, + 16).  `base` and `lds_addr`
// are the same in every lane.  The load counts in vmcnt like any other; the compiler does not know that it
// writes LDS, so the code that reads the tile waits (dn_wait_tiles) and synchronises explicitly.
__device__ __forceinline__ void dn_load_lds16(const char* base, uint32_t off, uint32_t lds_addr) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_addr), "v"(off), "s"(base) : "memory", "m0");
}
__device__ __forceinline__ void dn_wait_tiles() { asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

template <class E, int D, int NW>
__global__ __launch_bounds__(64 * NW) __attribute__((amdgpu_waves_per_eu(2, 2))) void dense_fwd_kernel(sfm_dense_desc p, const uint16_t* __restrict__ q,
                                                        const uint16_t* __restrict__ kp,
                                                        const uint16_t* __restrict__ vp, uint16_t* __restrict__ out,
                                                        float* __restrict__ lse) {
    using L = DnLds<D, NW>;
    constexpr int DS = D / 16, DT = D / 32;
    constexpr int NTH = 64 * NW;
    extern __shared__ __attribute__((aligned(256))) char lds[];
    const uint32_t lds0 = (uint32_t)(size_t)(__attribute__((address_space(3))) char*)lds;

    const int tid = threadIdx.x, lane = tid & 63, m = lane & 31, hf = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    // the query blocks of one (batch, head) go to one XCD: its K / V rows are fetched from memory once, not once per XCD
    const int nq = p.q_tokens, nk = p.kv_tokens;
    const int nqb = (nq + 32 * NW - 1) / (32 * NW);
    const int total = nqb * p.B * p.H;
    const int item = xcd_item(total);
    if (item >= total) return;
    const int unit = item / nqb;
    const int b = unit / p.H, h = unit % p.H;
    const int q0 = (item - unit * nqb) * (32 * NW) + wave * 32;

    const char* kg = (const char*)(kp + (int64_t)b * p.k_stride[0] + (int64_t)h * p.k_stride[2]);
    const char* vg = (const char*)(vp + (int64_t)b * p.v_stride[0] + (int64_t)h * p.v_stride[2]);
    const uint32_t krs = (uint32_t)p.k_stride[1] * 2, vrs = (uint32_t)p.v_stride[1] * 2;     // row strides in bytes

    // query operand (B of the logits MFMA): lane (m, hf) holds Q[q0 + m][16 ds + 8 hf + 0..7]
    u32x4 qb[DS];
    {
        const int qi = min(q0 + m, nq - 1);
        const uint16_t* qrow = q + (int64_t)b * p.q_stride[0] + (int64_t)qi * p.q_stride[1] + (int64_t)h * p.q_stride[2] + 8 * hf;
#pragma unroll
        for (int ds = 0; ds < DS; ++ds) qb[ds] = *(const u32x4*)(qrow + 16 * ds);
#pragma unroll
        for (int ds = 0; ds < DS; ++ds) asm volatile("" : "+v"(qb[ds]));      // loaded before any tile is awaited
    }

    // staging: thread `tid` moves chunks tid, tid + 256, ... of a tile.  LDS position P (16-byte units) holds
    // global chunk (P % kCPR) ^ swz(row) of row P / kCPR; a wave's 64 positions are contiguous.  Chunk i of a
    // thread is kRPC rows below chunk i - 1 in the same (swizzled) column, so one per-thread byte offset serves
    // all of them and everything else (tile, i) goes into the scalar base address.
    constexpr int kCh = 64 * L::kCPR / NTH;            // 4 chunks per thread for D = 128 with 4 waves
    constexpr int kRPC = NTH / L::kCPR;                // rows between a thread's consecutive chunks (multiple of 16)
    const int srow = tid / L::kCPR;
    const uint32_t scol = (uint32_t)(((tid % L::kCPR) ^ L::swz(srow)) * 16);
    const uint32_t koff = (uint32_t)srow * krs + scol, voff = (uint32_t)srow * vrs + scol;
    // full tile
    auto stage = [&](const char* g, uint32_t rs, uint32_t off, int tile, uint32_t dst) {
#pragma unroll
        for (int i = 0; i < kCh; ++i)
            dn_load_lds16(g + (size_t)(tile * 64 + i * kRPC) * rs, off, lds0 + dst + (uint32_t)(i * NTH + wave * 64) * 16);
    };
    // possibly ragged tile: rows past the last key repeat the last key (their logits are masked)
    auto stage_clamped = [&](const char* g, uint32_t rs, int tile, uint32_t dst) {
        const char* base = g + (size_t)tile * 64 * rs;
        const int last = nk - 1 - 64 * tile;           // >= 0
#pragma unroll
        for (int i = 0; i < kCh; ++i)
            dn_load_lds16(base, (uint32_t)min(srow + i * kRPC, last) * rs + scol, lds0 + dst + (uint32_t)(i * NTH + wave * 64) * 16);
    };

    // logits: A operand = K rows; lane (m, hf) reads chunk 2 ds + hf of row 32 t + m
    const uint32_t sA0 = (uint32_t)m * L::kPitch + (uint32_t)((hf ^ L::swz(m)) << 4);
    // output: A operand = V^T.  For head-dim rows 32 dt + 0..31 and contraction step st lane (m, hf) needs keys
    // l = 16 st + 4 hf + {0..3} and + 8 + {0..3} (the order in which the logits' accumulators hold l) of
    // head-dim column 32 dt + m: two transposing reads.
    // Head-dim block dt only changes chunk bits 2..3 of the (swizzled) chunk index: address ^ (dt << 6).
    uint32_t trA[2];
    {
        const int s16 = lane & 15, g16 = lane >> 4;
        const int rl = 4 * hf + (s16 >> 2);
        const int cl = 2 * (g16 & 1) + ((s16 & 3) >> 1);
#pragma unroll
        for (int half = 0; half < 2; ++half) {
            const int r = rl + 8 * half;
            trA[half] = (uint32_t)r * L::kPitch + (uint32_t)((cl ^ L::swz(r)) << 4) + (uint32_t)(s16 & 1) * 8;
        }
    }

    f32x16 oacc[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int v = 0; v < 16; ++v) oacc[dt][v] = 0.f;
    float mrun = -INFINITY, lrun = 0.f;            // running max (scaled, base-2 units) and sum
    const float sc2 = p.sm_scale * kLog2e;
    const int ntile = (nk + 63) / 64;
    const int lrem = nk - 64 * (ntile - 1);        // valid keys of the last tile (1..64)

    // Both phases of an iteration are sequences of steps, one MFMA each, with the step's A operand read from
    // LDS kAhead steps earlier into a ring of registers and a slice of the vector work beside it.
    constexpr int NA = 2 * DS;                     // logits steps: (ds, t) = (j / 2, j % 2)
    constexpr int NP = 4 * DT;                     // output steps: (dt, st) = (j / 4, j % 4)
    constexpr int kVA = 32 / NA;                   // logits per lane exponentiated beside one logits step
    constexpr int kVP = 32 / NP;                   // logits per lane reduced beside one output step
    constexpr int kAhead = 3, kRing = kAhead + 1;

    // `kbuf` / `vbuf` are constants, so that they and the row offsets go into the instructions' offset fields
    auto read_k = [&](uint32_t kbuf, int j) -> u32x4 {
        return *(const u32x4*)(lds + (sA0 ^ (uint32_t)((j >> 1) << 5)) + kbuf + (j & 1) * 32 * L::kPitch);
    };
    auto read_v = [&](uint32_t vbuf, int j) -> u32x4 {
        const u32x2 lo = dn_read_tr(lds + (trA[0] ^ (uint32_t)((j >> 2) << 6)), vbuf + (j & 3) * 16 * L::kPitch);
        const u32x2 hi = dn_read_tr(lds + (trA[1] ^ (uint32_t)((j >> 2) << 6)), vbuf + (j & 3) * 16 * L::kPitch);
        return u32x4{lo.x, lo.y, hi.x, hi.y};
    };
    auto mask_tail = [&](f32x16* s) {              // logits of the keys past the end of a ragged last tile
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int l = 32 * t + 8 * (v >> 2) + 4 * hf + (v & 3);
                s[t][v] = l < lrem ? s[t][v] : kMaskLogit;
            }
    };
    // value i (0..31) of a lane's logits, in the order the P^T operands take them
#define DN_SVAL(s, i) s[(i) >> 4][(i) & 15]

    f32x16 sbuf[2][2];                             // logits of tile n in sbuf[n & 1]
    u32x4 ring[kRing];                             // A operands on their way from LDS
    u32x4 pb[4];

    // ---- prologue: tile 0 (and K of tile 1) into LDS, logits and maximum of tile 0
    stage_clamped(kg, krs, 0, L::kK);
    stage_clamped(vg, vrs, 0, L::kV);
    if (ntile > 1) stage_clamped(kg, krs, 1, L::kK + L::kMat);
    dn_wait_tiles();
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int v = 0; v < 16; ++v) sbuf[0][t][v] = 0.f;
#pragma unroll
    for (int j = 0; j < NA; ++j) sbuf[0][j & 1] = E::mfma32(read_k(L::kK, j), qb[j >> 1], sbuf[0][j & 1]);
    if (ntile == 1 && lrem < 64) mask_tail(sbuf[0]);
    {
        float mx = sbuf[0][0][0];
#pragma unroll
        for (int i = 1; i < 32; ++i) mx = fmaxf(mx, DN_SVAL(sbuf[0], i));
        mrun = xhalf_max(mx) * sc2;
    }

    // One iteration consumes tile n (logits in sbuf[n & 1], maximum already folded into mrun) and, unless it is
    // the last one, produces the logits of tile n + 1.  PAR = n & 1 fixes every LDS buffer at compile time.
    // kind 0: the last tile; 1: any other tile; 2: a tile at least three before the last one (the tiles it
    // fetches are full ones: no tests, no clamping)
    auto iteration = [&](int n, auto par_c, auto kind_c) {
        constexpr int PAR = decltype(par_c)::value, kind = decltype(kind_c)::value;
        constexpr bool has_next = kind != 0;
        constexpr uint32_t kbuf = L::kK + (uint32_t)(PAR ^ 1) * L::kMat;     // K of tile n + 1; K of n + 2 goes where K of n was
        constexpr uint32_t vbuf = L::kV + (uint32_t)PAR * L::kMat;           // V of tile n; V of n + 1 goes to the other one
        f32x16* scur = sbuf[PAR];
        f32x16* snext = sbuf[PAR ^ 1];
        dn_wait_tiles();                 // K(n+1) and V(n) are in LDS; the buffers of K(n) and V(n-1) are free
        if (kind == 2) {
            stage(kg, krs, koff, n + 2, L::kK + (uint32_t)PAR * L::kMat);
            stage(vg, vrs, voff, n + 1, L::kV + (uint32_t)(PAR ^ 1) * L::kMat);
        } else if (kind == 1) {
            // only the last tile can be ragged
            if (n + 3 < ntile) stage(kg, krs, koff, n + 2, L::kK + (uint32_t)PAR * L::kMat);
            else if (n + 3 == ntile) stage_clamped(kg, krs, n + 2, L::kK + (uint32_t)PAR * L::kMat);
            if (n + 2 < ntile) stage(vg, vrs, voff, n + 1, L::kV + (uint32_t)(PAR ^ 1) * L::kMat);
            else stage_clamped(vg, vrs, n + 1, L::kV + (uint32_t)(PAR ^ 1) * L::kMat);
        }

        // phase A: logits of tile n + 1 beside the exponentials of tile n
        float psum = 0.f;
        if (has_next) {
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int v = 0; v < 16; ++v) snext[t][v] = 0.f;
#pragma unroll
            for (int j = 0; j < kAhead; ++j) ring[j % kRing] = read_k(kbuf, j);
        } else {
#pragma unroll
            for (int j = 0; j < kAhead; ++j) ring[(NA + j) % kRing] = read_v(vbuf, j);
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int j = 0; j < NA; ++j) {
            if (has_next) {
                const int ja = j + kAhead;
                if (ja < NA) ring[ja % kRing] = read_k(kbuf, ja);
                else ring[ja % kRing] = read_v(vbuf, ja - NA);
                snext[j & 1] = E::mfma32(ring[j % kRing], qb[j >> 1], snext[j & 1]);
            }
#pragma unroll
            for (int i = kVA * j; i < kVA * (j + 1); ++i) {
                const float e = fast_exp2(fmaf(DN_SVAL(scur, i), sc2, -mrun));
                psum += e;
                DN_SVAL(scur, i) = e;
            }
#pragma unroll
            for (int i = kVA * j; i < kVA * (j + 1); i += 2) pb[i >> 3][(i >> 1) & 3] = pack2<E>(DN_SVAL(scur, i), DN_SVAL(scur, i + 1));
            __builtin_amdgcn_sched_barrier(0);
        }
        lrun += psum;
        if (kind == 1) {
            if (n + 2 == ntile && lrem < 64) mask_tail(snext);
        }

        // phase B: P V of tile n beside the maximum of tile n + 1
        float mx = has_next ? snext[0][0] : 0.f;
#pragma unroll
        for (int j = 0; j < NP; ++j) {
            if (j + kAhead < NP) ring[(NA + j + kAhead) % kRing] = read_v(vbuf, j + kAhead);
            oacc[j >> 2] = E::mfma32(ring[(NA + j) % kRing], pb[j & 3], oacc[j >> 2]);
            if (has_next) {
#pragma unroll
                for (int i = kVP * j; i < kVP * (j + 1); ++i) mx = fmaxf(mx, DN_SVAL(snext, i));
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        if (has_next) {
            // rescale the running output only when some query of the wave raised its maximum
            const float mnew = fmaxf(mrun, xhalf_max(mx) * sc2);
            if (__builtin_amdgcn_ballot_w64(mnew > mrun) != 0) {
                const float alpha = fast_exp2(mrun - mnew);
                lrun *= alpha;
#pragma unroll
                for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                    for (int v = 0; v < 16; ++v) oacc[dt][v] *= alpha;
                mrun = mnew;
            }
        }
    };
    using c0 = std::integral_constant<int, 0>;
    using c1 = std::integral_constant<int, 1>;
    using c2 = std::integral_constant<int, 2>;
    int n = 0;
    for (; n + 4 < ntile; n += 2) {
        iteration(n, c0{}, c2{});
        iteration(n + 1, c1{}, c2{});
    }
    for (; n + 2 < ntile; n += 2) {                // at most once
        iteration(n, c0{}, c1{});
        iteration(n + 1, c1{}, c1{});
    }
    if (n + 1 < ntile) {
        iteration(n, c0{}, c1{});
        iteration(n + 1, c1{}, c0{});
    } else {
        iteration(n, c0{}, c0{});
    }
#undef DN_SVAL

    const float ltot = xhalf_sum(lrun);
    const float inv = 1.f / ltot;
    if (lse != nullptr && hf == 0 && q0 + m < nq)
        lse[((int64_t)b * p.H + h) * nq + q0 + m] = (mrun + log2f(ltot)) * kLn2;

    __syncthreads();                                   // tiles are dead; reuse LDS as output stage
    constexpr int kSP = D + 8;                         // u16 per staged row
    uint16_t* stage_o = (uint16_t*)lds + wave * 32 * kSP;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            u32x2 w;
            w.x = pack2<E>(oacc[dt][4 * g + 0] * inv, oacc[dt][4 * g + 1] * inv);
            w.y = pack2<E>(oacc[dt][4 * g + 2] * inv, oacc[dt][4 * g + 3] * inv);
            *(u32x2*)(stage_o + m * kSP + 32 * dt + 8 * g + 4 * hf) = w;
        }
    __syncthreads();
    {
        uint16_t* og = out + (int64_t)b * p.o_stride[0] + (int64_t)h * p.o_stride[2];
        constexpr int CH = D / 8;
        for (int c = lane; c < 32 * CH; c += 64) {
            int r = c / CH, ch = c % CH;
            if (q0 + r < nq) {
                u32x4 w = *(const u32x4*)(stage_o + r * kSP + ch * 8);
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
        // 256 queries per workgroup (8 waves, one workgroup per compute unit) stream every K / V tile once per compute
        // unit instead of twice; short query ranges keep 128 so that more compute units get a workgroup
        const bool wide = (int64_t)((d.q_tokens + 255) / 256) * d.B * d.H >= cu_count() / 2;
        const uint16_t* qq = (const uint16_t*)q;
        const uint16_t* kk = (const uint16_t*)k;
        const uint16_t* vv = (const uint16_t*)v;
        uint16_t* oo = (uint16_t*)out;
        auto go = [&](auto kern, int nw, size_t ldsb) -> int {
            hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)ldsb);
            if (e != hipSuccess) {
                set_error("hipFuncSetAttribute failed: %s", hipGetErrorString(e));
                return SFM_ERR_HIP;
            }
            const int total = (d.q_tokens + 32 * nw - 1) / (32 * nw) * d.B * d.H;
            dim3 grid(xcd_grid(total));
            hipLaunchKernelGGL(kern, grid, dim3(64 * nw), ldsb, stream, d, qq, kk, vv, oo, lse);
            return SFM_OK;
        };
        int rc;
        if (d.dtype == SFM_BF16) {
            if (d.D == 128) rc = wide ? go(dense_fwd_kernel<BF16, 128, 8>, 8, DnLds<128, 8>::kTotal) : go(dense_fwd_kernel<BF16, 128, 4>, 4, DnLds<128, 4>::kTotal);
            else rc = wide ? go(dense_fwd_kernel<BF16, 64, 8>, 8, DnLds<64, 8>::kTotal) : go(dense_fwd_kernel<BF16, 64, 4>, 4, DnLds<64, 4>::kTotal);
        } else {
            if (d.D == 128) rc = wide ? go(dense_fwd_kernel<F16, 128, 8>, 8, DnLds<128, 8>::kTotal) : go(dense_fwd_kernel<F16, 128, 4>, 4, DnLds<128, 4>::kTotal);
            else rc = wide ? go(dense_fwd_kernel<F16, 64, 8>, 8, DnLds<64, 8>::kTotal) : go(dense_fwd_kernel<F16, 64, 4>, 4, DnLds<64, 4>::kTotal);
        }
        if (rc) return rc;
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
