// The linear layers of the causal Wan attention block with their element-wise tails fused into the matrix product's
// epilogue, bf16 / fp16 on gfx950 MFMA:
//
//   SFM_EPI_NONE           out = x W^T + bias                                   (q/k/v, cross-attention projections)
//   SFM_EPI_GELU_TANH      out = gelu_tanh(x W^T + bias)                        (wan/modules/model.py:648-650, FFN up)
//   SFM_EPI_GATE_RESIDUAL  out = res + (x W^T + bias) * gate[frame of the row]  (wan/modules/causal_model.py:1189-1204:
//                          attention output projection and FFN down with the adaLN gates; gate = null: out = res + ...)
//
// Rounding points are those of the eager chain the epilogue replaces: the product plus bias is rounded to the tensor
// dtype (the nn.Linear output), GELU is evaluated on that in fp32 and rounded, the gated product is rounded and the
// residual sum is rounded.
//
// A workgroup of four waves owns 256 weight rows (output columns) x 64 TB activation rows of the output, TB = 4 or 2;
// a wave owns 128 x 32 TB of it (4 x TB MFMA 32x32x16 blocks, 64 TB accumulator registers, one wave per SIMD).  The
// weight rows are the MFMA A operand and the activation rows the B operand, so that a lane ends up with channels of ONE
// row and the half-swap of the other kernels turns them into 16-byte stores.  K is walked 64 elements at a time: 128
// bytes of a row are one cache line, and row pieces of half a line fetch every line twice (measured: 16.8 TB/s from the
// L2s with 64-byte pieces, 28.5 TB/s with 128-byte pieces).  Both operands go from global memory straight into LDS
// (global_load_lds_dwordx4, 8 rows per instruction) through a ring of five 32 KB slots, each holding the weight rows or
// the activation rows of one 64-wide stage, so that about three half stages are in flight while one stage is being
// multiplied.  Rows sit two to a 256-byte LDS line and the 16-byte pieces of a row are XOR-ed with the line index, so
// that the 16 lanes of an operand read hit 64 different banks.  LDS operand reads and load requests are issued one by
// one between the matrix instructions.  Tiles are numbered so that the workgroups resident on one XCD (every eighth
// one) cover a compact patch of the output and share their operand slabs in that XCD's L2.

#include <hip/hip_runtime.h>

#include "sfm_attn.h"
#include "sfm_common.hpp"

namespace sfm {
namespace {

constexpr int kTileN = 256;                  // weight rows (output columns) per workgroup
constexpr int kKS = 64;                      // K elements per stage: 128-byte row pieces, whole cache lines
constexpr int kSlotBytes = kTileN * kKS * 2; // a half stage: the weight rows or the activation rows of a stage
constexpr int kRing = 5;                     // slots
constexpr int kGroupM = 8;                   // row tiles per patch of the tile order

struct GemmArgs {
    const char* x;          // [M, K] rows x_stride apart
    const char* w;          // [N, K] contiguous
    const uint16_t* bias;   // [N] or null
    const char* res;        // [M, N] rows res_stride apart (may alias out) or null
    const uint16_t* gate;   // [frames, N] rows gate_stride apart, or null
    char* out;              // [M, N] rows out_stride apart
    int64_t M;
    int N, K;
    int64_t x_stride, out_stride, res_stride, gate_stride;
    int rows_per_frame;
    int tm, tn;             // tiles along M and N
};

__device__ __forceinline__ void bg_load_lds16(const char* base, uint32_t off, uint32_t lds_addr) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_addr), "v"(off), "s"(base) : "memory", "m0");
}
// waits until at most N of this wave's global loads are outstanding (they complete in order), then the barrier
template <int N>
__device__ __forceinline__ void bg_wait_stage() { asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(N) : "memory"); }

// LDS operand reads and their waits are written out, so that the reads can sit between the matrix instructions
template <int OFF>
__device__ __forceinline__ u32x4 bg_lds_read16(uint32_t addr) {
    u32x4 r;
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(r) : "v"(addr), "n"(OFF));
    return r;
}
template <int NF>
__device__ __forceinline__ void bg_wait_frags(u32x4 (&f)[NF]) {
    static_assert(NF == 8 || NF == 6, "4 weight blocks + 4 or 2 activation blocks");
    if constexpr (NF == 8)
        asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(f[0]), "+v"(f[1]), "+v"(f[2]), "+v"(f[3]), "+v"(f[4]), "+v"(f[5]), "+v"(f[6]), "+v"(f[7]));
    else
        asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(f[0]), "+v"(f[1]), "+v"(f[2]), "+v"(f[3]), "+v"(f[4]), "+v"(f[5]));
}

__device__ __forceinline__ float gelu_tanh(float x) {
    // 0.5 x (1 + tanh(u)) with u = sqrt(2/pi) (x + 0.044715 x^3), written as x / (1 + exp(-2u)): no cancellation
    // where tanh approaches -1
    const float u = 0.7978845608028654f * (x + 0.044715f * x * x * x);
    return x / (1.f + __expf(-2.f * u));
}

// One k step: 4 TB matrix instructions on the operand set fc (blocks 0..3: weights, 4..: activations).  The LDS reads of
// the next step's set fn (FETCH) follow the first 4 + TB of them one by one; NLOAD global -> LDS requests (rows
// off[LOAD0 ...] of the half stage at `base`, LDS destination mb + j * 4096) follow instructions of the second half, so
// that the issue cycles of both run under the matrix pipe instead of in front of it.
#define BG_KS(I)                                                                                                   \
    if constexpr ((I) < 4 * TB) {                                                                                  \
        acc[(I) / TB][(I) % TB] = E::mfma32(fc[(I) / TB], fc[4 + (I) % TB], acc[(I) / TB][(I) % TB]);              \
        __builtin_amdgcn_sched_barrier(0);                                                                         \
        if constexpr (FETCH && (I) < 4 + TB) {                                                                     \
            fn[(I)] = bg_lds_read16<((I) & 3) * 4096>((I) < 4 ? aa : bb);                                          \
            __builtin_amdgcn_sched_barrier(0);                                                                     \
        }                                                                                                          \
        if constexpr ((I) >= kFirst && ((I) - kFirst) % kStep == 0 && ((I) - kFirst) / kStep < NLOAD) {            \
            constexpr int j = LOAD0 + ((I) - kFirst) / kStep;                                                      \
            bg_load_lds16(base, off[j], mb + (uint32_t)j * 4096);                                                  \
            __builtin_amdgcn_sched_barrier(0);                                                                     \
        }                                                                                                          \
    }
template <class E, int TB, bool FETCH, int NLOAD, int LOAD0, int NOFF>
__device__ __forceinline__ void bg_kstep(f32x16 (&acc)[4][TB], const u32x4 (&fc)[4 + TB], u32x4 (&fn)[4 + TB], uint32_t aa,
                                         uint32_t bb, const char* base, const uint32_t (&off)[NOFF], uint32_t mb) {
    constexpr int kFirst = 2 * TB;                                     // the second half of the matrix instructions
    constexpr int kStep = NLOAD > 0 && 2 * TB / NLOAD > 1 ? 2 * TB / NLOAD : 1;
    static_assert(NLOAD * kStep <= 2 * TB + kStep - 1 && LOAD0 + NLOAD <= NOFF, "requests fit the second half");
    BG_KS(0) BG_KS(1) BG_KS(2) BG_KS(3) BG_KS(4) BG_KS(5) BG_KS(6) BG_KS(7)
    BG_KS(8) BG_KS(9) BG_KS(10) BG_KS(11) BG_KS(12) BG_KS(13) BG_KS(14) BG_KS(15)
}
#undef BG_KS

template <class E, int EPI, int TB>
__global__ __launch_bounds__(256) void block_gemm_kernel(GemmArgs p) {
    constexpr int kTileM = 64 * TB;                       // activation rows (output rows) per workgroup
    constexpr int NB = 2 * TB;                            // load instructions per wave of an activation half stage
    extern __shared__ __attribute__((aligned(256))) char lds[];
    const uint32_t lds0 = (uint32_t)(size_t)(__attribute__((address_space(3))) char*)lds;
    const int tid = threadIdx.x, lane = tid & 63, m = lane & 31, hf = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wn = wave & 1, wm = wave >> 1;

    // ---- which tile: every eighth workgroup shares an XCD; give each XCD a contiguous run of the patch order
    const int ntiles = p.tm * p.tn;
    const int per_xcd = (ntiles + 7) / 8;
    const int v = (int)(blockIdx.x % 8) * per_xcd + (int)(blockIdx.x / 8);
    if (v >= ntiles) return;
    const int patch = v / (kGroupM * p.tn);
    const int first = patch * kGroupM;
    const int gsize = min(kGroupM, p.tm - first);
    const int within = v - patch * kGroupM * p.tn;
    const int64_t m0 = (int64_t)(first + within % gsize) * kTileM;
    const int n0 = (within / gsize) * kTileN;

    // ---- what this lane stages: instruction j of a wave fills the 8 rows of block 4 j + wave of a half stage, 128
    // bytes each; lane -> (row of the block, piece position); rows sit two to a 256-byte LDS line and the piece a
    // position holds is XOR-ed with the line index (row >> 1) & 7
    const int g_row = lane >> 3;
    const int g_c = (lane & 7) ^ ((((wave & 1) << 2) + (lane >> 4)) & 7);
    uint32_t w_off[8], x_off[NB];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const int n = min(n0 + (4 * j + wave) * 8 + g_row, p.N - 1);
        w_off[j] = (uint32_t)((int64_t)n * p.K * 2 + g_c * 16);
    }
#pragma unroll
    for (int j = 0; j < NB; ++j) {
        const int64_t row = min(m0 + (4 * j + wave) * 8 + g_row, p.M - 1);
        x_off[j] = (uint32_t)(row * p.x_stride * 2 + g_c * 16);
    }

    f32x16 acc[4][TB];
#pragma unroll
    for (int cb = 0; cb < 4; ++cb)
#pragma unroll
        for (int tb = 0; tb < TB; ++tb)
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[cb][tb][i] = 0.f;

    // operand read addresses of the four 16-wide k steps of a stage, relative to the half stage's slot: row base + the
    // swizzled piece
    const int sw = (m >> 1) & 7;
    uint32_t ka[4], kb[4];
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
        const uint32_t ko = (uint32_t)(((2 * ks + hf) ^ sw) << 4);
        ka[ks] = lds0 + (uint32_t)((wn * 128 + m) * 128) + ko;
        kb[ks] = lds0 + (uint32_t)((wm * 32 * TB + m) * 128) + ko;
    }

    // LDS is a ring of five 32 KB slots; half stage h (2 s: the weight rows of stage s, 2 s + 1: its activation rows)
    // lives in slot h % 5.  Iteration s multiplies stage s in four k steps; the operands of a step are read from LDS
    // during the step before.  Before its last step a wave has read all of stage s: it waits for its own loads of
    // stage s + 1, meets the others at the barrier, and requests the activation half of stage s + 2 into the slot of
    // the weights of stage s; the weight half of stage s + 3 follows during the next iteration's first three steps
    // into the slot of the activations of stage s.  About three half stages are in flight at any time.
    const int nstage = p.K / kKS;
    const uint32_t wv = lds0 + (uint32_t)wave * 1024;
    auto half_w = [&](const char* base, uint32_t slot) {
#pragma unroll
        for (int j = 0; j < 8; ++j) bg_load_lds16(base, w_off[j], wv + slot * kSlotBytes + (uint32_t)j * 4096);
    };
    auto half_x = [&](const char* base, uint32_t slot) {
#pragma unroll
        for (int j = 0; j < NB; ++j) bg_load_lds16(base, x_off[j], wv + slot * kSlotBytes + (uint32_t)j * 4096);
    };
    half_w(p.w, 0);
    half_x(p.x, 1);
    if (nstage > 1) {
        half_w(p.w + kKS * 2, 2);
        half_x(p.x + kKS * 2, 3);
    }
    if (nstage > 2) {
        half_w(p.w + 2 * kKS * 2, 4);
        bg_wait_stage<16 + NB>();                          // a weight half is 8 load instructions per wave
    } else if (nstage > 1) {
        bg_wait_stage<8 + NB>();
    } else {
        bg_wait_stage<0>();
    }
    u32x4 f0[4 + TB], f1[4 + TB];
    f0[0] = bg_lds_read16<0>(ka[0]);
    f0[1] = bg_lds_read16<4096>(ka[0]);
    f0[2] = bg_lds_read16<8192>(ka[0]);
    f0[3] = bg_lds_read16<12288>(ka[0]);
    f0[4] = bg_lds_read16<0>(kb[0] + kSlotBytes);
    f0[5] = bg_lds_read16<4096>(kb[0] + kSlotBytes);
    if constexpr (TB == 4) {
        f0[6] = bg_lds_read16<8192>(kb[0] + kSlotBytes);
        f0[7] = bg_lds_read16<12288>(kb[0] + kSlotBytes);
    }

    const char* f_w = p.w + 3 * kKS * 2;                   // weight half of stage 3: the next one to request
    const char* f_x = p.x + 2 * kKS * 2;                   // activation half of stage 2
    uint32_t hs = 0;                                       // slot of the weights of the stage being multiplied
    auto wrap = [](uint32_t h) { return h >= 5 ? h - 5 : h; };
    // LA: request the weight half of stage s + 2 during the first three steps; LB: the activation half of stage
    // s + 2 during the last; W8: 8 requests (a weight half) may stay outstanding at the barrier; LAST: no barrier
#define BG_ITER(LA, LB, W8, LAST)                                                                                   \
    {                                                                                                               \
        const uint32_t sa = hs * kSlotBytes, sb = wrap(hs + 1) * kSlotBytes;                                        \
        const uint32_t mba = wv + wrap(hs + 4) * kSlotBytes;                                                        \
        bg_wait_frags(f0);                                                                                          \
        bg_kstep<E, TB, true, LA ? 3 : 0, 0>(acc, f0, f1, ka[1] + sa, kb[1] + sb, f_w, w_off, mba);                 \
        bg_wait_frags(f1);                                                                                          \
        bg_kstep<E, TB, true, LA ? 3 : 0, 3>(acc, f1, f0, ka[2] + sa, kb[2] + sb, f_w, w_off, mba);                 \
        bg_wait_frags(f0);                                                                                          \
        bg_kstep<E, TB, true, LA ? 2 : 0, 6>(acc, f0, f1, ka[3] + sa, kb[3] + sb, f_w, w_off, mba);                 \
        if (LA) f_w += kKS * 2;                                                                                     \
        bg_wait_frags(f1);                                  /* this wave has read all of the stage */               \
        if (!LAST) {                                                                                                \
            if (W8) bg_wait_stage<8>(); else bg_wait_stage<0>();                                                    \
            const uint32_t na = wrap(hs + 2) * kSlotBytes, nb = wrap(hs + 3) * kSlotBytes;                          \
            bg_kstep<E, TB, true, LB ? NB : 0, 0>(acc, f1, f0, ka[0] + na, kb[0] + nb, f_x, x_off, wv + sa);        \
            if (LB) f_x += kKS * 2;                                                                                 \
            hs = wrap(hs + 2);                                                                                      \
        } else {                                                                                                    \
            bg_kstep<E, TB, false, 0, 0>(acc, f1, f0, 0, 0, f_x, x_off, 0);                                         \
        }                                                                                                           \
    }
    if (nstage >= 3) {
        BG_ITER(false, true, true, false)
        for (int s = 1; s + 2 < nstage; ++s) BG_ITER(true, true, true, false)
    }
    if (nstage >= 2) BG_ITER(false, false, false, false)
    BG_ITER(false, false, false, true)
#undef BG_ITER

    // ---- epilogue: lane (m, hf) of block (cb, tb) holds output row 32 tb + m, channels 8 g + 4 hf + (i & 3) (i = 4 g + ..)
    const int cw = n0 + wn * 128;
#pragma unroll
    for (int cb = 0; cb < 4; ++cb) {
        const int cbase = cw + 32 * cb;
        float bia[16];
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const int c = cbase + 8 * g + 4 * hf;
            u32x2 bv = {0u, 0u};
            if (p.bias != nullptr && c + 4 <= p.N) bv = *(const u32x2*)(p.bias + c);
            bia[4 * g + 0] = E::to_float((uint16_t)(bv.x & 0xffffu));
            bia[4 * g + 1] = E::to_float((uint16_t)(bv.x >> 16));
            bia[4 * g + 2] = E::to_float((uint16_t)(bv.y & 0xffffu));
            bia[4 * g + 3] = E::to_float((uint16_t)(bv.y >> 16));
        }
#pragma unroll
        for (int tb = 0; tb < TB; ++tb) {
            const int64_t row = m0 + wm * 32 * TB + 32 * tb + m;
            const bool rok = row < p.M;
            const int64_t rc = rok ? row : p.M - 1;
            float val[16];
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                val[i] = acc[cb][tb][i] + bia[i];
                if (EPI == SFM_EPI_GELU_TANH) val[i] = gelu_tanh(E::to_float(E::from_float(val[i])));
            }
#pragma unroll
            for (int gp = 0; gp < 2; ++gp) {
                const int g0 = 2 * gp, g1 = 2 * gp + 1;
                auto rx = __builtin_amdgcn_permlane32_swap(pack2<E>(val[4 * g0 + 0], val[4 * g0 + 1]),
                                                           pack2<E>(val[4 * g1 + 0], val[4 * g1 + 1]), false, false);
                auto ry = __builtin_amdgcn_permlane32_swap(pack2<E>(val[4 * g0 + 2], val[4 * g0 + 3]),
                                                           pack2<E>(val[4 * g1 + 2], val[4 * g1 + 3]), false, false);
                u32x4 o = {(uint32_t)rx[0], (uint32_t)ry[0], (uint32_t)rx[1], (uint32_t)ry[1]};
                const int c = cbase + 16 * gp + 8 * hf;             // this lane's 8 consecutive channels of its row
                const bool ok = rok && c + 8 <= p.N;
                if (EPI == SFM_EPI_GATE_RESIDUAL) {
                    u32x4 rv = {0u, 0u, 0u, 0u}, gv = {0u, 0u, 0u, 0u};
                    if (c + 8 <= p.N) {
                        rv = *(const u32x4*)(p.res + (rc * p.res_stride + c) * 2);
                        if (p.gate != nullptr) gv = *(const u32x4*)(p.gate + (rc / p.rows_per_frame) * p.gate_stride + c);
                    }
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
#pragma clang fp contract(off)      // two eager ops in the reference: no fma
                        float y0 = E::to_float((uint16_t)(o[i] & 0xffffu)), y1 = E::to_float((uint16_t)(o[i] >> 16));
                        if (p.gate != nullptr) {
                            const float p0 = y0 * E::to_float((uint16_t)(gv[i] & 0xffffu));
                            const float p1 = y1 * E::to_float((uint16_t)(gv[i] >> 16));
                            y0 = E::to_float(E::from_float(p0));
                            y1 = E::to_float(E::from_float(p1));
                        }
                        o[i] = pack2<E>(E::to_float((uint16_t)(rv[i] & 0xffffu)) + y0, E::to_float((uint16_t)(rv[i] >> 16)) + y1);
                    }
                }
                if (ok) *(u32x4*)(p.out + (row * p.out_stride + c) * 2) = o;
            }
        }
    }
}

template <class E, int EPI, int TB>
int launch_tile(const GemmArgs& a0, hipStream_t st) {
    static bool configured = false;      // per instantiation and process (the attribute belongs to the function, not to a
                                         // device: every device of the process runs the same code object); racing
                                         // callers set the same value
    if (!configured) {
        hipError_t e = hipFuncSetAttribute((const void*)block_gemm_kernel<E, EPI, TB>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                           kRing * kSlotBytes);
        if (e != hipSuccess) {
            set_error("sfm_linear: hipFuncSetAttribute failed: %s", hipGetErrorString(e));
            return SFM_ERR_HIP;
        }
        configured = true;
    }
    GemmArgs a = a0;
    a.tm = (int)((a.M + 64 * TB - 1) / (64 * TB));
    a.tn = (a.N + kTileN - 1) / kTileN;
    const int ntiles = a.tm * a.tn;
    hipLaunchKernelGGL((block_gemm_kernel<E, EPI, TB>), dim3((unsigned)((ntiles + 7) / 8 * 8)), dim3(256), kRing * kSlotBytes, st, a);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        set_error("sfm_linear: launch failed: %s", hipGetErrorString(e));
        return SFM_ERR_HIP;
    }
    return SFM_OK;
}

// 256 x 256 tiles move the fewest operand bytes per product; 128-row tiles are taken when they fill the compute units
// so much better that it pays (few 256-row tiles: N = 1536 at 4680 rows is 114 of them on 256 compute units).
static bool half_tiles_pay(int64_t M, int N) {
    const int64_t cus = cu_count();
    const int64_t tn = (N + kTileN - 1) / kTileN;
    const int64_t t4 = (M + 255) / 256 * tn, t2 = (M + 127) / 128 * tn;
    const double r4 = (double)((t4 + cus - 1) / cus), r2 = (double)((t2 + cus - 1) / cus) * 0.62;   // rounds x time of a tile
    return r2 < r4;
}

template <class E, int EPI>
int launch_epi(const GemmArgs& a, int tile_rows, hipStream_t st) {
    const bool half = tile_rows == 128 || (tile_rows == 0 && half_tiles_pay(a.M, a.N));
    return half ? launch_tile<E, EPI, 2>(a, st) : launch_tile<E, EPI, 4>(a, st);
}

template <class E>
int launch_dtype(const GemmArgs& a, int epilogue, int tile_rows, hipStream_t st) {
    if (epilogue == SFM_EPI_GELU_TANH) return launch_epi<E, SFM_EPI_GELU_TANH>(a, tile_rows, st);
    if (epilogue == SFM_EPI_GATE_RESIDUAL) return launch_epi<E, SFM_EPI_GATE_RESIDUAL>(a, tile_rows, st);
    return launch_epi<E, SFM_EPI_NONE>(a, tile_rows, st);
}

}  // namespace

int launch_linear(const sfm_linear_desc& d, const void* x, const void* w, const void* bias, const void* res, const void* gate,
                  void* out, hipStream_t stream) {
    GemmArgs a;
    a.x = (const char*)x;
    a.w = (const char*)w;
    a.bias = (const uint16_t*)bias;
    a.res = (const char*)res;
    a.gate = (const uint16_t*)gate;
    a.out = (char*)out;
    a.M = d.M;
    a.N = d.N;
    a.K = d.K;
    a.x_stride = d.x_stride;
    a.out_stride = d.out_stride;
    a.res_stride = d.res_stride;
    a.gate_stride = d.gate_stride;
    a.rows_per_frame = d.rows_per_frame > 0 ? d.rows_per_frame : 1;
    a.tm = a.tn = 0;
    return d.dtype == SFM_BF16 ? launch_dtype<BF16>(a, d.epilogue, d.tile_rows, stream) : launch_dtype<F16>(a, d.epilogue, d.tile_rows, stream);
}

}  // namespace sfm
