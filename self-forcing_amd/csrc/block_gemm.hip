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
// A workgroup of four waves owns a 256-row x 256-column tile of the output; a wave owns 128 x 128 of it (4 x 4 MFMA
// 32x32x16 blocks, 256 accumulator registers, one wave per SIMD).  The weight rows are the MFMA A operand and the
// activation rows the B operand, so that a lane ends up with channels of ONE row and the half-swap of the other kernels
// turns them into 16-byte stores.  K is walked 32 elements at a time: both operands' 64-byte row pieces go from
// global memory straight into LDS (global_load_lds_dwordx4, 16 rows per instruction) through a ring of four 32 KB
// stage buffers; a stage is requested three iterations before it is multiplied, and the one barrier of an iteration
// sits between the two halves of its matrix instructions, so that the wait for the next stage's data runs under
// them.  Rows sit four to a 256-byte LDS line and the 16-byte pieces of a row are XOR-ed with the line index, so that
// the 16 lanes of an operand read hit 64 different banks.  Tiles are numbered so that the workgroups resident on one
// XCD (every eighth one) cover a compact patch of the output and share their operand slabs in that XCD's L2.

#include <hip/hip_runtime.h>

#include "sfm_attn.h"
#include "sfm_common.hpp"

namespace sfm {
namespace {

constexpr int kTile = 256;                   // output rows and columns per workgroup
constexpr int kKS = 32;                      // K elements per stage
constexpr int kStageBytes = 2 * kTile * kKS * 2;
constexpr int kRing = 4;                     // stage buffers
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

// byte offset of 16-byte piece c (0..3) of row r in a stage region of 64-byte rows
__device__ __forceinline__ uint32_t piece_off(int r, int c) {
    const int line = r >> 2;
    return (uint32_t)(line * 256 + ((r & 3) << 6) + ((c ^ (line & 3)) << 4));
}

__device__ __forceinline__ void bg_load_lds16(const char* base, uint32_t off, uint32_t lds_addr) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_addr), "v"(off), "s"(base) : "memory", "m0");
}
// waits until at most N of this wave's global loads are outstanding (they complete in order), then the barrier
template <int N>
__device__ __forceinline__ void bg_wait_stage() { asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(N) : "memory"); }

// LDS operand reads and their waits are written out: LDS operations complete in order, so "at most 8 outstanding" after
// issuing the next set of 8 means the previous set has arrived; the compiler's own counting waits for everything here.
template <int OFF>
__device__ __forceinline__ u32x4 bg_lds_read16(uint32_t addr) {
    u32x4 r;
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(r) : "v"(addr), "n"(OFF));
    return r;
}
template <int N>
__device__ __forceinline__ void bg_wait_frags(u32x4* f) {
    asm volatile("s_waitcnt lgkmcnt(%8)"
                 : "+v"(f[0]), "+v"(f[1]), "+v"(f[2]), "+v"(f[3]), "+v"(f[4]), "+v"(f[5]), "+v"(f[6]), "+v"(f[7])
                 : "n"(N));
}

__device__ __forceinline__ float gelu_tanh(float x) {
    // 0.5 x (1 + tanh(u)) with u = sqrt(2/pi) (x + 0.044715 x^3), written as x / (1 + exp(-2u)): no cancellation
    // where tanh approaches -1
    const float u = 0.7978845608028654f * (x + 0.044715f * x * x * x);
    return x / (1.f + __expf(-2.f * u));
}

template <class E, int EPI>
__global__ __launch_bounds__(256) void block_gemm_kernel(GemmArgs p) {
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
    const int64_t m0 = (int64_t)(first + within % gsize) * kTile;
    const int n0 = (within / gsize) * kTile;

    // ---- what this lane stages: instruction j of a wave fills rows (4 j + wave) * 16 .. + 16 of the stage (rows
    // 0..255: weights, 256..511: activations); lane -> (line, row slot, piece position); the piece it fetches follows
    // from the swizzle
    const int g_line = lane >> 4, g_slot = (lane >> 2) & 3;
    const int g_c = (lane & 3) ^ g_line;                              // (absolute line) & 3 == g_line for every j
    uint32_t w_off[4], x_off[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int r = (4 * j + wave) * 16 + 4 * g_line + g_slot;
        const int n = min(n0 + r, p.N - 1);
        const int64_t row = min(m0 + r, p.M - 1);
        w_off[j] = (uint32_t)((int64_t)n * p.K * 2 + g_c * 16);
        x_off[j] = (uint32_t)(row * p.x_stride * 2 + g_c * 16);
    }
    const char* f_w = p.w;
    const char* f_x = p.x;
    auto stage = [&](int ring) {
        const uint32_t mb = lds0 + (uint32_t)ring * kStageBytes + (uint32_t)wave * 1024;
#pragma unroll
        for (int j = 0; j < 4; ++j) bg_load_lds16(f_w, w_off[j], mb + (uint32_t)j * 4096);
#pragma unroll
        for (int j = 0; j < 4; ++j) bg_load_lds16(f_x, x_off[j], mb + (uint32_t)(4 + j) * 4096);
        f_w += kKS * 2;
        f_x += kKS * 2;
    };

    f32x16 acc[4][4];
#pragma unroll
    for (int cb = 0; cb < 4; ++cb)
#pragma unroll
        for (int tb = 0; tb < 4; ++tb)
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[cb][tb][i] = 0.f;

    // operand read offsets: row base + the swizzled piece of each 16-wide k step
    const int rl3 = (m >> 2) & 3;
    const uint32_t a_base = (uint32_t)(((wn * 128 + m) >> 2) * 256 + ((m & 3) << 6));
    const uint32_t b_base = (uint32_t)(((256 + wm * 128 + m) >> 2) * 256 + ((m & 3) << 6));
    uint32_t k_off[2];
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) k_off[ks] = (uint32_t)(((2 * ks + hf) ^ rl3) << 4);

    // operand fragments of one 16-wide k step: 4 weight blocks (32 rows = 8 lines = 2 KB apart), 4 activation blocks
    auto fetch = [&](u32x4* f, uint32_t buf, int ks) {
        const uint32_t aa = lds0 + buf + a_base + k_off[ks], bb = lds0 + buf + b_base + k_off[ks];
        f[0] = bg_lds_read16<0>(aa);
        f[1] = bg_lds_read16<2048>(aa);
        f[2] = bg_lds_read16<4096>(aa);
        f[3] = bg_lds_read16<6144>(aa);
        f[4] = bg_lds_read16<0>(bb);
        f[5] = bg_lds_read16<2048>(bb);
        f[6] = bg_lds_read16<4096>(bb);
        f[7] = bg_lds_read16<6144>(bb);
    };
    auto multiply = [&](const u32x4* f) {
#pragma unroll
        for (int cb = 0; cb < 4; ++cb)
#pragma unroll
            for (int tb = 0; tb < 4; ++tb) acc[cb][tb] = E::mfma32(f[cb], f[4 + tb], acc[cb][tb]);
    };

    // Iteration s multiplies stage s.  Its first k step was fetched from LDS in iteration s - 1; after the first half
    // of its matrix instructions are issued the wave waits for its own loads of stage s + 1 and meets the others at the
    // barrier: past it stage s + 1 is in LDS and nobody reads stage s - 1 any more, whose buffer takes stage s + 3.
    const int nstage = p.K / kKS;
    stage(0);
    if (nstage > 1) stage(1);
    if (nstage > 2) stage(2);
    if (nstage > 2) bg_wait_stage<16>();                   // a stage is 8 load instructions per wave
    else if (nstage > 1) bg_wait_stage<8>();
    else bg_wait_stage<0>();
    u32x4 f0[8], f1[8];
    fetch(f0, 0, 0);
    // the last two stages are peeled: the one before last waits for every load, the last one has nothing to wait for
    int s = 0;
    for (; s + 2 < nstage; ++s) {
        fetch(f1, (uint32_t)(s % kRing) * kStageBytes, 1);
        bg_wait_frags<8>(f0);
        multiply(f0);
        __builtin_amdgcn_sched_barrier(0);
        bg_wait_stage<8>();                                // outstanding: stage s + 2's loads
        if (s + 3 < nstage) stage((s + 3) % kRing);
        fetch(f0, (uint32_t)((s + 1) % kRing) * kStageBytes, 0);
        bg_wait_frags<8>(f1);
        multiply(f1);
        __builtin_amdgcn_sched_barrier(0);
    }
    if (s + 1 < nstage) {
        fetch(f1, (uint32_t)(s % kRing) * kStageBytes, 1);
        bg_wait_frags<8>(f0);
        multiply(f0);
        __builtin_amdgcn_sched_barrier(0);
        bg_wait_stage<0>();
        fetch(f0, (uint32_t)((s + 1) % kRing) * kStageBytes, 0);
        bg_wait_frags<8>(f1);
        multiply(f1);
        __builtin_amdgcn_sched_barrier(0);
        ++s;
    }
    fetch(f1, (uint32_t)(s % kRing) * kStageBytes, 1);
    bg_wait_frags<8>(f0);
    multiply(f0);
    bg_wait_frags<0>(f1);
    multiply(f1);

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
        for (int tb = 0; tb < 4; ++tb) {
            const int64_t row = m0 + wm * 128 + 32 * tb + m;
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

template <class E, int EPI>
int launch_epi(const GemmArgs& a, hipStream_t st) {
    static bool configured = false;                       // per instantiation; racing callers set the same value
    if (!configured) {
        hipError_t e = hipFuncSetAttribute((const void*)block_gemm_kernel<E, EPI>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                           kRing * kStageBytes);
        if (e != hipSuccess) {
            set_error("sfm_linear: hipFuncSetAttribute failed: %s", hipGetErrorString(e));
            return SFM_ERR_HIP;
        }
        configured = true;
    }
    const int ntiles = a.tm * a.tn;
    hipLaunchKernelGGL((block_gemm_kernel<E, EPI>), dim3((unsigned)((ntiles + 7) / 8 * 8)), dim3(256), kRing * kStageBytes, st, a);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        set_error("sfm_linear: launch failed: %s", hipGetErrorString(e));
        return SFM_ERR_HIP;
    }
    return SFM_OK;
}

template <class E>
int launch_dtype(const GemmArgs& a, int epilogue, hipStream_t st) {
    if (epilogue == SFM_EPI_GELU_TANH) return launch_epi<E, SFM_EPI_GELU_TANH>(a, st);
    if (epilogue == SFM_EPI_GATE_RESIDUAL) return launch_epi<E, SFM_EPI_GATE_RESIDUAL>(a, st);
    return launch_epi<E, SFM_EPI_NONE>(a, st);
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
    a.tm = (int)((d.M + kTile - 1) / kTile);
    a.tn = (d.N + kTile - 1) / kTile;
    return d.dtype == SFM_BF16 ? launch_dtype<BF16>(a, d.epilogue, stream) : launch_dtype<F16>(a, d.epilogue, stream);
}

}  // namespace sfm
