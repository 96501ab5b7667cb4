// Channels-last 3-D convolution as an implicit GEMM on gfx950 MFMA (bf16 / fp16), for the streaming VAE decoder
// (replaces the nn.Conv3d / nn.Conv2d calls of wan/modules/vae.py:17-36, :76-97, :186-220, :423-472).
//
//   y[t, h, w, co] = bias[co] + res[t, h, w, co] + sum_{dt, dh, dw, ci}  wt[dt, dh, dw, co, ci] * xp[t + dt, h' + dh, w' + dw, ci]
//
// xp is the input with its zero (or history) frames and its zero border already in place, so the kernel has no
// bounds tests; with `up2x` it is the half-resolution tensor and (h', w') = the row / column of xp that the
// nearest-neighbour x2 upsampling would have copied (vae.py:57-63, :77-79), i.e. the upsampled tensor is
// never materialised.
//
// GEMM view: M = output channels (A operand, rows of wt with ci contiguous), N = output voxels (B operand, rows of
// xp), K = taps x input channels, walked one tap and 32 channels at a time.  Each K step stages 64-byte rows
// (32 channels) of both operands straight into LDS (global_load_lds_dwordx4), four rows to a 256-byte line with
// the 16-byte chunks of a row rotated by the line index so that operand reads are conflict-free; two stage buffers, one
// barrier per stage.  A wave owns CB x 32 output channels by 64 voxels; accumulators leave through the same
// half-swap as the attention kernels (8 consecutive channels = 16 bytes per lane and voxel).

#include <hip/hip_runtime.h>

#include "sfm_attn.h"
#include "sfm_common.hpp"

namespace sfm {
namespace {

constexpr int kKC = 32;                      // input channels per stage
constexpr int kRowBytes = kKC * 2;           // one staged row

struct ConvArgs {
    const char* x;            // padded input, channels-last
    const char* wt;           // [taps][Cout_pad][Cin] (ci contiguous)
    const float* bias;        // [Cout] or null
    const char* res;          // residual input laid out like y, or null
    char* y;
    int T, H, W;              // output grid
    int Cin, Cout, Cout_pad;
    int kt, kh, kw;
    int up2x;
    int64_t xs_t, xs_h, xs_w; // input strides in elements (channel stride 1)
    int64_t ys_t, ys_h, ys_w; // output strides in elements
    int64_t voxels;           // T * H * W
};

// byte offset of chunk c (16 bytes) of row r in a tile of 64-byte rows: four rows to a 256-byte line, the chunks of a
// row stored at position c ^ (line & 3).  The 16 lanes that one cycle of a ds_read_b128 serves read the same chunk of 16
// consecutive rows, i.e. of four lines: the rotation puts them on 16 different 16-byte bank groups.
__device__ __forceinline__ uint32_t tile_off(int r, int c) {
    const int line = r >> 2;
    return (uint32_t)(line * 256 + ((r & 3) << 6) + ((c ^ (line & 3)) << 4));
}

__device__ __forceinline__ void cv_load_lds16(const char* base, uint32_t off, uint32_t lds_addr) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_addr), "v"(off), "s"(base) : "memory", "m0");
}
__device__ __forceinline__ void cv_wait_stage() { asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// Epilogue of one voxel (t, h, w) of a lane: residual and bias added in fp32, one rounding, CB blocks of 32 channels
// from channel cbase0 on.  Lane half hf of block cb holds channels 8 g + 4 hf + (e & 3) in acc[cb][vb][4 g + (e & 3)].
template <class E, int CB>
__device__ __forceinline__ void store_voxel(const ConvArgs& p, f32x16 (&acc)[CB][2], int vb, bool vok, int t, int h, int w,
                                            int cbase0, int hf) {
    const int64_t yoff = ((int64_t)t * p.ys_t + (int64_t)h * p.ys_h + (int64_t)w * p.ys_w) * 2;
    char* yrow = p.y + yoff;
#pragma unroll
    for (int cb = 0; cb < CB; ++cb) {
        const int cbase = cbase0 + 32 * cb;
        if (p.res != nullptr && vok) {
            // the block of the voxel that this lane completes: channels 8 g + 4 hf + 0..3
            const char* rrow = p.res + yoff;
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int co = cbase + 8 * g + 4 * hf;
                if (co + 4 <= p.Cout) {
                    const u32x2 rv = *(const u32x2*)(rrow + co * 2);
                    acc[cb][vb][4 * g + 0] += E::to_float((uint16_t)(rv.x & 0xffffu));
                    acc[cb][vb][4 * g + 1] += E::to_float((uint16_t)(rv.x >> 16));
                    acc[cb][vb][4 * g + 2] += E::to_float((uint16_t)(rv.y & 0xffffu));
                    acc[cb][vb][4 * g + 3] += E::to_float((uint16_t)(rv.y >> 16));
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        if (co + e < p.Cout) acc[cb][vb][4 * g + e] += E::to_float(*(const uint16_t*)(rrow + (co + e) * 2));
                }
            }
        }
        if (p.bias != nullptr) {
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const int co = cbase + 8 * (e >> 2) + 4 * hf + (e & 3);
                acc[cb][vb][e] += co < p.Cout ? p.bias[co] : 0.f;
            }
        }
        if (cbase + 32 <= p.Cout) {
#pragma unroll
            for (int gp = 0; gp < 2; ++gp) {
                const int g0 = 2 * gp, g1 = 2 * gp + 1;
                auto rx = __builtin_amdgcn_permlane32_swap(pack2<E>(acc[cb][vb][4 * g0 + 0], acc[cb][vb][4 * g0 + 1]),
                                                           pack2<E>(acc[cb][vb][4 * g1 + 0], acc[cb][vb][4 * g1 + 1]), false, false);
                auto ry = __builtin_amdgcn_permlane32_swap(pack2<E>(acc[cb][vb][4 * g0 + 2], acc[cb][vb][4 * g0 + 3]),
                                                           pack2<E>(acc[cb][vb][4 * g1 + 2], acc[cb][vb][4 * g1 + 3]), false, false);
                u32x4 o = {(uint32_t)rx[0], (uint32_t)ry[0], (uint32_t)rx[1], (uint32_t)ry[1]};
                if (vok) *(u32x4*)(yrow + (cbase + 16 * gp + 8 * hf) * 2) = o;
            }
        } else {
            // a partial last block (e.g. the 3 channels of the decoder's head): element stores
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const int co = cbase + 8 * (e >> 2) + 4 * hf + (e & 3);
                if (vok && co < p.Cout) *(uint16_t*)(yrow + co * 2) = E::from_float(acc[cb][vb][e]);
            }
        }
    }
}

// CB: 32-channel blocks per wave; WN: waves along the output channels (the other 4 / WN waves split the voxels);
// UP: the input is at half resolution (nearest x2 upsampling folded into the addresses).
template <class E, int CB, int WN, bool UP>
__global__ __launch_bounds__(256, 2) void conv3d_cl_kernel(ConvArgs p) {
    constexpr int WM = 4 / WN;
    constexpr int kVox = 64 * WM;                         // voxels per workgroup
    constexpr int kCo = 32 * CB * WN;                     // output channels per workgroup
    constexpr int kCoRows = (kCo + 63) / 64 * 64;         // weight rows staged (whole groups of 16 per wave)
    constexpr int kRows = kCoRows + kVox;
    constexpr int kStage = kRows * kRowBytes;
    constexpr int kWG = kCoRows / 64;                     // 16-row groups (one load instruction each) of weights per wave
    constexpr int kVG = kVox / 64;                        // ... of voxels per wave
    extern __shared__ __attribute__((aligned(256))) char lds[];
    const uint32_t lds0 = (uint32_t)(size_t)(__attribute__((address_space(3))) char*)lds;

    const int tid = threadIdx.x, lane = tid & 63, m = lane & 31, hf = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wn = wave % WN, wm = wave / WN;
    // consecutive workgroup ids go to the 8 XCDs in turn: give each XCD a contiguous range of voxel tiles, so that the
    // input rows that neighbouring tiles share (taps one row up and down) meet in one L2
    // and the channel blocks of one voxel tile follow each other within the XCD
    const int ny = (p.Cout_pad + kCo - 1) / kCo;
    const int per_xcd = (int)gridDim.x / 8;               // the grid is a multiple of 8 long
    const int seq = (int)(blockIdx.x >> 3);
    const int tile = (int)(blockIdx.x & 7) * (per_xcd / ny) + seq / ny;
    if ((int64_t)tile * kVox >= p.voxels) return;
    const int64_t v0 = (int64_t)tile * kVox;
    const int co0 = (seq % ny) * kCo;

    // ---- what this lane stages: for each of the wave's row groups one 16-byte chunk of one row
    // lane -> (line, quarter, chunk) of the group's 1 KB; the row sitting in that quarter is quarter ^ line
    // lane -> 16-byte slot of the group's 1 KB: line, row of the line, position; the chunk sitting there is position ^ line
    const int g_line = lane >> 4, g_row = lane >> 2, g_c = (lane & 3) ^ g_line;
    uint32_t w_off[kWG];                                  // byte offset of the weight row (without tap and channel step)
    uint32_t x_off[kVG];                                  // byte offset of the voxel's first tap (with UP: of its frame only)
    int vh[kVG], vw[kVG];
#pragma unroll
    for (int i = 0; i < kWG; ++i) {
        const int co = min(co0 + (i * 4 + wave) * 16 + g_row, p.Cout_pad - 1);
        w_off[i] = (uint32_t)(co * p.Cin * 2 + g_c * 16);
    }
#pragma unroll
    for (int i = 0; i < kVG; ++i) {
        const int64_t v = min(v0 + (i * 4 + wave) * 16 + g_row, p.voxels - 1);       // rows past the end repeat the last voxel
        const int w = (int)(v % p.W);
        const int64_t r = v / p.W;
        const int h = (int)(r % p.H), t = (int)(r / p.H);
        vh[i] = h;
        vw[i] = w;
        const int64_t e = UP ? t * p.xs_t : t * p.xs_t + h * p.xs_h + w * p.xs_w;
        x_off[i] = (uint32_t)(e * 2 + g_c * 16);
    }

    const int cin_steps = p.Cin / kKC;
    const int nstage = p.kt * p.kh * p.kw * cin_steps;
    const size_t w_tap = (size_t)p.Cout_pad * p.Cin * 2;  // bytes between taps of wt

    // position of the stage being fetched: channel step, tap column, tap row; the source pointers move by precomputed
    // deltas, so that issuing a stage costs a handful of scalar instructions
    int f_cs = 0, f_dw = 0, f_dh = 0;
    const char* f_w = p.wt;
    const char* f_x = p.x;
    const int64_t step_tap_w = (int64_t)w_tap - (int64_t)p.Cin * 2;                           // last channel step of a tap -> next tap's first
    const int64_t step_dw = (UP ? 0 : p.xs_w * 2) - (int64_t)p.Cin * 2;                       // next tap column
    const int64_t step_dh = UP ? 0 : (p.xs_h - (int64_t)p.kw * p.xs_w) * 2;                   // next tap row
    const int64_t step_dt = (UP ? p.xs_t : p.xs_t - (int64_t)p.kh * p.xs_h) * 2;              // next tap frame
    auto stage = [&](uint32_t buf) {
        const uint32_t mb = lds0 + buf + (uint32_t)wave * 1024;
#pragma unroll
        for (int i = 0; i < kWG; ++i) cv_load_lds16(f_w, w_off[i], mb + (uint32_t)i * 4096);
#pragma unroll
        for (int i = 0; i < kVG; ++i) {
            const uint32_t dst = mb + (uint32_t)(kCoRows / 16 + i * 4) * 1024;
            if (!UP) {
                cv_load_lds16(f_x, x_off[i], dst);
            } else {
                // tap d of output position o reads padded low-resolution index ((o + d - 1) >> 1) + 1
                const int hh = ((vh[i] + f_dh - 1) >> 1) + 1, ww = ((vw[i] + f_dw - 1) >> 1) + 1;
                cv_load_lds16(f_x, x_off[i] + (uint32_t)((hh * p.xs_h + ww * p.xs_w) * 2), dst);
            }
        }
        f_w += kKC * 2;
        f_x += kKC * 2;
        if (++f_cs == cin_steps) {
            f_cs = 0;
            f_w += step_tap_w;
            f_x += step_dw;
            if (++f_dw == p.kw) {
                f_dw = 0;
                f_x += step_dh;
                if (++f_dh == p.kh) {
                    f_dh = 0;
                    f_x += step_dt;
                }
            }
        }
    };

    f32x16 acc[CB][2];
#pragma unroll
    for (int cb = 0; cb < CB; ++cb)
#pragma unroll
        for (int vb = 0; vb < 2; ++vb)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[cb][vb][v] = 0.f;

    // operand read offsets within a stage: row r0 + m, chunk 2 ks + hf
    // blocks of 32 rows keep a row's line & 3, so one offset per k-step serves all blocks of an operand
    uint32_t a_off[2], b_off[2];
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
        a_off[ks] = tile_off(32 * CB * wn + m, 2 * ks + hf);
        b_off[ks] = tile_off(kCoRows + 64 * wm + m, 2 * ks + hf);
    }

    stage(0);
    for (int s = 0; s < nstage; ++s) {
        const uint32_t buf = (uint32_t)(s & 1) * kStage;
        cv_wait_stage();                                   // stage s is in LDS; the other buffer is free
        if (s + 1 < nstage) stage(buf ^ kStage);
#pragma unroll
        for (int ks = 0; ks < kKC / 16; ++ks) {
            u32x4 a[CB], b[2];
#pragma unroll
            for (int cb = 0; cb < CB; ++cb) a[cb] = *(const u32x4*)(lds + buf + a_off[ks] + cb * (32 * kRowBytes));
#pragma unroll
            for (int vb = 0; vb < 2; ++vb) b[vb] = *(const u32x4*)(lds + buf + b_off[ks] + vb * (32 * kRowBytes));
#pragma unroll
            for (int cb = 0; cb < CB; ++cb)
#pragma unroll
                for (int vb = 0; vb < 2; ++vb) acc[cb][vb] = E::mfma32(a[cb], b[vb], acc[cb][vb]);
        }
    }

    // ---- epilogue: lane (m, hf) of block (cb, vb) holds voxel 32 vb + m, channels 8 g + 4 hf + (v & 3)
#pragma unroll
    for (int vb = 0; vb < 2; ++vb) {
        const int64_t v = v0 + 64 * wm + 32 * vb + m;
        const bool vok = v < p.voxels;
        const int64_t vc = vok ? v : 0;
        const int w = (int)(vc % p.W);
        const int64_t r = vc / p.W;
        store_voxel<E, CB>(p, acc, vb, vok, (int)(r / p.H), (int)(r % p.H), w, co0 + 32 * CB * wn, hf);
    }
}

// The 3x3 spatial kernels on a contiguous padded input (x_stride = {(H + 2)(W + 2) Cin, (W + 2) Cin, Cin}): outputs are
// computed for every position u of the padded grid from its first to its last interior voxel (the two border columns
// between rows and the border rows between frames come out as garbage and are not stored: 0.7 % more work at 480 x
// 832), so that tap (dt, dh, dw) of position u is input row u + dt FS + (dh - 1) WP + (dw - 1) for all u alike.  A
// stage then holds one run of 258 consecutive input rows and the weights of the three taps of a kernel row: the
// three taps read the run at row offsets 0, 1, 2.  Per matrix instruction 3.9 staged rows instead of 7.3: the kernel
// above is bound by what the L2s deliver to the compute units.  One workgroup: 256 positions x CB x 32 channels.
template <class E, int CB>
__global__ __launch_bounds__(256, 2) void conv3d_row3_kernel(ConvArgs p) {
    constexpr int kVox = 256, kCo = 32 * CB;
    constexpr int kWRows = 3 * kCo;                       // weights of the three taps
    constexpr int kNWG = kWRows / 16, kNXG = 17;          // 16-row groups: weights, input run (258 rows -> 272)
    constexpr int kNG = kNWG + kNXG;
    constexpr int kPer = (kNG + 3) / 4;                   // groups a wave stages (the last one may repeat group kNG - 1)
    constexpr int kStage = kNG * 1024;
    extern __shared__ __attribute__((aligned(256))) char lds[];
    const uint32_t lds0 = (uint32_t)(size_t)(__attribute__((address_space(3))) char*)lds;

    const int tid = threadIdx.x, lane = tid & 63, m = lane & 31, hf = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int WP = p.W + 2;
    const int64_t FS = (int64_t)(p.H + 2) * WP;
    const int64_t u_first = WP + 1, u_last = (int64_t)(p.T - 1) * FS + (int64_t)p.H * WP + p.W;
    const int ny = p.Cout_pad / kCo;
    const int per_xcd = (int)gridDim.x / 8;               // as in conv3d_cl_kernel
    const int seq = (int)(blockIdx.x >> 3);
    const int64_t u0 = u_first + ((int64_t)(blockIdx.x & 7) * (per_xcd / ny) + seq / ny) * kVox;
    if (u0 > u_last) return;
    const int co0 = (seq % ny) * kCo;

    // lane -> 16-byte slot of the group's 1 KB: line, row of the line, position; the chunk sitting there is position ^ line
    const int g_line = lane >> 4, g_row = lane >> 2, g_c = (lane & 3) ^ g_line;
    uint32_t src[kPer];
#pragma unroll
    for (int i = 0; i < kPer; ++i) {
        const int g = min(wave + 4 * i, kNG - 1);
        const int j = g * 16 + g_row;
        if (g < kNWG) {
            const int dw = j / kCo, r = j - dw * kCo;
            src[i] = (uint32_t)(((int64_t)dw * p.Cout_pad + co0 + r) * p.Cin * 2 + g_c * 16);
        } else {
            // staged row s is the input row of tap (dt = 0, dh = 0, dw = 0) of position u0 + s; rows past the last
            // position's taps repeat the last one
            const int64_t u = min(u0 + (j - kWRows), u_last + 2) - WP - 1;
            src[i] = (uint32_t)(u * p.Cin * 2 + g_c * 16);
        }
    }

    const int cin_steps = p.Cin / kKC;
    const int nstage = p.kt * 3 * cin_steps;
    const char* f_w = p.wt;
    const char* f_x = p.x;
    const int64_t w_next_row = 3 * (int64_t)p.Cout_pad * p.Cin * 2 - (int64_t)p.Cin * 2;      // next kernel row: three taps on
    const int64_t x_next_row = ((int64_t)WP - 1) * p.Cin * 2;
    const int64_t x_next_frame = (FS - 3 * (int64_t)WP) * p.Cin * 2;
    int f_cs = 0, f_dh = 0;
    auto stage = [&](uint32_t buf) {
#pragma unroll
        for (int i = 0; i < kPer; ++i) {
            const int g = min(wave + 4 * i, kNG - 1);
            cv_load_lds16(g < kNWG ? f_w : f_x, src[i], lds0 + buf + (uint32_t)g * 1024);
        }
        f_w += kKC * 2;
        f_x += kKC * 2;
        if (++f_cs == cin_steps) {
            f_cs = 0;
            f_w += w_next_row;
            f_x += x_next_row;
            if (++f_dh == 3) {
                f_dh = 0;
                f_x += x_next_frame;
            }
        }
    };

    f32x16 acc[CB][2];
#pragma unroll
    for (int cb = 0; cb < CB; ++cb)
#pragma unroll
        for (int vb = 0; vb < 2; ++vb)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[cb][vb][v] = 0.f;

    // blocks of 32 rows (and the weights of the next tap, kCo rows on) keep a row's line & 3: one offset per k-step
    // for the weights, one per k-step and tap for the input rows
    uint32_t a_off[2], b_off[3][2];
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
        a_off[ks] = tile_off(m, 2 * ks + hf);
#pragma unroll
        for (int dw = 0; dw < 3; ++dw) b_off[dw][ks] = tile_off(kWRows + 64 * wave + m + dw, 2 * ks + hf);
    }

    stage(0);
    for (int s = 0; s < nstage; ++s) {
        const uint32_t buf = (uint32_t)(s & 1) * kStage;
        cv_wait_stage();
        if (s + 1 < nstage) stage(buf ^ kStage);
#pragma unroll
        for (int dw = 0; dw < 3; ++dw)
#pragma unroll
            for (int ks = 0; ks < kKC / 16; ++ks) {
                u32x4 a[CB], b[2];
#pragma unroll
                for (int cb = 0; cb < CB; ++cb) a[cb] = *(const u32x4*)(lds + buf + a_off[ks] + (dw * kCo + 32 * cb) * kRowBytes);
#pragma unroll
                for (int vb = 0; vb < 2; ++vb) b[vb] = *(const u32x4*)(lds + buf + b_off[dw][ks] + vb * (32 * kRowBytes));
#pragma unroll
                for (int cb = 0; cb < CB; ++cb)
#pragma unroll
                    for (int vb = 0; vb < 2; ++vb) acc[cb][vb] = E::mfma32(a[cb], b[vb], acc[cb][vb]);
            }
    }

#pragma unroll
    for (int vb = 0; vb < 2; ++vb) {
        const int64_t u = u0 + 64 * wave + 32 * vb + m;
        const int64_t uc = min(u, u_last);
        const int t = (int)(uc / FS);
        const int rem = (int)(uc - (int64_t)t * FS);
        const int hp = rem / WP, wp = rem - hp * WP;
        const bool vok = u <= u_last && hp >= 1 && hp <= p.H && wp >= 1 && wp <= p.W;
        store_voxel<E, CB>(p, acc, vb, vok, vok ? t : 0, vok ? hp - 1 : 0, vok ? wp - 1 : 0, co0, hf);
    }
}

template <class E, int CB>
int launch_row3(const ConvArgs& a, hipStream_t st) {
    constexpr int ldsb = 2 * (3 * 32 * CB / 16 + 17) * 1024;
    static bool configured = false;                       // per instantiation; racing callers set the same value
    if (!configured) {
        hipError_t e = hipFuncSetAttribute((const void*)conv3d_row3_kernel<E, CB>, hipFuncAttributeMaxDynamicSharedMemorySize, ldsb);
        if (e != hipSuccess) {
            set_error("sfm_conv3d_cl: hipFuncSetAttribute failed: %s", hipGetErrorString(e));
            return SFM_ERR_HIP;
        }
        configured = true;
    }
    const int64_t WP = a.W + 2, FS = (int64_t)(a.H + 2) * WP;
    const int64_t positions = (int64_t)(a.T - 1) * FS + (int64_t)(a.H - 1) * WP + a.W;     // first to last interior voxel
    const unsigned tiles = (unsigned)((positions + 255) / 256);
    hipLaunchKernelGGL((conv3d_row3_kernel<E, CB>), dim3((tiles + 7) / 8 * 8 * (unsigned)(a.Cout_pad / (32 * CB))), dim3(256), ldsb,
                       st, a);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        set_error("sfm_conv3d_cl: launch failed: %s", hipGetErrorString(e));
        return SFM_ERR_HIP;
    }
    return SFM_OK;
}

template <class E, int CB, int WN>
int launch_cfg(const ConvArgs& a, hipStream_t st) {
    constexpr int kVox = 64 * (4 / WN), kCo = 32 * CB * WN, kCoRows = (kCo + 63) / 64 * 64;
    constexpr int ldsb = 2 * (kCoRows + kVox) * kRowBytes;
    const unsigned tiles = (unsigned)((a.voxels + kVox - 1) / kVox);
    dim3 grid((tiles + 7) / 8 * 8 * (unsigned)((a.Cout_pad + kCo - 1) / kCo));
    if (a.up2x) hipLaunchKernelGGL((conv3d_cl_kernel<E, CB, WN, true>), grid, dim3(256), ldsb, st, a);
    else hipLaunchKernelGGL((conv3d_cl_kernel<E, CB, WN, false>), grid, dim3(256), ldsb, st, a);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        set_error("sfm_conv3d_cl: launch failed: %s", hipGetErrorString(e));
        return SFM_ERR_HIP;
    }
    return SFM_OK;
}

template <class E>
int launch_dtype(const ConvArgs& a, hipStream_t st) {
    const bool run = a.kh == 3 && !a.up2x && a.xs_w == a.Cin && a.xs_h == (int64_t)(a.W + 2) * a.Cin &&
                     a.xs_t == (int64_t)(a.H + 2) * (a.W + 2) * a.Cin && 3 * (int64_t)a.Cout_pad * a.Cin * 2 < ((int64_t)1 << 32);
    if (run && a.Cout_pad % 96 == 0) return launch_row3<E, 3>(a, st);
    if (run && a.Cout_pad == 32) return launch_row3<E, 1>(a, st);
    if (a.Cout_pad % 192 == 0) return launch_cfg<E, 3, 2>(a, st);
    if (a.Cout_pad % 96 == 0) return launch_cfg<E, 3, 1>(a, st);
    return launch_cfg<E, 1, 1>(a, st);                    // Cout_pad a multiple of 32
}


// ------------------------------------------------------------------------------------------------
// RMS norm over the channels, optional SiLU (vae.py:39-54 + nn.SiLU of :192-197, :418-420), channels-last, fp32
// inside, one rounding at the end.  GL lanes share a voxel (8 channels each, the first C / 8 of them active).
// ------------------------------------------------------------------------------------------------
struct NormArgs {
    const char* x;
    char* y;
    const uint16_t* gamma;
    int T, H, W, C, act;
    int64_t xs_t, xs_h, xs_w, ys_t, ys_h, ys_w;
    int64_t voxels;
};

template <class E, int GL>
__global__ __launch_bounds__(256) void vae_norm_act_kernel(NormArgs p) {
    const int tid = threadIdx.x;
    const int sub = tid % GL;
    const int64_t v = (int64_t)blockIdx.x * (256 / GL) + tid / GL;
    const bool active = v < p.voxels && sub < p.C / 8;
    const int64_t vc = v < p.voxels ? v : p.voxels - 1;
    const int w = (int)(vc % p.W);
    const int64_t r = vc / p.W;
    const int h = (int)(r % p.H), t = (int)(r / p.H);
    u32x4 raw = {0u, 0u, 0u, 0u};
    if (active) raw = *(const u32x4*)(p.x + (t * p.xs_t + h * p.xs_h + w * p.xs_w + sub * 8) * 2);
    float f[8];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        f[2 * i] = E::to_float((uint16_t)(raw[i] & 0xffffu));
        f[2 * i + 1] = E::to_float((uint16_t)(raw[i] >> 16));
    }
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) ss += f[i] * f[i];
#pragma unroll
    for (int o = GL / 2; o > 0; o >>= 1) ss += __shfl_xor(ss, o, GL);
    // x / max(|x|, 1e-12) * sqrt(C)  (F.normalize's clamp, vae.py:51-54)
    const float inv = sqrtf((float)p.C) / fmaxf(sqrtf(ss), 1e-12f);
    if (active) {
        const u32x4 g = *(const u32x4*)(p.gamma + sub * 8);
        u32x4 o;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            float a = f[2 * i] * inv * E::to_float((uint16_t)(g[i] & 0xffffu));
            float b = f[2 * i + 1] * inv * E::to_float((uint16_t)(g[i] >> 16));
            if (p.act) {
                a = a / (1.f + __expf(-a));
                b = b / (1.f + __expf(-b));
            }
            o[i] = pack2<E>(a, b);
        }
        *(u32x4*)(p.y + (t * p.ys_t + h * p.ys_h + w * p.ys_w + sub * 8) * 2) = o;
    }
}

// The decoder's channel counts are 96, 192, 384 = 24 x {4, 8, 16}: three 16-byte chunks per lane, GL lanes per voxel,
// every lane busy and three loads in flight per lane.
template <class E, int GL>
__global__ __launch_bounds__(256) void vae_norm_act3_kernel(NormArgs p) {
    const int tid = threadIdx.x;
    const int sub = tid % GL;
    const int64_t v = (int64_t)blockIdx.x * (256 / GL) + tid / GL;
    const bool active = v < p.voxels;
    const int64_t vc = active ? v : p.voxels - 1;
    const int w = (int)(vc % p.W);
    const int64_t r = vc / p.W;
    const int h = (int)(r % p.H), t = (int)(r / p.H);
    const char* src = p.x + (t * p.xs_t + h * p.xs_h + w * p.xs_w) * 2;
    u32x4 raw[3];
#pragma unroll
    for (int k = 0; k < 3; ++k) raw[k] = *(const u32x4*)(src + (sub + k * GL) * 16);
    float f[3][8];
    float ss = 0.f;
#pragma unroll
    for (int k = 0; k < 3; ++k)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            f[k][2 * i] = E::to_float((uint16_t)(raw[k][i] & 0xffffu));
            f[k][2 * i + 1] = E::to_float((uint16_t)(raw[k][i] >> 16));
            ss += f[k][2 * i] * f[k][2 * i] + f[k][2 * i + 1] * f[k][2 * i + 1];
        }
#pragma unroll
    for (int o = GL / 2; o > 0; o >>= 1) ss += __shfl_xor(ss, o, GL);
    const float inv = sqrtf((float)p.C) / fmaxf(sqrtf(ss), 1e-12f);
    if (active) {
        char* dst = p.y + (t * p.ys_t + h * p.ys_h + w * p.ys_w) * 2;
#pragma unroll
        for (int k = 0; k < 3; ++k) {
            const u32x4 g = *(const u32x4*)(p.gamma + (sub + k * GL) * 8);
            u32x4 o;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                float a = f[k][2 * i] * inv * E::to_float((uint16_t)(g[i] & 0xffffu));
                float b = f[k][2 * i + 1] * inv * E::to_float((uint16_t)(g[i] >> 16));
                if (p.act) {
                    a = a / (1.f + __expf(-a));
                    b = b / (1.f + __expf(-b));
                }
                o[i] = pack2<E>(a, b);
            }
            *(u32x4*)(dst + (sub + k * GL) * 16) = o;
        }
    }
}

template <class E>
int launch_norm(const NormArgs& a, hipStream_t st) {
    const int gl3 = a.C % 24 == 0 ? a.C / 24 : 0;
    if (gl3 == 4 || gl3 == 8 || gl3 == 16) {
        const unsigned blocks = (unsigned)((a.voxels + 256 / gl3 - 1) / (256 / gl3));
        if (gl3 == 4) hipLaunchKernelGGL((vae_norm_act3_kernel<E, 4>), dim3(blocks), dim3(256), 0, st, a);
        else if (gl3 == 8) hipLaunchKernelGGL((vae_norm_act3_kernel<E, 8>), dim3(blocks), dim3(256), 0, st, a);
        else hipLaunchKernelGGL((vae_norm_act3_kernel<E, 16>), dim3(blocks), dim3(256), 0, st, a);
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) {
            set_error("sfm_vae_norm_act: launch failed: %s", hipGetErrorString(e));
            return SFM_ERR_HIP;
        }
        return SFM_OK;
    }
    const int lanes = a.C / 8;
    const int gl = lanes <= 16 ? 16 : lanes <= 32 ? 32 : 64;
    const unsigned blocks = (unsigned)((a.voxels + 256 / gl - 1) / (256 / gl));
    if (gl == 16) hipLaunchKernelGGL((vae_norm_act_kernel<E, 16>), dim3(blocks), dim3(256), 0, st, a);
    else if (gl == 32) hipLaunchKernelGGL((vae_norm_act_kernel<E, 32>), dim3(blocks), dim3(256), 0, st, a);
    else hipLaunchKernelGGL((vae_norm_act_kernel<E, 64>), dim3(blocks), dim3(256), 0, st, a);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        set_error("sfm_vae_norm_act: launch failed: %s", hipGetErrorString(e));
        return SFM_ERR_HIP;
    }
    return SFM_OK;
}

}  // namespace
}  // namespace sfm

extern "C" int sfm_conv3d_cl(const sfm_conv_desc* d, const void* x, const void* wt, const float* bias, const void* res, void* y,
                             void* stream) {
    using namespace sfm;
    if (d == nullptr || x == nullptr || wt == nullptr || y == nullptr) {
        set_error("sfm_conv3d_cl: null argument");
        return SFM_ERR_NULL;
    }
    if (d->dtype != SFM_BF16 && d->dtype != SFM_F16) {
        set_error("sfm_conv3d_cl: dtype %d (need SFM_BF16 or SFM_F16)", d->dtype);
        return SFM_ERR_DTYPE;
    }
    if (d->T < 1 || d->H < 1 || d->W < 1 || d->Cin < 32 || d->Cin % 32 != 0 || d->Cout < 1 || d->Cout_pad < d->Cout ||
        d->Cout_pad % 32 != 0 || d->kt < 1 || d->kt > 3 || (d->kh != 1 && d->kh != 3) || d->kh != d->kw) {
        set_error("sfm_conv3d_cl: T,H,W >= 1, Cin a multiple of 32, Cout_pad >= Cout a multiple of 32, kt in 1..3, kh = kw in {1, 3}");
        return SFM_ERR_SHAPE;
    }
    if (d->up2x && (d->kh != 3 || d->H % 2 != 0 || d->W % 2 != 0)) {
        set_error("sfm_conv3d_cl: up2x needs a 3x3 spatial kernel and even H, W");
        return SFM_ERR_SHAPE;
    }
    for (int i = 0; i < 3; ++i) {
        // whole 32-channel blocks leave as 16-byte stores, a partial last block element by element
        if (d->x_stride[i] < d->Cin || d->x_stride[i] % 8 != 0 || d->y_stride[i] < d->Cout || (d->Cout >= 32 && d->y_stride[i] % 8 != 0)) {
            set_error("sfm_conv3d_cl: strides must be at least the channel count and (input always, output when Cout >= 32) multiples of 8 elements");
            return SFM_ERR_STRIDE;
        }
    }
    // extents of the padded input the kernel will touch, in elements, must fit the 32-bit lane offsets
    const int64_t hin = (d->up2x ? d->H / 2 : d->H) + (d->kh - 1), win = (d->up2x ? d->W / 2 : d->W) + (d->kw - 1);
    const int64_t span = ((int64_t)(d->T + d->kt - 2) * d->x_stride[0] + (hin - 1) * d->x_stride[1] + (win - 1) * d->x_stride[2] + d->Cin) * 2;
    if (span >= ((int64_t)1 << 32) || (int64_t)d->Cout_pad * d->Cin * 2 >= ((int64_t)1 << 32)) {
        set_error("sfm_conv3d_cl: the input of one call must stay below 4 GiB (%lld bytes)", (long long)span);
        return SFM_ERR_RANGE;
    }
    if ((((uintptr_t)x | (uintptr_t)wt) & 15) || (((uintptr_t)y | (uintptr_t)res) & (d->Cout >= 32 ? 15 : 1))) {
        set_error("sfm_conv3d_cl: x, wt, y must be 16-byte aligned");
        return SFM_ERR_ALIGN;
    }
    ConvArgs a;
    a.x = (const char*)x;
    a.wt = (const char*)wt;
    a.bias = bias;
    a.res = (const char*)res;
    a.y = (char*)y;
    a.T = d->T; a.H = d->H; a.W = d->W;
    a.Cin = d->Cin; a.Cout = d->Cout; a.Cout_pad = d->Cout_pad;
    a.kt = d->kt; a.kh = d->kh; a.kw = d->kw;
    a.up2x = d->up2x;
    a.xs_t = d->x_stride[0]; a.xs_h = d->x_stride[1]; a.xs_w = d->x_stride[2];
    a.ys_t = d->y_stride[0]; a.ys_h = d->y_stride[1]; a.ys_w = d->y_stride[2];
    a.voxels = (int64_t)d->T * d->H * d->W;
    hipStream_t st = (hipStream_t)stream;
    return d->dtype == SFM_BF16 ? launch_dtype<BF16>(a, st) : launch_dtype<F16>(a, st);
}

extern "C" int sfm_vae_norm_act(int32_t dtype, int32_t T, int32_t H, int32_t W, int32_t C, int32_t act, const void* x,
                                const int64_t x_stride[3], const void* gamma, void* y, const int64_t y_stride[3], void* stream) {
    using namespace sfm;
    if (x == nullptr || y == nullptr || gamma == nullptr || x_stride == nullptr || y_stride == nullptr) {
        set_error("sfm_vae_norm_act: null argument");
        return SFM_ERR_NULL;
    }
    if (dtype != SFM_BF16 && dtype != SFM_F16) {
        set_error("sfm_vae_norm_act: dtype %d (need SFM_BF16 or SFM_F16)", dtype);
        return SFM_ERR_DTYPE;
    }
    if (T < 1 || H < 1 || W < 1 || C < 8 || C > 512 || C % 8 != 0) {
        set_error("sfm_vae_norm_act: T,H,W >= 1 and C a multiple of 8 up to 512");
        return SFM_ERR_SHAPE;
    }
    for (int i = 0; i < 3; ++i) {
        if (x_stride[i] < C || x_stride[i] % 8 != 0 || y_stride[i] < C || y_stride[i] % 8 != 0) {
            set_error("sfm_vae_norm_act: strides must be multiples of 8 elements and at least C");
            return SFM_ERR_STRIDE;
        }
    }
    if (((uintptr_t)x | (uintptr_t)y | (uintptr_t)gamma) & 15) {
        set_error("sfm_vae_norm_act: x, y, gamma must be 16-byte aligned");
        return SFM_ERR_ALIGN;
    }
    NormArgs a;
    a.x = (const char*)x;
    a.y = (char*)y;
    a.gamma = (const uint16_t*)gamma;
    a.T = T; a.H = H; a.W = W; a.C = C; a.act = act;
    a.xs_t = x_stride[0]; a.xs_h = x_stride[1]; a.xs_w = x_stride[2];
    a.ys_t = y_stride[0]; a.ys_h = y_stride[1]; a.ys_w = y_stride[2];
    a.voxels = (int64_t)T * H * W;
    hipStream_t st = (hipStream_t)stream;
    return dtype == SFM_BF16 ? launch_norm<BF16>(a, st) : launch_norm<F16>(a, st);
}
