// Shared device/host helpers for the gfx950 attention kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "sfm_attn.h"

namespace sfm {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

// ---------------------------------------------------------------------------------------------
// 16-bit element traits.  Storage is uint16_t; eight elements travel as one u32x4 (16 bytes).
//
// MFMA 32x32x16 operand layout on gfx950 (wave64):
//   A (32 x 16): lane L supplies row  m = L % 32, k = 8*(L/32) + e, e = 0..7
//   B (16 x 32): lane L supplies col  n = L % 32, k = 8*(L/32) + e
//   D (32 x 32): lane L holds col n = L % 32; register v (0..15) holds row
//                m = 8*(v/4) + 4*(L/32) + v%4
// ---------------------------------------------------------------------------------------------
struct BF16 {
    static constexpr int kDtype = SFM_BF16;
    static __device__ __forceinline__ float to_float(uint16_t u) { return __uint_as_float(((uint32_t)u) << 16); }
    static __device__ __forceinline__ uint16_t from_float(float f) {
        __bf16 b = (__bf16)f;
        return __builtin_bit_cast(uint16_t, b);
    }
    // two floats -> one dword of two round-to-nearest-even elements (a single packed convert)
    static __device__ __forceinline__ uint32_t pack(float lo, float hi) {
        f32x2 v = {lo, hi};
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
    }
    static __device__ __forceinline__ f32x16 mfma32(u32x4 a, u32x4 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
    }
    // 16x16x32: A lane L supplies row L % 16, k = 8 (L / 16) + e; B column L % 16, same k; D column L % 16, rows 4 (L / 16) + v
    static __device__ __forceinline__ f32x4 mfma16(u32x4 a, u32x4 b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
    }
};

struct F16 {
    static constexpr int kDtype = SFM_F16;
    static __device__ __forceinline__ float to_float(uint16_t u) { return (float)__builtin_bit_cast(_Float16, u); }
    static __device__ __forceinline__ uint16_t from_float(float f) {
        _Float16 b = (_Float16)f;
        return __builtin_bit_cast(uint16_t, b);
    }
    static __device__ __forceinline__ uint32_t pack(float lo, float hi) {
        f32x2 v = {lo, hi};
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, f16x2_t));
    }
    static __device__ __forceinline__ f32x16 mfma32(u32x4 a, u32x4 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8_t, a), __builtin_bit_cast(f16x8_t, b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ f32x4 mfma16(u32x4 a, u32x4 b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8_t, a), __builtin_bit_cast(f16x8_t, b), c, 0, 0, 0);
    }
};

template <class E>
__device__ __forceinline__ uint32_t pack2(float lo, float hi) {
    return E::pack(lo, hi);
}

// v_exp_f32 without the denormal-range fix-up of exp2f(): arguments here are <= 0 and results that
// underflow may flush to zero.
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// Logit value given to masked positions: finite, so that 0 * mask stays 0 in entropy sums, and far
// enough below any real logit that exp2(mask - max) underflows to exactly 0.
constexpr float kMaskLogit = -1.0e30f;

__device__ __forceinline__ float xhalf_max(float x) { return fmaxf(x, __shfl_xor(x, 32)); }
__device__ __forceinline__ float xhalf_sum(float x) { return x + __shfl_xor(x, 32); }

// Workgroup barrier that orders LDS traffic only: waits for this wave's LDS operations, then s_barrier.
// Unlike __syncthreads() it does not drain outstanding global loads/stores, so register prefetches and
// streaming stores stay in flight across it.
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }
// Orders a wave's own LDS writes before its later LDS reads (wave-private staging buffers).
__device__ __forceinline__ void lds_wave_sync() { asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); }

// Row of the 16x16-dword-permuted contraction index used when a D tile (rows = contraction
// index) is fed back as a B operand: element e of lane-half hf in 16-wide step s.
__device__ __forceinline__ int perm_row(int s, int hf, int e) { return 16 * s + 4 * hf + (e < 4 ? e : e + 4); }

// ---------------------------------------------------------------------------------------------
// Token index of a Monarch block coordinate (block-frame bf, block row i, block col 0).
// natural = 0: rows are stored in block order ((bf*b1 + i)*b2 + j), the KV-cache layout.
// natural = 1: rows are stored in (frame,row,col) token order and
//     frame = A*f_tied + ft, row = c*hh + ii, col = e*ww + j  with  bf = (A*h_reduce + c)*w_reduce + e,
//     i = ft*hh + ii.
// Block columns j are always consecutive tokens.
// ---------------------------------------------------------------------------------------------
struct TokMap {
    int b1, b2, hh, ww, h, w, f_tied, h_reduce, w_reduce, natural;
    __host__ __device__ __forceinline__ int64_t row(int bf, int i) const {
        if (!natural) return ((int64_t)bf * b1 + i) * b2;
        int e = bf % w_reduce;
        int t = bf / w_reduce;
        int c = t % h_reduce;
        int A = t / h_reduce;
        int ft = i / hh;
        int ii = i - ft * hh;
        return ((int64_t)(A * f_tied + ft) * h + (c * hh + ii)) * w + e * ww;
    }
    // row(bf, i) - row(bf, 0): the same for every block-frame
    __host__ __device__ __forceinline__ int row_delta(int i) const {
        if (!natural) return i * b2;
        int ft = i / hh;
        return (ft * h + (i - ft * hh)) * w;
    }
};

// Workgroups of a launch go to the eight XCDs in turn (workgroup i to XCD i % 8) and every XCD has its own L2.  A 1-D
// grid of xcd_grid(total) workgroups that takes its work item from xcd_item(total) gives each XCD one contiguous range
// of items, so that items which read the same rows (the query blocks of one head, say) meet in one L2.  Items >= total
// have nothing to do.
__host__ __device__ __forceinline__ int xcd_grid(int total) { return (total + 7) / 8 * 8; }
#if defined(__HIPCC__)
__device__ __forceinline__ int xcd_item(int total) {
    const int per_xcd = (total + 7) / 8;
    return (int)(blockIdx.x % 8) * per_xcd + (int)(blockIdx.x / 8);
}
#endif

struct MonarchArgs {
    const void* q;
    const void* k;
    const void* v;
    void* out;
    void* kbar;      // [units_per_pass][na][b2][r_pad][D]   16-bit (MFMA path) or float (generic path)
    void* y;         // same shape
    float* cl;       // [units_per_pass][na][b2][r_pad]      sum_l R log2 R  (log2 units); MFMA kernels: see cl_unit below
    void* rep;       // iterated refinement only: query representatives, same shape and element type as kbar
    float* wgt;      // iterated refinement only: their weights, same shape as cl
    int iter_mode;   // MFMA step 1: 0 = queries from q; 1 = first refinement pass (q, logits / (1 + 1e-6));
                     // 2 = later pass (queries from rep, logits * min(1 / (wgt + 1e-6), 1e4))
    int B, H, D, na, nf, b1, b2;
    int r_pad;       // rows per (a, j) block of the workspace: round_up(nf*b1, 32)
    // scratch row index of (unit ul, a, j, r) = ul*ws_unit + (a*b2 + j)*ws_aj + r*ws_row
    uint32_t ws_unit, ws_aj, ws_row;
    uint32_t ws_f;   // MFMA step 1 only: rows between consecutive kv block-frames f of one (unit, a, j, k); 0 = b1 * ws_row
    // MFMA kernels only: cl of the scratch row above sits at ul*cl_unit + (a*b2 + j)*cl_aj + (r*ws_row)*cl_row.  The forward
    // keeps cl row-major (cl_aj = 1, cl_row = na*b2): the columns of one K/V tile are then one contiguous run, which step 1
    // writes as whole cache lines (one float per (a, j)-major row is a partial write of a 32-byte sector each, and 1.2 M of
    // those per call cost step 1 7 % of its time); step 2 gathers its column with that stride, out of the L2.
    uint32_t cl_unit, cl_aj, cl_row;
    void* rb;        // MFMA step 1 only, optional: the right factor R, 16 bit, 64 values per scratch row (same row index)
    float* stats;    // MFMA step 2 only, optional: log2-sum-exp of each query row's left-factor logits,
    uint32_t stats_ld;   // at ((b*H + h) * na*b2 + a*b2 + j) * stats_ld + i
    int unit0;       // first (b*H + h) unit of this pass
    int causal;      // block-causal size in block-frames, 0 = none
    float scale;
    TokMap qmap, kmap;
    int64_t qs[3], ks[3], vs[3], os[3];
    int a_chunk;     // query block-frames per step-1 workgroup
    int n_achunks;
    int s1_wgs;      // step-1 workgroups, 0 = one per CU (tuning override)
    int s1_groups;   // wave groups per step-1 workgroup
    int s1_total;    // step-1 work items: (unit, k, a-chunk, f) tiles
};

// Backward: the forward arguments (scratch matrices in float) plus the gradient tensors.
struct MonarchBwdArgs {
    MonarchArgs p;
    const void* dout;        // [B, Sq, H, D] tensor dtype, strides dos
    int64_t dos[3];
    float* dq;               // [B, Sq, H, D] float, strides dqs
    int64_t dqs[3];
    void* dk;                // tensor dtype, rows kmap.row(f, k) + l - dk_row0, strides dks
    void* dv;
    int64_t dks[3];
    int64_t dk_row0;
    float* dkbar;            // same layout as p.kbar
    float* dy;               // same layout as p.y
    float* dcl;              // same layout as p.cl: gradient of sum_l R ln R
    int kv_f0, kv_f1;        // kv block-frames whose dK / dV are wanted
    const void* fout;        // optional, with fstats: the forward's output (layout of dout) and its row statistics
    const float* fstats;     // (MonarchArgs::stats of that forward, row pitch round_up(b1, 32))
};

// Optional timing hooks: ev[0] is recorded before step 1, ev[1] between the steps, ev[2] after step 2.
struct StepEvents {
    hipEvent_t ev[3];
};

int launch_monarch_mfma(const MonarchArgs& a, int dtype, int nunits, hipStream_t stream, const StepEvents* ev);
int launch_monarch_generic(const MonarchArgs& a, int dtype, int nunits, hipStream_t stream, const StepEvents* ev);
bool monarch_mfma_supported(int dtype, int D, int b2);
// one-kernel forward (monarch_fused.hip): Kbar / Y stay in LDS; `ws` holds monarch_fused_bytes for a pass of nunits units
bool monarch_fused_supported(int dtype, int D, int b1, int b2, int causal);
size_t monarch_fused_bytes(int na, int nf, int b1, int b2, int nunits);
int launch_monarch_fused(const MonarchArgs& a, int dtype, int nunits, void* ws, size_t ws_bytes, hipStream_t stream, const StepEvents* ev);
int launch_monarch_iter(const MonarchArgs& a, int dtype, int nunits, int num_iters, hipStream_t stream);
// the refinement on the MFMA kernels (16-bit, head_dim 64 / 128, b1 <= 128, b2 <= 128): a.rep in the tensor dtype, a.stats
// [units][na * b2][a.stats_ld] scratch for the left factor's row statistics
bool monarch_iter_mfma_supported(int dtype, int D, int b1, int b2);
int launch_monarch_iter_mfma(const MonarchArgs& a, int dtype, int nunits, int num_iters, hipStream_t stream);
int launch_monarch_bwd(const MonarchBwdArgs& g, int dtype, int nunits, hipStream_t stream);
bool monarch_bwd_gemm_available();
// process-wide implementation switches (SFM_SW_* of the header), read from the environment once at load
unsigned switches();
bool rocblas_disabled();           // SFM_NO_ROCBLAS was set at load
int step1_wgs_override();          // SFM_S1_WGS at load, 0 = none
// every part of the chain runs as a fused kernel for this problem: no library GEMM is called
bool monarch_bwd_all_fused(const MonarchArgs& p, int dtype, const int64_t* dkv_stride);
size_t monarch_bwd_gemm_bytes(const MonarchArgs& p, int dtype, int nunits, const int64_t* dkv_stride);
int launch_monarch_bwd_gemm(const MonarchBwdArgs& g, int dtype, int nunits, void* workspace, hipStream_t stream);
// step 1 of the MFMA forward alone, with the scratch strides of `a` and, if a.rb is set, the right factor written out
int launch_monarch_step1(const MonarchArgs& a, int dtype, int nunits, hipStream_t stream);
// fused left-factor part of the backward (monarch_bwd_left.hip): q, dout (and out, with stats) are the callers' tensors,
// 16-byte aligned rows; everything else in the GEMM path's scratch layouts
bool monarch_bwd_left_supported(int dtype, int D, int b1);
int launch_monarch_bwd_left(int dtype, int D, int n, int b1, int b2, int AJ, int nf, int causal, float scale, const void* q,
                            const int64_t* qs, const void* dout, const void* out, const int64_t* os, const TokMap& qmap, int H,
                            int unit0, const void* kbar, const void* y, const float* c, int c_rows, void* dkbar, void* dy, float* dc,
                            void* ds2, int ds2_ld, const float* stats, int stats_ld, hipStream_t stream);
// dq rows (caller's layout) = s dS2 Kbar per (unit, a, j) + the right factor's dQk; same limits as the left kernel
int launch_monarch_bwd_dqa(int dtype, int D, int n, int b1, int b2, int AJ, int nf, float scale, const void* kbar, const void* ds2,
                           int ds2_ld, const float* dqk, float* dq, const int64_t* dqs, const TokMap& map, int H, int unit0,
                           hipStream_t stream);
// fused right-factor part of the backward (monarch_bwd_right.hip): per tile t = (unit, k, f) the dS1 block (scratch, for
// dQ = s dS1 K) and the finished dK / dV rows of kv block-frames [f0, f1) in the caller's tensors; q, k and v are the caller's tensors too
bool monarch_bwd_right_supported(int dtype, int D, int b2, int AJ);
int launch_monarch_bwd_right(int dtype, int D, int64_t ntiles, int b1, int b2, int AJ, int nf, float scale, const void* kk,
                             const int64_t* ks, const void* v, const int64_t* vs, const void* rb, const void* dkbar, const void* dy, const float* dc, const void* q,
                             const int64_t* qs, const TokMap& qmap, void* ds1, void* dk, void* dv, const int64_t* dks, int64_t row0,
                             const TokMap& kmap, int H, int unit0, int f0, int f1, hipStream_t stream);

// dQ of the right factor (monarch_bwd_right.hip): dqk[(u, k)][aj][:] = s sum_{f, l} dS1 K, float; k is the caller's tensor
bool monarch_bwd_dqk_supported(int dtype, int D, int b2, int AJ);
int launch_monarch_bwd_dqk(int dtype, int D, int64_t nuk, int b1, int b2, int AJ, int nf, float scale, const void* k, const int64_t* ks,
                           const TokMap& kmap, const void* ds1, float* dqk, int H, int unit0, hipStream_t stream);

// backward of the dense attention (dense_attn_bwd.hip); scratch is 2*B*H*q_tokens floats
bool dense_bwd_supported(int dtype, int D);
int launch_dense_bwd(const sfm_dense_desc& d, const int64_t* dq_stride, const int64_t* dkv_stride, int64_t kv0, int64_t kv1,
                     const void* q, const void* k, const void* v, const void* out, const float* lse, const void* dout, float* dq,
                     void* dk, void* dv, float* scratch, hipStream_t stream);

void set_error(const char* fmt, ...);
int cu_count();                                  // compute units of the current device (cached per thread)

}  // namespace sfm
