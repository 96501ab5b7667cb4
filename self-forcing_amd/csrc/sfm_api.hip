// extern "C" entry points: argument validation, workspace accounting, pass scheduling.
#include <pthread.h>
#include <atomic>
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "sfm_common.hpp"

namespace sfm {

static thread_local char g_err[512] = "";

namespace {
// The environment is read here, once, when the library is loaded; nothing reads it afterwards.
struct Switches {
    std::atomic<unsigned> mask{0};
    bool no_rocblas = false;
    int s1_wgs = 0;
    Switches() {
        static const struct { const char* name; unsigned bit; } names[] = {
            {"SFM_BWD_SIMT", SFM_SW_BWD_SIMT},           {"SFM_BWD_LEFT_GEMM", SFM_SW_BWD_LEFT_GEMM},
            {"SFM_BWD_FWD_GEMM", SFM_SW_BWD_FWD_GEMM},   {"SFM_BWD_DQA_GEMM", SFM_SW_BWD_DQA_GEMM},
            {"SFM_BWD_RIGHT_GEMM", SFM_SW_BWD_RIGHT_GEMM}, {"SFM_BWD_DQK_GEMM", SFM_SW_BWD_DQK_GEMM},
            {"SFM_ITER_SIMT", SFM_SW_ITER_SIMT}};
        unsigned m = 0;
        for (const auto& n : names) {
            const char* e = getenv(n.name);
            if (e && strcmp(e, "0") != 0) m |= n.bit;
        }
        mask.store(m);
        no_rocblas = getenv("SFM_NO_ROCBLAS") != nullptr;
        if (const char* e = getenv("SFM_S1_WGS")) {
            const int v = atoi(e);
            if (v >= 1 && v <= 65535) s1_wgs = v;
        }
    }
};
Switches g_sw;
}  // namespace

unsigned switches() { return g_sw.mask.load(std::memory_order_relaxed); }
bool rocblas_disabled() { return g_sw.no_rocblas; }
int step1_wgs_override() { return g_sw.s1_wgs; }

void set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

int launch_kv_cache_write(int esz, int B, int H, int D, const TokMap& map, int nbf, const void* nk, const void* nv,
                          const int64_t ns[3], void* kc, void* vc, const int64_t cs[3], int64_t start,
                          hipStream_t stream);
int launch_dense(const sfm_dense_desc& d, const void* q, const void* k, const void* v, void* out, float* lse,
                 hipStream_t stream);
int launch_prologue(const sfm_prologue_desc& d, const TokMap& map, const void* xq, const void* xk, const void* xv,
                    const void* wq, const void* wk, const double* rope, void* q_out, void* kc, void* vc,
                    hipStream_t stream);
int launch_linear(const sfm_linear_desc& d, const void* x, const void* w, const void* bias, const void* res, const void* gate,
                  void* out, hipStream_t stream);
bool monarch_generic_supported(const MonarchArgs& a);
bool monarch_iter_supported(const MonarchArgs& a);
int launch_ln_modulate(int dtype, int64_t rows, int C, float eps, const void* x, int64_t xs, void* y, int64_t ys,
                       const void* scale, const void* shift, int64_t ms, int rows_per_frame, const void* weight,
                       const void* bias, hipStream_t stream);
int launch_gate_residual_ln(int dtype, int64_t rows, int C, float eps, void* x, int64_t xs, const void* y, int64_t ys,
                            const void* gate, int64_t gms, int g_rows_per_frame, void* out, int64_t os, const void* scale,
                            const void* shift, int64_t ms, int rows_per_frame, const void* weight, const void* bias,
                            hipStream_t stream);
int launch_gate_residual(int dtype, int64_t rows, int C, void* x, int64_t xs, const void* y, int64_t ys,
                         const void* gate, int64_t ms, int rows_per_frame, hipStream_t stream);
int launch_rms_norm(int dtype, int64_t rows, int C, float eps, const void* x, int64_t xs, void* y, int64_t ys,
                    const void* weight, hipStream_t stream);

static int check_rows(int dtype, int64_t rows, int C, int64_t xs, int64_t ys) {
    if (dtype != SFM_BF16 && dtype != SFM_F16 && dtype != SFM_F32) {
        set_error("unsupported dtype %d", dtype);
        return SFM_ERR_DTYPE;
    }
    if (rows < 1 || rows > 0x7fffffff || C < 8 || C % 8 || C > 8192) {
        set_error("rows=%lld, C=%d: need rows >= 1 and C a multiple of 8 up to 8192", (long long)rows, C);
        return SFM_ERR_SHAPE;
    }
    const int esz = dtype == SFM_F32 ? 4 : 2;
    if (xs < C || ys < C || (xs * esz) % 16 || (ys * esz) % 16) {
        set_error("row strides must be >= C and multiples of 16 bytes");
        return SFM_ERR_STRIDE;
    }
    return SFM_OK;
}

static int elem_size(int dtype) { return dtype == SFM_F32 ? 4 : 2; }
static bool aligned16(const void* p) { return (((uintptr_t)p) & 15) == 0; }

static int check_tiling(const sfm_tiling& t) {
    if (t.f_tied < 1 || t.h_reduce < 1 || t.w_reduce < 1 || t.h < 1 || t.w < 1) {
        set_error("tiling: f_tied, h_reduce, w_reduce, h, w must be >= 1");
        return SFM_ERR_SHAPE;
    }
    if (t.h % t.h_reduce || t.w % t.w_reduce) {
        set_error("tiling: h_reduce (%d) must divide h (%d) and w_reduce (%d) must divide w (%d)", t.h_reduce, t.h,
                  t.w_reduce, t.w);
        return SFM_ERR_SHAPE;
    }
    return SFM_OK;
}

static TokMap make_map(const sfm_tiling& t, int natural) {
    TokMap m;
    m.hh = t.h / t.h_reduce;
    m.ww = t.w / t.w_reduce;
    m.b1 = t.f_tied * m.hh;
    m.b2 = m.ww;
    m.h = t.h;
    m.w = t.w;
    m.f_tied = t.f_tied;
    m.h_reduce = t.h_reduce;
    m.w_reduce = t.w_reduce;
    m.natural = natural;
    return m;
}

static int check_strides(const char* name, const int64_t s[3], int64_t tokens, int H, int D, int B, int esz) {
    if (s[2] < D || s[1] < 1 || s[0] < 0) {
        set_error("%s: strides (%lld, %lld, %lld) too small for H=%d, D=%d", name, (long long)s[0], (long long)s[1],
                  (long long)s[2], H, D);
        return SFM_ERR_STRIDE;
    }
    (void)B;
    // kernels address a (batch, head) slice with 32-bit element offsets
    if ((tokens + 1) * s[1] >= ((int64_t)1 << 31)) {
        set_error("%s: tokens * token-stride must stay below 2^31 elements", name);
        return SFM_ERR_STRIDE;
    }
    if ((s[0] * esz) % 16 || (s[1] * esz) % 16 || (s[2] * esz) % 16) {
        set_error("%s: strides must be multiples of 16 bytes", name);
        return SFM_ERR_STRIDE;
    }
    return SFM_OK;
}

struct MonarchPlan {
    int na, nf, b1, b2, r_pad, units;
    bool mfma, iter;
    bool iter_mfma;    // num_iters > 1 on the MFMA kernels (16-bit scratch + the left factor's row statistics)
    bool fused;        // the one-kernel forward (monarch_fused.hip) runs: its scratch is sized per pass, not per unit
    size_t per_unit;   // workspace bytes of a pass over one (batch x head) unit: the least a call needs
};

// Workspace of passes over up to n units.  The one-kernel forward's scratch is not monotonic in the units of a pass
// (fewer units mean shorter tile ranges per workgroup and more partial-result slots per unit), and the last pass of a
// call may be shorter than the others, so its size is the largest over every pass length up to n.
static size_t pass_bytes(const MonarchPlan& pl, int n) {
    if (!pl.fused) return pl.per_unit * (size_t)n;
    size_t mx = 0;
    for (int m = 1; m <= n; ++m) {
        const size_t b = monarch_fused_bytes(pl.na, pl.nf, pl.b1, pl.b2, m);
        if (b > mx) mx = b;
    }
    return mx;
}

static int plan_monarch(const sfm_monarch_desc* d, MonarchPlan* pl) {
    if (!d) {
        set_error("desc is NULL");
        return SFM_ERR_NULL;
    }
    if (d->dtype != SFM_BF16 && d->dtype != SFM_F16 && d->dtype != SFM_F32) {
        set_error("unsupported dtype %d", d->dtype);
        return SFM_ERR_DTYPE;
    }
    if (d->B < 1 || d->H < 1 || d->D < 8 || d->D % 8 || d->D > 256) {
        set_error("B=%d, H=%d, D=%d: need B,H >= 1 and D a multiple of 8 in [8,256]", d->B, d->H, d->D);
        return SFM_ERR_SHAPE;
    }
    int rc = check_tiling(d->tiling);
    if (rc) return rc;
    const sfm_tiling& t = d->tiling;
    const int64_t group = (int64_t)t.f_tied * t.h * t.w;
    if (d->q_tokens < 1 || d->kv_tokens < 1 || d->q_tokens % group || d->kv_tokens % group) {
        set_error("q_tokens=%d / kv_tokens=%d must be positive multiples of f_tied*h*w=%lld", d->q_tokens, d->kv_tokens,
                  (long long)group);
        return SFM_ERR_SHAPE;
    }
    const int per = t.h_reduce * t.w_reduce;
    pl->na = (int)(d->q_tokens / group) * per;
    pl->nf = (int)(d->kv_tokens / group) * per;
    pl->b1 = t.f_tied * (t.h / t.h_reduce);
    pl->b2 = t.w / t.w_reduce;
    if (d->causal_block_frames < 0) {
        set_error("causal_block_frames must be >= 0");
        return SFM_ERR_SHAPE;
    }
    if (d->causal_block_frames > 0) {
        if (d->q_tokens != d->kv_tokens) {
            set_error("block-causal Monarch needs kv_tokens == q_tokens");
            return SFM_ERR_SHAPE;
        }
        if (pl->na % d->causal_block_frames) {
            set_error("causal_block_frames=%d must divide the %d block-frames", d->causal_block_frames, pl->na);
            return SFM_ERR_SHAPE;
        }
    }
    if (!(d->sm_scale > 0.f) || d->sm_scale != d->sm_scale) {
        set_error("sm_scale must be a positive number");
        return SFM_ERR_SHAPE;
    }
    const int esz = elem_size(d->dtype);
    if ((rc = check_strides("q", d->q_stride, d->q_tokens, d->H, d->D, d->B, esz))) return rc;
    if ((rc = check_strides("k", d->k_stride, d->kv_tokens, d->H, d->D, d->B, esz))) return rc;
    if ((rc = check_strides("v", d->v_stride, d->kv_tokens, d->H, d->D, d->B, esz))) return rc;
    if ((rc = check_strides("out", d->o_stride, d->q_tokens, d->H, d->D, d->B, esz))) return rc;
    if (memcmp(d->k_stride, d->v_stride, sizeof(d->k_stride)) != 0) {
        set_error("k and v must share strides");
        return SFM_ERR_STRIDE;
    }
    pl->r_pad = (pl->nf * pl->b1 + 31) / 32 * 32;   // whole 32-row chunks per (a, j) block
    pl->units = d->B * d->H;
    if (d->num_iters < 1) {
        set_error("num_iters must be >= 1");
        return SFM_ERR_SHAPE;
    }
    if (d->num_iters > 1 && d->causal_block_frames) {
        set_error("block-causal masking is defined for num_iters == 1 only");
        return SFM_ERR_UNSUPPORTED;
    }
    pl->iter = d->num_iters > 1;
    pl->mfma = !pl->iter && monarch_mfma_supported(d->dtype, d->D, pl->b2);
    pl->iter_mfma = pl->iter && monarch_iter_mfma_supported(d->dtype, d->D, pl->b1, pl->b2) && !(switches() & SFM_SW_ITER_SIMT);
    const size_t rows = (size_t)pl->na * pl->b2 * pl->r_pad;
    pl->per_unit = rows * d->D * (pl->mfma || pl->iter_mfma ? 2 : 4) * (pl->iter ? 3 : 2) + rows * sizeof(float) * (pl->iter ? 2 : 1) +
                   (pl->iter_mfma ? (size_t)pl->na * pl->b2 * ((pl->b1 + 31) / 32 * 32) * sizeof(float) : 0);
    pl->per_unit = (pl->per_unit + 255) / 256 * 256;
    // the fp32 kernels' own limits, checked here so that no entry point has written anything (the KV-cache entry points
    // write the cache before the forward is launched) when they are exceeded
    if (!pl->mfma && !pl->iter_mfma) {
        MonarchArgs lim;
        memset(&lim, 0, sizeof(lim));
        lim.D = d->D; lim.na = pl->na; lim.nf = pl->nf; lim.b1 = pl->b1; lim.b2 = pl->b2;
        if (pl->iter ? !monarch_iter_supported(lim) : !monarch_generic_supported(lim)) {
            set_error("block shape b1=%d, b2=%d, %d rows per column, head_dim %d exceeds the LDS budget of the fp32 kernels that "
                      "this dtype / shape / num_iters runs on", pl->b1, pl->b2, pl->nf * pl->b1, d->D);
            return SFM_ERR_UNSUPPORTED;
        }
    }
    if (d->flags & ~SFM_MONARCH_ONE_KERNEL) {
        set_error("unknown bits in flags (0x%x)", (unsigned)d->flags);
        return SFM_ERR_SHAPE;
    }
    pl->fused = pl->mfma && (d->flags & SFM_MONARCH_ONE_KERNEL) && monarch_fused_supported(d->dtype, d->D, pl->b1, pl->b2, d->causal_block_frames);
    if (pl->fused) pl->per_unit = monarch_fused_bytes(pl->na, pl->nf, pl->b1, pl->b2, 1);
    return SFM_OK;
}

// Default number of units per pass: all of them while the scratch stays under 4 GiB (one launch pair
// fills the chip best; smaller passes only pay when the scratch would not fit).
static int default_units_per_pass(const MonarchPlan& pl) {
    if (pl.fused) return pl.units;                // a few MB per unit
    const size_t budget = (size_t)3 << 30;        // keeps 32-bit element offsets into each scratch matrix
    size_t n = budget / pl.per_unit;
    if (n < 1) n = 1;
    if (n > (size_t)pl.units) n = pl.units;
    return (int)n;
}

}  // namespace sfm

using namespace sfm;

extern "C" {

int sfm_version(void) { return 9; }

unsigned sfm_set_switches(unsigned mask) {
    if (mask & ~SFM_SW_ALL) {
        set_error("unknown switch bits 0x%x", mask & ~SFM_SW_ALL);
        return (unsigned)-1;
    }
    return g_sw.mask.exchange(mask);
}

unsigned sfm_get_switches(void) { return switches(); }

const char* sfm_last_error(void) { return g_err; }

int sfm_monarch_workspace_bytes(const sfm_monarch_desc* desc, int32_t heads_per_pass, size_t* bytes) {
    if (!bytes) {
        set_error("bytes is NULL");
        return SFM_ERR_NULL;
    }
    MonarchPlan pl;
    int rc = plan_monarch(desc, &pl);
    if (rc) return rc;
    if (heads_per_pass < 0) {
        set_error("heads_per_pass must be >= 0");
        return SFM_ERR_SHAPE;
    }
    int upp = heads_per_pass == 0 ? default_units_per_pass(pl) : (heads_per_pass > pl.units ? pl.units : heads_per_pass);
    *bytes = pass_bytes(pl, upp);
    return SFM_OK;
}

// Everything of the kernel arguments that does not depend on the pass: shapes, index maps, strides, scratch
// geometry.
static void init_args(const sfm_monarch_desc* desc, const MonarchPlan& pl, MonarchArgs* pa) {
    MonarchArgs& a = *pa;
    memset(&a, 0, sizeof(a));
    a.B = desc->B; a.H = desc->H; a.D = desc->D;
    a.na = pl.na; a.nf = pl.nf; a.b1 = pl.b1; a.b2 = pl.b2; a.r_pad = pl.r_pad;
    a.causal = desc->causal_block_frames;
    a.scale = desc->sm_scale;
    a.qmap = make_map(desc->tiling, 1);
    a.kmap = make_map(desc->tiling, desc->kv_block_order ? 0 : 1);
    for (int i = 0; i < 3; ++i) {
        a.qs[i] = desc->q_stride[i]; a.ks[i] = desc->k_stride[i];
        a.vs[i] = desc->v_stride[i]; a.os[i] = desc->o_stride[i];
    }
    const size_t rows = (size_t)pl.na * pl.b2 * pl.r_pad;
    a.ws_unit = (uint32_t)rows;
    // (a, j)-major scratch: the rows one step-2 wave streams are consecutive.  (An r-major layout, in
    // which the rows a step-1 workgroup writes are consecutive instead, measured the same for step 1.)
    a.ws_aj = (uint32_t)pl.r_pad;
    a.ws_row = 1;
    a.cl_unit = a.ws_unit;
    a.cl_aj = a.ws_aj;
    a.cl_row = 1;
    if (pl.mfma || pl.iter_mfma) {       // row-major cl: a tile's columns are contiguous (see MonarchArgs)
        a.cl_aj = 1;
        a.cl_row = (uint32_t)(pl.na * pl.b2);
    }
    // step 1 takes as many query block-frames per workgroup as fit 256 (a, j) columns
    int a_max = 256 / pl.b2;
    if (a_max < 1) a_max = 1;
    a.n_achunks = (pl.na + a_max - 1) / a_max;
    a.a_chunk = (pl.na + a.n_achunks - 1) / a.n_achunks;
    a.n_achunks = (pl.na + a.a_chunk - 1) / a.a_chunk;
    a.s1_wgs = step1_wgs_override();            // tuning override: step-1 workgroups (default 0: one per CU)
}

static int monarch_fwd_impl(const sfm_monarch_desc* desc, const void* q, const void* k, const void* v, void* out,
                            void* workspace, size_t workspace_bytes, void* stream, float* step_ms, float* stats = nullptr) {
    MonarchPlan pl;
    int rc = plan_monarch(desc, &pl);
    if (rc) return rc;
    if (stats && (!pl.mfma || pl.iter)) {
        set_error("row statistics come from the MFMA forward only (16-bit tensors, head_dim 64 or 128, b2 <= 128, num_iters 1)");
        return SFM_ERR_UNSUPPORTED;
    }
    if (!q || !k || !v || !out) {
        set_error("q, k, v and out must be non-NULL");
        return SFM_ERR_NULL;
    }
    if (!aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(out)) {
        set_error("q, k, v and out must be 16-byte aligned");
        return SFM_ERR_ALIGN;
    }
    if (!workspace || (((uintptr_t)workspace) & 255) || workspace_bytes < pl.per_unit) {
        set_error("workspace must be non-NULL, 256-byte aligned and hold at least %zu bytes (one unit)", pl.per_unit);
        return SFM_ERR_WORKSPACE;
    }
    MonarchArgs a;
    init_args(desc, pl, &a);
    a.q = q; a.k = k; a.v = v; a.out = out;
    a.stats = stats;
    a.stats_ld = (uint32_t)((pl.b1 + 31) / 32 * 32);
    if (pl.fused) {
        // as many units per pass as the workspace holds (the scratch of a pass is not linear in its units)
        int upp = pl.units;
        while (upp > 1 && pass_bytes(pl, upp) > workspace_bytes) --upp;
        for (int u0 = 0; u0 < pl.units; u0 += upp) {
            const int n = pl.units - u0 < upp ? pl.units - u0 : upp;
            a.unit0 = u0;
            StepEvents se;
            if (step_ms)
                for (int i = 0; i < 3; ++i)
                    if (hipEventCreate(&se.ev[i]) != hipSuccess) {
                        set_error("hipEventCreate failed");
                        return SFM_ERR_HIP;
                    }
            rc = launch_monarch_fused(a, desc->dtype, n, workspace, workspace_bytes, (hipStream_t)stream, step_ms ? &se : nullptr);
            if (step_ms) {
                float t1 = 0.f, t2 = 0.f;
                hipError_t e = rc ? hipSuccess : hipEventSynchronize(se.ev[2]);
                if (!rc && e == hipSuccess) e = hipEventElapsedTime(&t1, se.ev[0], se.ev[1]);
                if (!rc && e == hipSuccess) e = hipEventElapsedTime(&t2, se.ev[1], se.ev[2]);
                for (int i = 0; i < 3; ++i) (void)hipEventDestroy(se.ev[i]);
                if (!rc && e != hipSuccess) {
                    set_error("event timing failed: %s", hipGetErrorString(e));
                    return SFM_ERR_HIP;
                }
                step_ms[0] += t1;
                step_ms[1] += t2;
            }
            if (rc) return rc;
        }
        return SFM_OK;
    }
    size_t upp_sz = workspace_bytes / pl.per_unit;
    if (upp_sz * pl.per_unit > ((size_t)3 << 30)) upp_sz = ((size_t)3 << 30) / pl.per_unit;   // 32-bit offsets
    if (upp_sz < 1) {
        set_error("one (batch, head) unit needs %zu bytes of scratch, more than the 3 GiB a pass may use", pl.per_unit);
        return SFM_ERR_UNSUPPORTED;
    }
    const int upp = upp_sz > (size_t)pl.units ? pl.units : (int)upp_sz;
    const size_t rows = (size_t)pl.na * pl.b2 * pl.r_pad;
    const size_t mat_bytes = rows * desc->D * (pl.mfma || pl.iter_mfma ? 2 : 4);
    for (int u0 = 0; u0 < pl.units; u0 += upp) {
        const int n = pl.units - u0 < upp ? pl.units - u0 : upp;
        a.unit0 = u0;
        // [kbar | y | cl] blocks, each sized for `upp` units
        a.kbar = workspace;
        a.y = (char*)workspace + mat_bytes * upp;
        a.cl = (float*)((char*)workspace + 2 * mat_bytes * upp);
        if (pl.iter) {
            a.rep = (char*)a.cl + rows * sizeof(float) * upp;
            a.wgt = (float*)((char*)a.rep + mat_bytes * upp);
            if (step_ms) {
                set_error("the timed variant covers num_iters == 1 only");
                return SFM_ERR_UNSUPPORTED;
            }
            if (pl.iter_mfma) {
                // the kernels index the row statistics with the global unit (as the caller's buffer of
                // sfm_monarch_fwd_stats needs); the scratch holds one pass, so its base is moved back by the
                // pass's first unit
                a.stats_ld = (uint32_t)((pl.b1 + 31) / 32 * 32);
                const uintptr_t stats0 = (uintptr_t)a.wgt + rows * sizeof(float) * upp;
                a.stats = (float*)(stats0 - (size_t)u0 * pl.na * pl.b2 * a.stats_ld * sizeof(float));
                rc = launch_monarch_iter_mfma(a, desc->dtype, n, desc->num_iters, (hipStream_t)stream);
            } else {
                rc = launch_monarch_iter(a, desc->dtype, n, desc->num_iters, (hipStream_t)stream);
            }
            if (rc) return rc;
            continue;
        }
        StepEvents se;
        if (step_ms) {
            for (int i = 0; i < 3; ++i)
                if (hipEventCreate(&se.ev[i]) != hipSuccess) {
                    set_error("hipEventCreate failed");
                    return SFM_ERR_HIP;
                }
        }
        rc = pl.mfma ? launch_monarch_mfma(a, desc->dtype, n, (hipStream_t)stream, step_ms ? &se : nullptr)
                     : launch_monarch_generic(a, desc->dtype, n, (hipStream_t)stream, step_ms ? &se : nullptr);
        if (step_ms) {
            float t1 = 0.f, t2 = 0.f;
            hipError_t e = rc ? hipSuccess : hipEventSynchronize(se.ev[2]);
            if (!rc && e == hipSuccess) e = hipEventElapsedTime(&t1, se.ev[0], se.ev[1]);
            if (!rc && e == hipSuccess) e = hipEventElapsedTime(&t2, se.ev[1], se.ev[2]);
            for (int i = 0; i < 3; ++i) (void)hipEventDestroy(se.ev[i]);
            if (!rc && e != hipSuccess) {
                set_error("event timing failed: %s", hipGetErrorString(e));
                return SFM_ERR_HIP;
            }
            step_ms[0] += t1;
            step_ms[1] += t2;
        }
        if (rc) return rc;
    }
    return SFM_OK;
}

int sfm_monarch_fwd(const sfm_monarch_desc* desc, const void* q, const void* k, const void* v, void* out,
                    void* workspace, size_t workspace_bytes, void* stream) {
    return monarch_fwd_impl(desc, q, k, v, out, workspace, workspace_bytes, stream, nullptr);
}

int sfm_monarch_stats_bytes(const sfm_monarch_desc* desc, size_t* bytes) {
    if (!bytes) {
        set_error("bytes is NULL");
        return SFM_ERR_NULL;
    }
    MonarchPlan pl;
    int rc = plan_monarch(desc, &pl);
    if (rc) return rc;
    *bytes = pl.mfma && !pl.iter ? (size_t)pl.units * pl.na * pl.b2 * ((pl.b1 + 31) / 32 * 32) * sizeof(float) : 0;
    return SFM_OK;
}

int sfm_monarch_fwd_stats(const sfm_monarch_desc* desc, const void* q, const void* k, const void* v, void* out, float* stats,
                          void* workspace, size_t workspace_bytes, void* stream) {
    if (!stats) {
        set_error("stats is NULL");
        return SFM_ERR_NULL;
    }
    return monarch_fwd_impl(desc, q, k, v, out, workspace, workspace_bytes, stream, nullptr, stats);
}

int sfm_monarch_fwd_timed(const sfm_monarch_desc* desc, const void* q, const void* k, const void* v, void* out,
                          void* workspace, size_t workspace_bytes, void* stream, float* step1_ms, float* step2_ms) {
    if (!step1_ms || !step2_ms) {
        set_error("step1_ms / step2_ms are NULL");
        return SFM_ERR_NULL;
    }
    float ms[2] = {0.f, 0.f};
    int rc = monarch_fwd_impl(desc, q, k, v, out, workspace, workspace_bytes, stream, ms);
    *step1_ms = ms[0];
    *step2_ms = ms[1];
    return rc;
}

static int plan_bwd(const sfm_monarch_bwd_desc* bd, MonarchPlan* pl, size_t* per_unit) {
    if (!bd) {
        set_error("desc is NULL");
        return SFM_ERR_NULL;
    }
    int rc = plan_monarch(&bd->fwd, pl);
    if (rc) return rc;
    if (bd->fwd.num_iters != 1) {
        set_error("the backward covers num_iters == 1 (the reference's refinement path has no custom backward either)");
        return SFM_ERR_UNSUPPORTED;
    }
    if (bd->kv_grad_frame_start < 0 || bd->kv_grad_frame_end > pl->nf || bd->kv_grad_frame_start >= bd->kv_grad_frame_end) {
        set_error("kv gradient block-frames [%d, %d) outside [0, %d)", bd->kv_grad_frame_start, bd->kv_grad_frame_end, pl->nf);
        return SFM_ERR_RANGE;
    }
    if (!bd->fwd.kv_block_order && (bd->kv_grad_frame_start != 0 || bd->kv_grad_frame_end != pl->nf)) {
        set_error("a partial kv gradient needs k, v in block order (the KV-cache entry point)");
        return SFM_ERR_UNSUPPORTED;
    }
    const int esz = bd->fwd.dtype == SFM_F32 ? 4 : 2;
    const int64_t dkv_tokens = (int64_t)(bd->kv_grad_frame_end - bd->kv_grad_frame_start) * pl->b1 * pl->b2;
    if ((rc = check_strides("dq", bd->dq_stride, bd->fwd.q_tokens, bd->fwd.H, bd->fwd.D, bd->fwd.B, 4))) return rc;
    if ((rc = check_strides("dk/dv", bd->dkv_stride, dkv_tokens, bd->fwd.H, bd->fwd.D, bd->fwd.B, esz))) return rc;
    const size_t rows = (size_t)pl->na * pl->b2 * pl->r_pad;
    *per_unit = rows * bd->fwd.D * sizeof(float) * 4 + rows * sizeof(float) * 2;    // Kbar, Y, dKbar, dY; c, dc
    return SFM_OK;
}

// The batched-GEMM backward is used whenever rocBLAS can be loaded; the SFM_SW_BWD_SIMT switch selects the fp32 SIMT kernels.
static bool bwd_uses_gemm() {
    if (switches() & SFM_SW_BWD_SIMT) return false;
    return monarch_bwd_gemm_available();
}

int sfm_monarch_bwd_uses_gemm(void) { return bwd_uses_gemm() ? 1 : 0; }

// The chain of fused kernels and library products runs when rocBLAS is there, and also without it when every part of
// the chain has a fused kernel for this problem.
static bool bwd_uses_chain(const sfm_monarch_bwd_desc* desc, const MonarchPlan& pl) {
    if (switches() & SFM_SW_BWD_SIMT) return false;
    if (monarch_bwd_gemm_available()) return true;
    MonarchArgs a;
    init_args(&desc->fwd, pl, &a);
    return monarch_bwd_all_fused(a, desc->fwd.dtype, desc->dkv_stride);
}

int sfm_monarch_bwd_workspace_bytes(const sfm_monarch_bwd_desc* desc, int32_t heads_per_pass, size_t* bytes) {
    if (!bytes) {
        set_error("bytes is NULL");
        return SFM_ERR_NULL;
    }
    MonarchPlan pl;
    size_t per_unit = 0;
    int rc = plan_bwd(desc, &pl, &per_unit);
    if (rc) return rc;
    if (heads_per_pass < 0) {
        set_error("heads_per_pass must be >= 0");
        return SFM_ERR_SHAPE;
    }
    if (bwd_uses_chain(desc, pl)) {
        MonarchArgs a;
        init_args(&desc->fwd, pl, &a);
        int n = heads_per_pass > 0 ? (heads_per_pass > pl.units ? pl.units : heads_per_pass) : pl.units;
        if (heads_per_pass == 0)
            while (n > 1 && monarch_bwd_gemm_bytes(a, desc->fwd.dtype, n, desc->dkv_stride) > ((size_t)7 << 29)) --n;     // 3.5 GiB
        *bytes = monarch_bwd_gemm_bytes(a, desc->fwd.dtype, n, desc->dkv_stride);
        return SFM_OK;
    }
    size_t n = heads_per_pass > 0 ? (size_t)heads_per_pass : ((size_t)3 << 30) / per_unit;
    if (n < 1) n = 1;
    if (n > (size_t)pl.units) n = pl.units;
    *bytes = per_unit * n;
    return SFM_OK;
}

static int monarch_bwd_impl(const sfm_monarch_bwd_desc* desc, const void* q, const void* k, const void* v, const void* out,
                            const float* stats, const void* dout, float* dq, void* dk, void* dv, void* workspace,
                            size_t workspace_bytes, void* stream);

int sfm_monarch_bwd(const sfm_monarch_bwd_desc* desc, const void* q, const void* k, const void* v, const void* dout,
                    float* dq, void* dk, void* dv, void* workspace, size_t workspace_bytes, void* stream) {
    return monarch_bwd_impl(desc, q, k, v, nullptr, nullptr, dout, dq, dk, dv, workspace, workspace_bytes, stream);
}

int sfm_monarch_bwd_saved(const sfm_monarch_bwd_desc* desc, const void* q, const void* k, const void* v, const void* out,
                          const float* stats, const void* dout, float* dq, void* dk, void* dv, void* workspace,
                          size_t workspace_bytes, void* stream) {
    if (!out || !stats) {
        set_error("out and stats must be non-NULL (sfm_monarch_bwd recomputes them)");
        return SFM_ERR_NULL;
    }
    if (!aligned16(out) || (((uintptr_t)stats) & 3)) {
        set_error("out must be 16-byte aligned, stats 4-byte aligned");
        return SFM_ERR_ALIGN;
    }
    return monarch_bwd_impl(desc, q, k, v, out, stats, dout, dq, dk, dv, workspace, workspace_bytes, stream);
}

static int monarch_bwd_impl(const sfm_monarch_bwd_desc* desc, const void* q, const void* k, const void* v, const void* out,
                            const float* stats, const void* dout, float* dq, void* dk, void* dv, void* workspace,
                            size_t workspace_bytes, void* stream) {
    MonarchPlan pl;
    size_t per_unit = 0;
    int rc = plan_bwd(desc, &pl, &per_unit);
    if (rc) return rc;
    if (!q || !k || !v || !dout || !dq || !dk || !dv) {
        set_error("q, k, v, dout, dq, dk and dv must be non-NULL");
        return SFM_ERR_NULL;
    }
    if (!aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(dout) || !aligned16(dq) || !aligned16(dk) || !aligned16(dv)) {
        set_error("tensors must be 16-byte aligned");
        return SFM_ERR_ALIGN;
    }
    if (!workspace || (((uintptr_t)workspace) & 255)) {
        set_error("workspace must be non-NULL and 256-byte aligned");
        return SFM_ERR_WORKSPACE;
    }
    if (bwd_uses_chain(desc, pl)) {
        MonarchBwdArgs g;
        memset(&g, 0, sizeof(g));
        init_args(&desc->fwd, pl, &g.p);
        int n = pl.units;
        while (n > 1 && monarch_bwd_gemm_bytes(g.p, desc->fwd.dtype, n, desc->dkv_stride) > workspace_bytes) --n;
        if (monarch_bwd_gemm_bytes(g.p, desc->fwd.dtype, n, desc->dkv_stride) > workspace_bytes) {
            set_error("workspace holds %zu bytes, one (batch, head) unit needs %zu", workspace_bytes,
                      monarch_bwd_gemm_bytes(g.p, desc->fwd.dtype, 1, desc->dkv_stride));
            return SFM_ERR_WORKSPACE;
        }
        g.p.q = q; g.p.k = k; g.p.v = v;
        g.dout = dout; g.dq = dq; g.dk = dk; g.dv = dv;
        g.fout = out; g.fstats = stats;
        for (int i = 0; i < 3; ++i) {
            g.dos[i] = desc->fwd.o_stride[i];
            g.dqs[i] = desc->dq_stride[i];
            g.dks[i] = desc->dkv_stride[i];
        }
        g.kv_f0 = desc->kv_grad_frame_start;
        g.kv_f1 = desc->kv_grad_frame_end;
        g.dk_row0 = (int64_t)g.kv_f0 * pl.b1 * pl.b2;
        for (int u0 = 0; u0 < pl.units; u0 += n) {
            g.p.unit0 = u0;
            rc = launch_monarch_bwd_gemm(g, desc->fwd.dtype, pl.units - u0 < n ? pl.units - u0 : n, workspace, (hipStream_t)stream);
            if (rc) return rc;
        }
        return SFM_OK;
    }
    if (workspace_bytes < per_unit) {
        set_error("workspace must hold at least %zu bytes (one unit)", per_unit);
        return SFM_ERR_WORKSPACE;
    }
    const size_t rows = (size_t)pl.na * pl.b2 * pl.r_pad;
    // 32-bit element offsets into each scratch matrix (float)
    size_t upp_sz = workspace_bytes / per_unit;
    const size_t cap = (((size_t)1 << 31) - 1) / (rows * desc->fwd.D);
    if (upp_sz > cap) upp_sz = cap;
    if (upp_sz < 1) {
        set_error("one (batch, head) unit needs %zu bytes of scratch, more than a pass can address", per_unit);
        return SFM_ERR_UNSUPPORTED;
    }
    const int upp = upp_sz > (size_t)pl.units ? pl.units : (int)upp_sz;

    MonarchBwdArgs g;
    memset(&g, 0, sizeof(g));
    init_args(&desc->fwd, pl, &g.p);
    g.p.q = q; g.p.k = k; g.p.v = v; g.p.out = nullptr;
    g.dout = dout; g.dq = dq; g.dk = dk; g.dv = dv;
    for (int i = 0; i < 3; ++i) {
        g.dos[i] = desc->fwd.o_stride[i];
        g.dqs[i] = desc->dq_stride[i];
        g.dks[i] = desc->dkv_stride[i];
    }
    g.kv_f0 = desc->kv_grad_frame_start;
    g.kv_f1 = desc->kv_grad_frame_end;
    g.dk_row0 = (int64_t)g.kv_f0 * pl.b1 * pl.b2;       // non-zero only in block order
    const size_t mat = rows * desc->fwd.D * sizeof(float);
    for (int u0 = 0; u0 < pl.units; u0 += upp) {
        const int n = pl.units - u0 < upp ? pl.units - u0 : upp;
        g.p.unit0 = u0;
        char* w = (char*)workspace;
        g.p.kbar = w;
        g.p.y = w + mat * upp;
        g.dkbar = (float*)(w + 2 * mat * upp);
        g.dy = (float*)(w + 3 * mat * upp);
        g.p.cl = (float*)(w + 4 * mat * upp);
        g.dcl = g.p.cl + rows * upp;
        rc = launch_monarch_bwd(g, desc->fwd.dtype, n, (hipStream_t)stream);
        if (rc) return rc;
    }
    return SFM_OK;
}

int sfm_kv_cache_write(int32_t dtype, int32_t B, int32_t H, int32_t D, const sfm_tiling* tiling, const void* new_k,
                       const void* new_v, const int64_t new_stride[3], void* k_cache, void* v_cache,
                       const int64_t cache_stride[3], int64_t cache_tokens, int64_t start_idx, int64_t end_idx,
                       void* stream) {
    if (!tiling || !new_k || !new_v || !new_stride || !k_cache || !v_cache || !cache_stride) {
        set_error("NULL argument");
        return SFM_ERR_NULL;
    }
    if (dtype != SFM_BF16 && dtype != SFM_F16 && dtype != SFM_F32) {
        set_error("unsupported dtype %d", dtype);
        return SFM_ERR_DTYPE;
    }
    if (B < 1 || H < 1 || D < 8 || D % 8) {
        set_error("B=%d, H=%d, D=%d invalid", B, H, D);
        return SFM_ERR_SHAPE;
    }
    int rc = check_tiling(*tiling);
    if (rc) return rc;
    const int64_t group = (int64_t)tiling->f_tied * tiling->h * tiling->w;
    const int64_t n = end_idx - start_idx;
    if (start_idx < 0 || end_idx > cache_tokens || n < 0) {
        set_error("start_idx=%lld, end_idx=%lld outside the cache of %lld tokens", (long long)start_idx,
                  (long long)end_idx, (long long)cache_tokens);
        return SFM_ERR_RANGE;
    }
    if (n % group) {
        set_error("end_idx - start_idx = %lld is not a multiple of f_tied*h*w = %lld", (long long)n, (long long)group);
        return SFM_ERR_RANGE;
    }
    const int esz = elem_size(dtype);
    if ((rc = check_strides("new_k/new_v", new_stride, n, H, D, B, esz))) return rc;
    if ((rc = check_strides("k_cache/v_cache", cache_stride, cache_tokens, H, D, B, esz))) return rc;
    if (!aligned16(new_k) || !aligned16(new_v) || !aligned16(k_cache) || !aligned16(v_cache)) {
        set_error("tensors must be 16-byte aligned");
        return SFM_ERR_ALIGN;
    }
    if (n == 0) return SFM_OK;
    TokMap map = make_map(*tiling, 1);
    const int nbf = (int)(n / group) * tiling->h_reduce * tiling->w_reduce;
    return launch_kv_cache_write(esz, B, H, D, map, nbf, new_k, new_v, new_stride, k_cache, v_cache, cache_stride,
                                 start_idx, (hipStream_t)stream);
}

int sfm_monarch_attn_with_kv_cache(const sfm_monarch_desc* desc, const void* q, void* k_cache, void* v_cache,
                                   const void* new_k, const void* new_v, const int64_t new_stride[3],
                                   int64_t start_idx, int64_t end_idx, void* out, void* workspace,
                                   size_t workspace_bytes, void* stream) {
    MonarchPlan pl;
    int rc = plan_monarch(desc, &pl);
    if (rc) return rc;
    if (!desc->kv_block_order) {
        set_error("the KV cache holds rows in Monarch block order: kv_block_order must be 1");
        return SFM_ERR_UNSUPPORTED;
    }
    if (desc->causal_block_frames) {
        set_error("the KV-cache op takes no causal mask");
        return SFM_ERR_UNSUPPORTED;
    }
    const int64_t blk = (int64_t)pl.b1 * pl.b2;
    if (start_idx < 0 || end_idx < start_idx || end_idx > desc->kv_tokens) {
        set_error("start_idx=%lld, end_idx=%lld outside the cache view of %d tokens", (long long)start_idx,
                  (long long)end_idx, desc->kv_tokens);
        return SFM_ERR_RANGE;
    }
    if (start_idx % blk || end_idx % blk) {
        set_error("start_idx=%lld / end_idx=%lld must be multiples of b1*b2=%lld", (long long)start_idx,
                  (long long)end_idx, (long long)blk);
        return SFM_ERR_RANGE;
    }
    // validate everything the forward will check BEFORE the cache is touched
    if (!q || !k_cache || !v_cache || !out || !new_k || !new_v || !new_stride) {
        set_error("NULL argument");
        return SFM_ERR_NULL;
    }
    if (!aligned16(q) || !aligned16(k_cache) || !aligned16(v_cache) || !aligned16(out)) {
        set_error("q, caches and out must be 16-byte aligned");
        return SFM_ERR_ALIGN;
    }
    if (!workspace || (((uintptr_t)workspace) & 255) || workspace_bytes < pl.per_unit) {
        set_error("workspace must be non-NULL, 256-byte aligned and hold at least %zu bytes (one unit)", pl.per_unit);
        return SFM_ERR_WORKSPACE;
    }
    rc = sfm_kv_cache_write(desc->dtype, desc->B, desc->H, desc->D, &desc->tiling, new_k, new_v, new_stride, k_cache,
                            v_cache, desc->k_stride, desc->kv_tokens, start_idx, end_idx, stream);
    if (rc) return rc;
    return sfm_monarch_fwd(desc, q, k_cache, v_cache, out, workspace, workspace_bytes, stream);
}

}  // extern "C"

// Scratch of sfm_monarch_attn_with_kv_cache_static: one array per GPU, allocated with the code object and held until
// the process ends.  In host code the array's name only stands for the symbol; the device address is looked up once per
// device and that pointer is what the kernels, and every other use on the host, get.
static __device__ __align__(256) unsigned char scratch[SFM_STATIC_SCRATCH_BYTES];

namespace {
constexpr int kMaxDevices = 64;
void* g_scratch_ptr[kMaxDevices];
bool g_scratch_ok[kMaxDevices];
pthread_mutex_t g_scratch_mutex = PTHREAD_MUTEX_INITIALIZER;

// Device address of `scratch` on the current device (looked up on the first call per device).
int static_scratch_ptr(void** out) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess || dev < 0 || dev >= kMaxDevices) {
        set_error("static scratch: no current device (%s)", e == hipSuccess ? "device index out of range" : hipGetErrorString(e));
        return SFM_ERR_HIP;
    }
    pthread_mutex_lock(&g_scratch_mutex);
    if (!g_scratch_ok[dev]) {
        void* ptr = nullptr;
        e = hipGetSymbolAddress((void**)&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !ptr) {
            pthread_mutex_unlock(&g_scratch_mutex);
            set_error("hipGetSymbolAddress(scratch) failed on device %d: %s", dev, hipGetErrorString(e));
            return SFM_ERR_HIP;
        }
        g_scratch_ptr[dev] = ptr;
        g_scratch_ok[dev] = true;
    }
    *out = g_scratch_ptr[dev];
    pthread_mutex_unlock(&g_scratch_mutex);
    return SFM_OK;
}
}  // namespace

extern "C" {

int sfm_monarch_attn_with_kv_cache_static(const sfm_monarch_desc* desc, const void* q, void* k_cache, void* v_cache,
                                          const void* new_k, const void* new_v, const int64_t new_stride[3],
                                          int64_t start_idx, int64_t end_idx, void* out, void* stream) {
    MonarchPlan pl;
    int rc = plan_monarch(desc, &pl);
    if (rc) return rc;
    if (pl.per_unit > (size_t)SFM_STATIC_SCRATCH_BYTES) {
        set_error("one (batch, head) unit needs %zu bytes of scratch, more than the %zu-byte static scratch of this entry "
                  "point; use sfm_monarch_attn_with_kv_cache with a caller-owned workspace",
                  pl.per_unit, (size_t)SFM_STATIC_SCRATCH_BYTES);
        return SFM_ERR_WORKSPACE;
    }
    void* ws = nullptr;
    if ((rc = static_scratch_ptr(&ws))) return rc;
    // Every pass overwrites the rows of the scratch that it reads (step 1 writes each Kbar / Y / cl row that step 2
    // loads), so nothing of an earlier call's contents has to be cleared.
    return sfm_monarch_attn_with_kv_cache(desc, q, k_cache, v_cache, new_k, new_v, new_stride, start_idx, end_idx, out, ws,
                                          (size_t)SFM_STATIC_SCRATCH_BYTES, stream);
}

static int check_dense(const sfm_dense_desc* d) {
    if (!d) {
        set_error("desc is NULL");
        return SFM_ERR_NULL;
    }
    if (d->dtype != SFM_BF16 && d->dtype != SFM_F16 && d->dtype != SFM_F32) {
        set_error("unsupported dtype %d", d->dtype);
        return SFM_ERR_DTYPE;
    }
    if (d->B < 1 || d->H < 1 || d->D < 8 || d->D % 8 || d->D > 256 || d->q_tokens < 1 || d->kv_tokens < 1) {
        set_error("B=%d, H=%d, D=%d, q_tokens=%d, kv_tokens=%d invalid", d->B, d->H, d->D, d->q_tokens, d->kv_tokens);
        return SFM_ERR_SHAPE;
    }
    if (!(d->sm_scale > 0.f)) {
        set_error("sm_scale must be a positive number");
        return SFM_ERR_SHAPE;
    }
    const int esz = elem_size(d->dtype);
    int rc;
    if ((rc = check_strides("q", d->q_stride, d->q_tokens, d->H, d->D, d->B, esz))) return rc;
    if ((rc = check_strides("k", d->k_stride, d->kv_tokens, d->H, d->D, d->B, esz))) return rc;
    if ((rc = check_strides("v", d->v_stride, d->kv_tokens, d->H, d->D, d->B, esz))) return rc;
    if ((rc = check_strides("out", d->o_stride, d->q_tokens, d->H, d->D, d->B, esz))) return rc;
    return SFM_OK;
}

int sfm_dense_fwd(const sfm_dense_desc* desc, const void* q, const void* k, const void* v, void* out, float* lse,
                  void* stream) {
    int rc = check_dense(desc);
    if (rc) return rc;
    if (!q || !k || !v || !out) {
        set_error("q, k, v and out must be non-NULL");
        return SFM_ERR_NULL;
    }
    if (!aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(out)) {
        set_error("q, k, v and out must be 16-byte aligned");
        return SFM_ERR_ALIGN;
    }
    return launch_dense(*desc, q, k, v, out, lse, (hipStream_t)stream);
}

int sfm_full_attention_with_kv_cache(const sfm_dense_desc* desc, const void* q, void* k_cache, void* v_cache,
                                     const void* new_k, const void* new_v, const int64_t new_stride[3],
                                     int64_t start_idx, int64_t end_idx, void* out, float* lse, void* stream) {
    int rc = check_dense(desc);
    if (rc) return rc;
    if (!q || !k_cache || !v_cache || !out || !new_k || !new_v || !new_stride) {
        set_error("NULL argument");
        return SFM_ERR_NULL;
    }
    if (start_idx < 0 || end_idx < start_idx || end_idx > desc->kv_tokens) {
        set_error("start_idx=%lld, end_idx=%lld outside the cache view of %d tokens", (long long)start_idx,
                  (long long)end_idx, desc->kv_tokens);
        return SFM_ERR_RANGE;
    }
    if (memcmp(desc->k_stride, desc->v_stride, sizeof(desc->k_stride)) != 0) {
        set_error("k_cache and v_cache must share strides");
        return SFM_ERR_STRIDE;
    }
    if (!aligned16(q) || !aligned16(k_cache) || !aligned16(v_cache) || !aligned16(out) || !aligned16(new_k) ||
        !aligned16(new_v)) {
        set_error("tensors must be 16-byte aligned");
        return SFM_ERR_ALIGN;
    }
    const int64_t n = end_idx - start_idx;
    if (n > 0) {
        // token-order slice assignment = the identity tiling with one "frame" of n tokens
        sfm_tiling ident = {1, 1, 1, 1, (int32_t)n};
        rc = sfm_kv_cache_write(desc->dtype, desc->B, desc->H, desc->D, &ident, new_k, new_v, new_stride, k_cache,
                                v_cache, desc->k_stride, desc->kv_tokens, start_idx, end_idx, stream);
        if (rc) return rc;
    }
    return launch_dense(*desc, q, k_cache, v_cache, out, lse, (hipStream_t)stream);
}

static int check_dense_bwd(const sfm_dense_bwd_desc* bd) {
    if (!bd) {
        set_error("desc is NULL");
        return SFM_ERR_NULL;
    }
    int rc = check_dense(&bd->fwd);
    if (rc) return rc;
    if (!dense_bwd_supported(bd->fwd.dtype, bd->fwd.D)) {
        set_error("dense backward: bf16 / fp16 tensors with head_dim 64 or 128 only");
        return SFM_ERR_UNSUPPORTED;
    }
    if (bd->kv_grad_start < 0 || bd->kv_grad_end > bd->fwd.kv_tokens || bd->kv_grad_start > bd->kv_grad_end) {
        set_error("kv gradient range [%lld, %lld) outside [0, %d)", (long long)bd->kv_grad_start, (long long)bd->kv_grad_end,
                  bd->fwd.kv_tokens);
        return SFM_ERR_RANGE;
    }
    if ((rc = check_strides("dq", bd->dq_stride, bd->fwd.q_tokens, bd->fwd.H, bd->fwd.D, bd->fwd.B, 4))) return rc;
    if (bd->kv_grad_end > bd->kv_grad_start &&
        (rc = check_strides("dk/dv", bd->dkv_stride, bd->kv_grad_end - bd->kv_grad_start, bd->fwd.H, bd->fwd.D, bd->fwd.B, 2)))
        return rc;
    return SFM_OK;
}

int sfm_dense_bwd_workspace_bytes(const sfm_dense_bwd_desc* desc, size_t* bytes) {
    if (!bytes) {
        set_error("bytes is NULL");
        return SFM_ERR_NULL;
    }
    int rc = check_dense_bwd(desc);
    if (rc) return rc;
    *bytes = ((size_t)2 * desc->fwd.B * desc->fwd.H * desc->fwd.q_tokens * sizeof(float) + 255) / 256 * 256;
    return SFM_OK;
}

int sfm_dense_bwd(const sfm_dense_bwd_desc* desc, const void* q, const void* k, const void* v, const void* out, const float* lse,
                  const void* dout, float* dq, void* dk, void* dv, void* workspace, size_t workspace_bytes, void* stream) {
    int rc = check_dense_bwd(desc);
    if (rc) return rc;
    const bool want_kv = desc->kv_grad_end > desc->kv_grad_start;
    if (!q || !k || !v || !out || !lse || !dout || !dq || (want_kv && (!dk || !dv))) {
        set_error("q, k, v, out, lse, dout, dq (and dk, dv for a non-empty key range) must be non-NULL");
        return SFM_ERR_NULL;
    }
    if (!aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(out) || !aligned16(dout) || !aligned16(dq) ||
        !aligned16(dk) || !aligned16(dv) || (((uintptr_t)lse) & 3)) {
        set_error("tensors must be 16-byte aligned (lse: 4-byte)");
        return SFM_ERR_ALIGN;
    }
    const size_t need = (size_t)2 * desc->fwd.B * desc->fwd.H * desc->fwd.q_tokens * sizeof(float);
    if (!workspace || (((uintptr_t)workspace) & 255) || workspace_bytes < need) {
        set_error("workspace must be non-NULL, 256-byte aligned and hold at least %zu bytes", need);
        return SFM_ERR_WORKSPACE;
    }
    return launch_dense_bwd(desc->fwd, desc->dq_stride, desc->dkv_stride, desc->kv_grad_start, desc->kv_grad_end, q, k, v, out, lse,
                            dout, dq, dk, dv, (float*)workspace, (hipStream_t)stream);
}

int sfm_qk_prologue(const sfm_prologue_desc* d, const void* xq, const void* xk, const void* xv, const void* wq,
                    const void* wk, const double* rope_cos_sin, int32_t rope_max_pos, void* q_out, void* k_cache,
                    void* v_cache, void* stream) {
    if (!d || !xq || !xk || !xv || !wq || !wk || !rope_cos_sin || !q_out || !k_cache || !v_cache) {
        set_error("NULL argument");
        return SFM_ERR_NULL;
    }
    if (d->dtype != SFM_BF16 && d->dtype != SFM_F16 && d->dtype != SFM_F32) {
        set_error("unsupported dtype %d", d->dtype);
        return SFM_ERR_DTYPE;
    }
    if (d->B < 1 || d->H < 1 || d->D < 8 || d->D % 8 || d->S < 1 || d->F < 1 || d->h < 1 || d->w < 1 ||
        (int64_t)d->F * d->h * d->w != d->S) {
        set_error("B=%d, S=%d, H=%d, D=%d, grid=(%d,%d,%d): need S == F*h*w and D a multiple of 8", d->B, d->S, d->H,
                  d->D, d->F, d->h, d->w);
        return SFM_ERR_SHAPE;
    }
    if ((int64_t)d->H * d->D > 8192) {
        set_error("model dim %d exceeds the 8192 the fused prologue handles", d->H * d->D);
        return SFM_ERR_UNSUPPORTED;
    }
    int rc = check_tiling(d->tiling);
    if (rc) return rc;
    if (d->tiling.h != d->h || d->tiling.w != d->w || d->F % d->tiling.f_tied) {
        set_error("tiling (h=%d, w=%d, f_tied=%d) does not match the grid (%d,%d,%d)", d->tiling.h, d->tiling.w,
                  d->tiling.f_tied, d->F, d->h, d->w);
        return SFM_ERR_SHAPE;
    }
    if (d->start_frame < 0 || d->start_frame + d->F > rope_max_pos || d->h > rope_max_pos || d->w > rope_max_pos) {
        set_error("RoPE positions exceed the table of %d rows", rope_max_pos);
        return SFM_ERR_RANGE;
    }
    if (d->start_idx < 0 || d->start_idx + d->S > d->cache_tokens) {
        set_error("start_idx=%lld + S=%d exceeds the cache of %lld tokens", (long long)d->start_idx, d->S,
                  (long long)d->cache_tokens);
        return SFM_ERR_RANGE;
    }
    const int esz = elem_size(d->dtype);
    const int64_t C = (int64_t)d->H * d->D;
    if (d->x_stride[1] < C || (d->x_stride[0] * esz) % 16 || (d->x_stride[1] * esz) % 16) {
        set_error("x strides invalid");
        return SFM_ERR_STRIDE;
    }
    if ((rc = check_strides("q_out", d->q_stride, d->S, d->H, d->D, d->B, esz))) return rc;
    if ((rc = check_strides("k_cache/v_cache", d->cache_stride, d->cache_tokens, d->H, d->D, d->B, esz))) return rc;
    if (!aligned16(xq) || !aligned16(xk) || !aligned16(xv) || !aligned16(wq) || !aligned16(wk) || !aligned16(q_out) ||
        !aligned16(k_cache) || !aligned16(v_cache) || !aligned16(rope_cos_sin)) {
        set_error("tensors must be 16-byte aligned");
        return SFM_ERR_ALIGN;
    }
    TokMap map = make_map(d->tiling, 1);
    return launch_prologue(*d, map, xq, xk, xv, wq, wk, rope_cos_sin, q_out, k_cache, v_cache, (hipStream_t)stream);
}

int sfm_ln_modulate(int32_t dtype, int64_t rows, int32_t C, float eps, const void* x, int64_t x_stride, void* y,
                    int64_t y_stride, const void* scale, const void* shift, int64_t mod_stride, int32_t rows_per_frame,
                    const void* weight, const void* bias, void* stream) {
    int rc = check_rows(dtype, rows, C, x_stride, y_stride);
    if (rc) return rc;
    const bool affine = weight != nullptr || bias != nullptr;
    if (!x || !y || (affine && (!weight || !bias)) || (!affine && (!scale || !shift))) {
        set_error("x, y and either (scale, shift) or (weight, bias) must be non-NULL");
        return SFM_ERR_NULL;
    }
    if (!affine && (rows_per_frame < 1 || mod_stride < 0 || (mod_stride * (dtype == SFM_F32 ? 4 : 2)) % 16)) {
        set_error("rows_per_frame must be >= 1 and mod_stride a multiple of 16 bytes");
        return SFM_ERR_STRIDE;
    }
    if (!aligned16(x) || !aligned16(y) || !aligned16(scale) || !aligned16(shift) || !aligned16(weight) || !aligned16(bias)) {
        set_error("tensors must be 16-byte aligned");
        return SFM_ERR_ALIGN;
    }
    return launch_ln_modulate(dtype, rows, C, eps, x, x_stride, y, y_stride, scale, shift, mod_stride,
                              affine ? 1 : rows_per_frame, weight, bias, (hipStream_t)stream);
}

int sfm_gate_residual_ln(int32_t dtype, int64_t rows, int32_t C, float eps, void* x, int64_t x_stride, const void* y,
                         int64_t y_stride, const void* gate, int64_t gate_stride, int32_t gate_rows_per_frame, void* out,
                         int64_t out_stride, const void* scale, const void* shift, int64_t mod_stride, int32_t rows_per_frame,
                         const void* weight, const void* bias, void* stream) {
    int rc = check_rows(dtype, rows, C, x_stride, y_stride);
    if (!rc) rc = check_rows(dtype, rows, C, x_stride, out_stride);
    if (rc) return rc;
    const bool affine = weight != nullptr || bias != nullptr;
    if (!x || !y || !out || (affine && (!weight || !bias)) || (!affine && (!scale || !shift))) {
        set_error("x, y, out and either (scale, shift) or (weight, bias) must be non-NULL");
        return SFM_ERR_NULL;
    }
    const int esz = dtype == SFM_F32 ? 4 : 2;
    if ((gate && (gate_rows_per_frame < 1 || gate_stride < 0 || (gate_stride * esz) % 16)) ||
        (!affine && (rows_per_frame < 1 || mod_stride < 0 || (mod_stride * esz) % 16))) {
        set_error("rows_per_frame must be >= 1 and modulation strides multiples of 16 bytes");
        return SFM_ERR_STRIDE;
    }
    if (!aligned16(x) || !aligned16(y) || !aligned16(out) || !aligned16(gate) || !aligned16(scale) || !aligned16(shift) ||
        !aligned16(weight) || !aligned16(bias)) {
        set_error("tensors must be 16-byte aligned");
        return SFM_ERR_ALIGN;
    }
    return launch_gate_residual_ln(dtype, rows, C, eps, x, x_stride, y, y_stride, gate, gate_stride, gate ? gate_rows_per_frame : 1,
                                   out, out_stride, scale, shift, mod_stride, affine ? 1 : rows_per_frame, weight, bias,
                                   (hipStream_t)stream);
}

int sfm_gate_residual(int32_t dtype, int64_t rows, int32_t C, void* x, int64_t x_stride, const void* y, int64_t y_stride,
                      const void* gate, int64_t mod_stride, int32_t rows_per_frame, void* stream) {
    int rc = check_rows(dtype, rows, C, x_stride, y_stride);
    if (rc) return rc;
    if (!x || !y) {
        set_error("x and y must be non-NULL");
        return SFM_ERR_NULL;
    }
    if (gate && (rows_per_frame < 1 || mod_stride < 0 || (mod_stride * (dtype == SFM_F32 ? 4 : 2)) % 16)) {
        set_error("rows_per_frame must be >= 1 and mod_stride a multiple of 16 bytes");
        return SFM_ERR_STRIDE;
    }
    if (!aligned16(x) || !aligned16(y) || !aligned16(gate)) {
        set_error("tensors must be 16-byte aligned");
        return SFM_ERR_ALIGN;
    }
    return launch_gate_residual(dtype, rows, C, x, x_stride, y, y_stride, gate, mod_stride, gate ? rows_per_frame : 1,
                                (hipStream_t)stream);
}

int sfm_linear(const sfm_linear_desc* d, const void* x, const void* w, const void* bias, const void* res, const void* gate,
               void* out, void* stream) {
    if (!d || !x || !w || !out) {
        set_error("desc, x, w and out must be non-NULL");
        return SFM_ERR_NULL;
    }
    if (d->dtype != SFM_BF16 && d->dtype != SFM_F16) {
        set_error("sfm_linear takes 16-bit tensors (dtype %d)", d->dtype);
        return SFM_ERR_DTYPE;
    }
    if (d->epilogue < SFM_EPI_NONE || d->epilogue > SFM_EPI_GATE_RESIDUAL) {
        set_error("unknown epilogue %d", d->epilogue);
        return SFM_ERR_SHAPE;
    }
    if (d->M < 1 || d->N < 8 || d->N % 8 || d->K < 64 || d->K % 64) {
        set_error("M=%lld, N=%d, K=%d: need M >= 1, N a multiple of 8 and K a multiple of 64", (long long)d->M, d->N, d->K);
        return SFM_ERR_SHAPE;
    }
    if (d->tile_rows != 0 && d->tile_rows != 128 && d->tile_rows != 256) {
        set_error("tile_rows must be 0, 128 or 256");
        return SFM_ERR_SHAPE;
    }
    const bool gr = d->epilogue == SFM_EPI_GATE_RESIDUAL;
    if (gr && !res) {
        set_error("the gated-residual epilogue needs res");
        return SFM_ERR_NULL;
    }
    if (d->x_stride < d->K || d->x_stride % 8 || d->out_stride < d->N || d->out_stride % 8 ||
        (gr && (d->res_stride < d->N || d->res_stride % 8)) ||
        (gr && gate && (d->rows_per_frame < 1 || d->gate_stride < 0 || d->gate_stride % 8))) {
        set_error("row strides must cover a row and be multiples of 8 elements; rows_per_frame >= 1");
        return SFM_ERR_STRIDE;
    }
    if ((uint64_t)d->M * (uint64_t)d->x_stride * 2 >= ((uint64_t)1 << 32) || (uint64_t)d->N * (uint64_t)d->K * 2 >= ((uint64_t)1 << 32)) {
        set_error("x and w must span less than 4 GiB each");
        return SFM_ERR_SHAPE;
    }
    if (!aligned16(x) || !aligned16(w) || !aligned16(bias) || !aligned16(res) || !aligned16(gate) || !aligned16(out)) {
        set_error("tensors must be 16-byte aligned");
        return SFM_ERR_ALIGN;
    }
    // the product reads whole rows of x and w while other workgroups already write out: they must not overlap
    // (res may be out: every element is read and written by the same lane)
    const char* o0 = (const char*)out;
    const char* o1 = o0 + ((size_t)(d->M - 1) * d->out_stride + d->N) * 2;
    const char* x0 = (const char*)x;
    const char* x1 = x0 + ((size_t)(d->M - 1) * d->x_stride + d->K) * 2;
    const char* w0 = (const char*)w;
    const char* w1 = w0 + (size_t)d->N * d->K * 2;
    if ((x0 < o1 && o0 < x1) || (w0 < o1 && o0 < w1)) {
        set_error("out overlaps x or w");
        return SFM_ERR_RANGE;
    }
    return launch_linear(*d, x, w, bias, gr ? res : nullptr, gr ? gate : nullptr, out, (hipStream_t)stream);
}

int sfm_rms_norm(int32_t dtype, int64_t rows, int32_t C, float eps, const void* x, int64_t x_stride, void* y,
                 int64_t y_stride, const void* weight, void* stream) {
    int rc = check_rows(dtype, rows, C, x_stride, y_stride);
    if (rc) return rc;
    if (!x || !y || !weight) {
        set_error("x, y and weight must be non-NULL");
        return SFM_ERR_NULL;
    }
    if (!aligned16(x) || !aligned16(y) || !aligned16(weight)) {
        set_error("tensors must be 16-byte aligned");
        return SFM_ERR_ALIGN;
    }
    return launch_rms_norm(dtype, rows, C, eps, x, x_stride, y, y_stride, weight, (hipStream_t)stream);
}

}  // extern "C"
