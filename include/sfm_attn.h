/* sfm_attn.h -- C ABI of the MI355X (gfx950) Monarch / KV-cache attention library.
 *
 * Plain pointers and sizes only; every entry point returns 0 on success or a negative
 * SFM_ERR_* code, never aborts, allocates nothing, keeps no global state besides a
 * thread-local error string, and enqueues its work on the hipStream_t passed as `stream`
 * (NULL = the default stream) without synchronising.  All tensor pointers are device
 * pointers; strides are in ELEMENTS; the innermost (head_dim) axis is contiguous.
 *
 * Citations are file:line of the reference (krishagarwal/Self-Forcing) interface each
 * entry point replaces.
 */
#ifndef SFM_ATTN_H
#define SFM_ATTN_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SFM_OK               0
#define SFM_ERR_NULL        -1   /* a required pointer is NULL */
#define SFM_ERR_DTYPE       -2   /* dtype not one of SFM_BF16 / SFM_F16 / SFM_F32 (or not allowed for the op) */
#define SFM_ERR_SHAPE       -3   /* sizes inconsistent with the tiling (e.g. tokens not a multiple of b1*b2) */
#define SFM_ERR_RANGE       -4   /* start/end index out of range or not aligned to a block-frame */
#define SFM_ERR_STRIDE      -5   /* stride too small / K and V strides differ where they must agree */
#define SFM_ERR_WORKSPACE   -6   /* workspace NULL, misaligned or too small */
#define SFM_ERR_ALIGN       -7   /* a tensor pointer is not 16-byte aligned */
#define SFM_ERR_HIP         -8   /* the HIP runtime refused a launch (see sfm_last_error) */
#define SFM_ERR_UNSUPPORTED -9   /* combination not implemented */

#define SFM_BF16 0
#define SFM_F16  1
#define SFM_F32  2

/* Token tiling of the Monarch op: wan/modules/monarch_attn.py:1696-1703 (_get_rearrange_fns).
 * Tokens are (frame,row,col) ordered with h rows x w cols per frame.
 *   b1 = f_tied*h/h_reduce rows per block, b2 = w/w_reduce cols per block,
 *   block-frames = tokens/(f_tied*h*w) * h_reduce*w_reduce. */
typedef struct sfm_tiling {
    int32_t f_tied, h_reduce, w_reduce, h, w;
} sfm_tiling;

/* sfm_monarch_desc.flags: run the forward as ONE kernel that keeps Kbar / Y / cl in LDS instead of the workspace, where
 * that kernel applies (16-bit tensors, head_dim 128, b1 <= 32, b2 <= 64, no causal mask, num_iters 1; elsewhere the
 * flag is ignored).  Its workspace is a few MB per unit instead of tens; at the 480p shapes it is slower than the two
 * kernels (it re-reads every K/V tile once per group of 12 (a, j) columns), so it is opt-in.  Results agree to rounding. */
#define SFM_MONARCH_ONE_KERNEL 1

typedef struct sfm_monarch_desc {
    int32_t dtype;            /* SFM_BF16 | SFM_F16 | SFM_F32 : type of q, k, v, out */
    int32_t B, H, D;          /* batch, heads, head_dim */
    int32_t q_tokens;         /* Sq  (multiple of f_tied*h*w) */
    int32_t kv_tokens;        /* Skv (multiple of f_tied*h*w): the whole cache view / key sequence */
    sfm_tiling tiling;
    int32_t kv_block_order;   /* 1: k/v rows are stored in Monarch block order (KV-cache layout,
                                 monarch_attn.py:1784-1785, 1233-1234); 0: token order like q */
    int32_t causal_block_frames; /* 0 = every query sees every key; else block-causal in units of
                                 block-frames (monarch_attn.py:139-141, 804-807), requires Sq == Skv */
    float   sm_scale;         /* logit scale; the reference default is D^-0.5 (monarch_attn.py:1780-1781) */
    int32_t num_iters;        /* 1: the two-kernel fast path; > 1: alternating refinement of the two factors
                                 (monarch_attn_slow, monarch_attn.py:1705-1751), no causal mask.  Both run MFMA kernels
                                 for 16-bit tensors with head_dim 64 / 128 and b2 <= 128 (refinement: b1 <= 128 as well),
                                 fp32 SIMT kernels for everything else */
    int32_t flags;            /* 0, or SFM_MONARCH_ONE_KERNEL */
    int64_t q_stride[3];      /* batch, token, head */
    int64_t k_stride[3];
    int64_t v_stride[3];      /* must equal k_stride (monarch_attn.py:1261) */
    int64_t o_stride[3];
} sfm_monarch_desc;

/* Bytes of device scratch sfm_monarch_fwd needs when it processes `heads_per_pass`
 * (batch x head) units at a time (0 = library default).  Replaces the per-call torch.empty
 * scratch of monarch_attn.py:1246-1259.  The size is not proportional to heads_per_pass. */
int sfm_monarch_workspace_bytes(const sfm_monarch_desc* desc, int32_t heads_per_pass, size_t* bytes);

/* One-iteration Monarch attention forward.  Replaces _attention_with_cache.forward /
 * _attention_no_cache.forward and their two Triton kernels: monarch_attn.py:1225-1323,
 * 1472-1563, 109-253 (_al_cl_y_fwd), 698-842 (_z_fwd).  q and out are in token order.
 * The number of (batch x head) units per pass is derived from workspace_bytes (as many as it holds). */
int sfm_monarch_fwd(const sfm_monarch_desc* desc, const void* q, const void* k, const void* v, void* out,
                    void* workspace, size_t workspace_bytes, void* stream);

/* Forward that also keeps what the backward can reuse, as the reference's forward does under autograd
 * (OUTPUT_FULL_LSE and ctx.save_for_backward(q, k, v, z, z_lse), monarch_attn.py:1309, 1317, 1559): `stats` receives
 * one float per (batch, head, query token), the base-2 log-sum-exp of the row's left-factor logits, in the library's
 * own order (row pitch round_up(b1, 32) per (batch, head, a, j)); treat it as opaque and hand it to
 * sfm_monarch_bwd_saved together with `out`.  sfm_monarch_stats_bytes gives its size, 0 when the forward that would
 * run for this descriptor produces no statistics (then use sfm_monarch_fwd and sfm_monarch_bwd). */
int sfm_monarch_stats_bytes(const sfm_monarch_desc* desc, size_t* bytes);
int sfm_monarch_fwd_stats(const sfm_monarch_desc* desc, const void* q, const void* k, const void* v, void* out, float* stats,
                          void* workspace, size_t workspace_bytes, void* stream);

/* Measurement variant of sfm_monarch_fwd: brackets the two kernels of every pass with hipEvents recorded on
 * `stream`, WAITS for them, and returns the summed kernel durations in milliseconds.  No counterpart in the
 * reference (its pipeline times whole chunks with torch.cuda.Event, pipeline/causal_inference.py:105-115). */
int sfm_monarch_fwd_timed(const sfm_monarch_desc* desc, const void* q, const void* k, const void* v, void* out,
                          void* workspace, size_t workspace_bytes, void* stream, float* step1_ms, float* step2_ms);

/* Backward of sfm_monarch_fwd (num_iters == 1).  Replaces the Triton kernels _z_bwd_preprocess, _z_bwd,
 * _al_cl_y_bwd and their orchestration in _attention_with_cache.backward / _attention_no_cache.backward
 * (monarch_attn.py:852-886, 1034-1222, 403-596, 1326-1470, 1566-1693).
 *   fwd                 the forward descriptor; o_stride describes `dout`
 *   dq                  float32 [B, q_tokens, H, D] (the reference returns grad_q in float32, :1470)
 *   dk, dv              tensor dtype, [B, (kv_grad_frame_end - kv_grad_frame_start) * b1 * b2, H, D], rows in the
 *                       order of k: token order, or block order when fwd.kv_block_order = 1
 *   kv_grad_frame_*     kv block-frames whose gradients are produced; a proper sub-range is the reference's
 *                       grad_only_new_kv (:1364-1374) and needs block order
 * Everything is recomputed from q, k, v (see sfm_monarch_bwd_saved for the variant that reuses the forward's output).  The workspace size depends
 * on the implementation in use (sfm_monarch_bwd_uses_gemm); query it in the same process state. */
typedef struct sfm_monarch_bwd_desc {
    sfm_monarch_desc fwd;
    int64_t dq_stride[3];
    int64_t dkv_stride[3];
    int32_t kv_grad_frame_start;
    int32_t kv_grad_frame_end;
} sfm_monarch_bwd_desc;

int sfm_monarch_bwd_workspace_bytes(const sfm_monarch_bwd_desc* desc, int32_t heads_per_pass, size_t* bytes);
/* 1 when rocBLAS was found at run time and the SFM_SW_BWD_SIMT switch is off.  The backward is a chain of parts, each a fused
 * MFMA kernel where the problem allows (16-bit tensors, head_dim 64 / 128, b1 <= 128, b2 <= 64 a multiple of 4, at
 * most 480 (a, j) columns) and batched rocBLAS GEMMs + row kernels otherwise; when every part is fused the chain
 * runs with or without rocBLAS, else without rocBLAS the fp32 SIMT kernels run.  The first GEMM call on a device
 * creates a rocBLAS handle, which allocates; every other entry point of this header allocates nothing.  No
 * counterpart in the reference. */
int sfm_monarch_bwd_uses_gemm(void);
int sfm_monarch_bwd(const sfm_monarch_bwd_desc* desc, const void* q, const void* k, const void* v, const void* dout,
                    float* dq, void* dk, void* dv, void* workspace, size_t workspace_bytes, void* stream);

/* sfm_monarch_bwd with the forward's output and row statistics (sfm_monarch_fwd_stats on the same descriptor and
 * inputs) at hand, as the reference's backward has z and z_lse (monarch_attn.py:1327, 1567): the left factor's
 * statistics pass is skipped.  `out` has the layout of `dout` (fwd.o_stride).  Same results as sfm_monarch_bwd up to
 * rounding; implementations that cannot use the saved tensors ignore them. */
int sfm_monarch_bwd_saved(const sfm_monarch_bwd_desc* desc, const void* q, const void* k, const void* v, const void* out,
                          const float* stats, const void* dout, float* dq, void* dk, void* dv, void* workspace,
                          size_t workspace_bytes, void* stream);

/* Writes new_k/new_v [B, n_new, H, D] (token order) into k_cache/v_cache[:, start_idx:end_idx]
 * in Monarch block order.  Replaces monarch_attn.py:1784-1785 + 1230-1231.
 * strides: new_stride for new_k and new_v, cache_stride for both caches. */
int sfm_kv_cache_write(int32_t dtype, int32_t B, int32_t H, int32_t D, const sfm_tiling* tiling,
                       const void* new_k, const void* new_v, const int64_t new_stride[3],
                       void* k_cache, void* v_cache, const int64_t cache_stride[3],
                       int64_t cache_tokens, int64_t start_idx, int64_t end_idx, void* stream);

/* monarch_attn_with_kv_cache (monarch_attn.py:1778-1796): cache write at [start_idx,end_idx)
 * followed by sfm_monarch_fwd over the whole cache view (desc->kv_tokens tokens,
 * desc->kv_block_order must be 1). */
int sfm_monarch_attn_with_kv_cache(const sfm_monarch_desc* desc, const void* q, void* k_cache, void* v_cache,
                                   const void* new_k, const void* new_v, const int64_t new_stride[3],
                                   int64_t start_idx, int64_t end_idx, void* out,
                                   void* workspace, size_t workspace_bytes, void* stream);

/* sfm_monarch_attn_with_kv_cache for callers that cannot allocate or hand over a workspace (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  The scratch is a
 * file-scope device array of SFM_STATIC_SCRATCH_BYTES inside the library, one copy per GPU, held until the process
 * ends; the (batch x head) units are processed in as many passes as that size requires.  Returns SFM_ERR_WORKSPACE
 * when a single unit needs more than the array holds (the size sfm_monarch_workspace_bytes reports for
 * heads_per_pass = 1).  The call allocates nothing and never synchronises; its first call on a device looks up the
 * array's address (make that call outside a graph capture).  All calls on one GPU share the array: calls that may
 * overlap on one GPU (different streams, different threads) race on it and must be serialised by the caller. */
#define SFM_STATIC_SCRATCH_BYTES (128u << 20)
int sfm_monarch_attn_with_kv_cache_static(const sfm_monarch_desc* desc, const void* q, void* k_cache, void* v_cache,
                                          const void* new_k, const void* new_v, const int64_t new_stride[3],
                                          int64_t start_idx, int64_t end_idx, void* out, void* stream);

typedef struct sfm_dense_desc {
    int32_t dtype;            /* SFM_BF16 | SFM_F16 (attn_patch.py:317) | SFM_F32 */
    int32_t B, H, D;
    int32_t q_tokens, kv_tokens;
    float   sm_scale;         /* reference default D^-0.5 (attention.py:179-186, attn_patch.py:417-418) */
    int64_t q_stride[3];
    int64_t k_stride[3];
    int64_t v_stride[3];
    int64_t o_stride[3];
} sfm_dense_desc;

/* Dense non-causal softmax attention of q against the first kv_tokens of k/v.  Replaces
 * attention() (attention.py:141-187) and _attn_fwd (attn_patch.py:20-110).  lse (float32,
 * [B,H,q_tokens], natural log) may be NULL. */
int sfm_dense_fwd(const sfm_dense_desc* desc, const void* q, const void* k, const void* v, void* out,
                  float* lse, void* stream);

/* full_attention_with_kv_cache (attn_patch.py:416-419, 305-351): slice-assign new_k/new_v into
 * the cache at [start_idx,end_idx) (token order, no permutation), then sfm_dense_fwd. */
int sfm_full_attention_with_kv_cache(const sfm_dense_desc* desc, const void* q, void* k_cache, void* v_cache,
                                     const void* new_k, const void* new_v, const int64_t new_stride[3],
                                     int64_t start_idx, int64_t end_idx, void* out, float* lse, void* stream);

/* Backward of sfm_dense_fwd / sfm_full_attention_with_kv_cache.  Replaces _attn_bwd_preprocess, _attn_bwd and
 * _attention.backward (attn_patch.py:121-166, 169-302, 354-413): bf16 / fp16, head_dim 64 or 128.
 *   fwd                 the forward descriptor; o_stride describes both `out` and `dout`
 *   out, lse            what the forward returned (lse: float32 [B, H, q_tokens], natural log)
 *   dq                  float32 [B, q_tokens, H, D] (the reference accumulates and returns grad_q in float32, :361, :413)
 *   dk, dv              tensor dtype, [B, kv_grad_end - kv_grad_start, H, D]: gradients of keys kv_grad_start ..
 *                       kv_grad_end - 1; a proper sub-range is the reference's grad_only_new_kv (:362-364); an empty
 *                       range produces dq only
 *   workspace           sfm_dense_bwd_workspace_bytes (two floats per batch, head and query) */
typedef struct sfm_dense_bwd_desc {
    sfm_dense_desc fwd;
    int64_t dq_stride[3];
    int64_t dkv_stride[3];
    int64_t kv_grad_start;
    int64_t kv_grad_end;
} sfm_dense_bwd_desc;

int sfm_dense_bwd_workspace_bytes(const sfm_dense_bwd_desc* desc, size_t* bytes);
int sfm_dense_bwd(const sfm_dense_bwd_desc* desc, const void* q, const void* k, const void* v, const void* out, const float* lse,
                  const void* dout, float* dq, void* dk, void* dv, void* workspace, size_t workspace_bytes, void* stream);

typedef struct sfm_prologue_desc {
    int32_t dtype;            /* SFM_BF16 | SFM_F16 | SFM_F32 */
    int32_t B, S, H, D;       /* S new tokens (= F*h*w), model dim C = H*D */
    int32_t F, h, w;          /* grid of the new tokens */
    int32_t start_frame;      /* RoPE frame offset (causal_model.py:900-905) */
    float   eps;              /* RMSNorm epsilon (causal_model.py:773-774) */
    sfm_tiling tiling;        /* order in which K/V rows are laid into the cache */
    int64_t x_stride[2];      /* batch, token strides of xq, xk, xv ([B,S,C], C contiguous) */
    int64_t q_stride[3];      /* q_out [B,S,H,D] */
    int64_t cache_stride[3];  /* k_cache, v_cache [B,cache_tokens,H,D] */
    int64_t cache_tokens;
    int64_t start_idx;        /* K/V rows are written to cache[:, start_idx : start_idx+S] */
} sfm_prologue_desc;

/* Fused q/k prologue: RMSNorm over the full model dim (model.py:462-478) with weights wq/wk [C],
 * 3-D RoPE on interleaved pairs (causal_model.py:687-715; angles from the float64 table
 * `rope_cos_sin` [max_pos, D/2, 2] built as model.py:421-428 + causal_model.py:1350-1357),
 * q -> q_out (token order), roped k and v -> cache rows in Monarch block order
 * (monarch_attn.py:1784-1785, 1230-1231; causal_model.py:961-962 when the tiling is the identity). */
int sfm_qk_prologue(const sfm_prologue_desc* desc, const void* xq, const void* xk, const void* xv,
                    const void* wq, const void* wk, const double* rope_cos_sin, int32_t rope_max_pos,
                    void* q_out, void* k_cache, void* v_cache, void* stream);

/* Block-level element-wise fusions around the attention op (rows = B*L token rows of C channels, C <= 8192,
 * row strides in elements).  They keep the rounding points of the reference's eager ops.
 *
 * sfm_ln_modulate: y = LayerNorm(x) * (1 + scale[f]) + shift[f] with per-frame modulation rows
 *   scale/shift + (row / rows_per_frame) * mod_stride (wan/modules/causal_model.py:1179-1183, 1198-1201), or,
 *   when weight/bias are given (scale = shift = NULL), the affine LayerNorm of norm3 (causal_model.py:1194).
 * sfm_gate_residual: x += y * gate[f] in place (causal_model.py:1189, 1203-1204); gate = NULL gives x += y.
 * sfm_rms_norm: WanRMSNorm (wan/modules/model.py:462-478).
 * sfm_gate_residual_ln: sfm_gate_residual followed by sfm_ln_modulate of the updated rows in one pass (the residual
 *   update and the next sub-layer's norm, causal_model.py:1189+1194, 1196+1198): x is updated in place, out gets the
 *   normalised rows. */
int sfm_ln_modulate(int32_t dtype, int64_t rows, int32_t C, float eps, const void* x, int64_t x_stride, void* y,
                    int64_t y_stride, const void* scale, const void* shift, int64_t mod_stride, int32_t rows_per_frame,
                    const void* weight, const void* bias, void* stream);
int sfm_gate_residual(int32_t dtype, int64_t rows, int32_t C, void* x, int64_t x_stride, const void* y, int64_t y_stride,
                      const void* gate, int64_t mod_stride, int32_t rows_per_frame, void* stream);
int sfm_rms_norm(int32_t dtype, int64_t rows, int32_t C, float eps, const void* x, int64_t x_stride, void* y,
                 int64_t y_stride, const void* weight, void* stream);
int sfm_gate_residual_ln(int32_t dtype, int64_t rows, int32_t C, float eps, void* x, int64_t x_stride, const void* y,
                         int64_t y_stride, const void* gate, int64_t gate_stride, int32_t gate_rows_per_frame, void* out,
                         int64_t out_stride, const void* scale, const void* shift, int64_t mod_stride, int32_t rows_per_frame,
                         const void* weight, const void* bias, void* stream);

/* The block's linear layers with their element-wise tails in the matrix product's epilogue (16-bit tensors, fp32
 * accumulation on MFMA).  x: [M, K] activations, rows x_stride elements apart; w: [N, K] contiguous (nn.Linear.weight);
 * bias: [N] or NULL; out: [M, N], rows out_stride apart.
 *   SFM_EPI_NONE           out = x w^T + bias                        nn.Linear (wan/modules/model.py:592-596, 632-650)
 *   SFM_EPI_GELU_TANH      out = gelu_tanh(x w^T + bias)             the FFN's first half (model.py:648-650)
 *   SFM_EPI_GATE_RESIDUAL  out = res + (x w^T + bias) * gate[m / rows_per_frame]   the output projections with the adaLN
 *                          gates and the residual update (wan/modules/causal_model.py:1189, 1196, 1203-1204);
 *                          gate = NULL: out = res + (x w^T + bias); res ([M, N], rows res_stride apart) may be `out`.
 * Rounding points are the eager chain's: the product plus bias is rounded to the tensor dtype, the GELU of that value
 * is rounded, the gated product is rounded, the residual sum is rounded.  K a multiple of 64, N a multiple of 8, all
 * strides multiples of 8 elements, pointers 16-byte aligned, operands below 4 GiB each.  `out` must not overlap x or
 * w (SFM_ERR_RANGE): workgroups read whole rows of both while others already store. */
#define SFM_EPI_NONE          0
#define SFM_EPI_GELU_TANH     1
#define SFM_EPI_GATE_RESIDUAL 2
typedef struct sfm_linear_desc {
    int32_t dtype;            /* SFM_BF16 | SFM_F16 */
    int32_t epilogue;         /* SFM_EPI_* */
    int64_t M;
    int32_t N, K;
    int64_t x_stride, out_stride, res_stride, gate_stride;   /* elements */
    int32_t rows_per_frame;   /* rows sharing one gate row (GATE_RESIDUAL with a gate) */
    int32_t tile_rows;        /* output rows per workgroup: 0 = chosen from the shape, 128 or 256 = forced (measurements) */
} sfm_linear_desc;
int sfm_linear(const sfm_linear_desc* desc, const void* x, const void* w, const void* bias, const void* res, const void* gate,
               void* out, void* stream);

typedef struct sfm_conv_desc {
    int32_t dtype;            /* SFM_BF16 | SFM_F16 */
    int32_t T, H, W;          /* output frames, rows, columns */
    int32_t Cin, Cout;        /* Cin a multiple of 32 */
    int32_t Cout_pad;         /* rows per tap in `wt`: a multiple of 32, >= Cout (rows past Cout are never stored) */
    int32_t kt, kh, kw;       /* kt in 1..3; kh = kw in {1, 3} */
    int32_t up2x;             /* 1: the input is at half resolution and is upsampled x2 (nearest) on the fly */
    int32_t reserved;
    int64_t x_stride[3];      /* frame, row, column strides of the padded input, in elements (channels contiguous) */
    int64_t y_stride[3];      /* same for the output */
} sfm_conv_desc;

/* Channels-last convolution of the streaming VAE decoder: the nn.Conv3d / nn.Conv2d calls of wan/modules/vae.py
 * (CausalConv3d :17-36; the 3x3 conv after the nearest x2 upsampling :76-79; residual, head and shortcut
 * convolutions :186-220, :423-472).  `x` is the input with its kt - 1 history (or zero) frames in front and,
 * for a 3x3 spatial kernel, a one-pixel zero border, i.e. [T + kt - 1][H + kh - 1][W + kw - 1][Cin] (with up2x:
 * [T + kt - 1][H/2 + 2][W/2 + 2][Cin]); `wt` is the weight as [kt][kh][kw][Cout_pad][Cin]; `bias` (fp32, [Cout])
 * may be NULL; `res` (a residual input added to the result, the `x + h` of vae.py:220; same layout and strides as
 * `y`) may be NULL; `y` is [T][H][W][Cout].  One call's input must stay below 4 GiB.  A 3x3 spatial kernel on a contiguous padded
 * input (x_stride = {(H + 2)(W + 2) Cin, (W + 2) Cin, Cin}) with Cout_pad a multiple of 96 or equal to 32 runs the kernel
 * that stages one run of input rows for the three taps of a kernel row; any other strides run the general kernel
 * (same result up to the order of the fp32 sums). */
int sfm_conv3d_cl(const sfm_conv_desc* desc, const void* x, const void* wt, const float* bias, const void* res, void* y,
                  void* stream);

/* RMS norm over the channels with optional SiLU for channels-last activations [T][H][W][C]: y = x / max(|x|_2, 1e-12)
 * * sqrt(C) * gamma, then y * sigmoid(y) if act != 0 (wan/modules/vae.py:39-54 and the nn.SiLU that follows it in
 * :192-197, :418-420).  fp32 inside, one rounding.  Strides in elements (frame, row, column); x and y may be views
 * into larger buffers (e.g. the interior of the next convolution's padded input).  gamma has the dtype of x. */
int sfm_vae_norm_act(int32_t dtype, int32_t T, int32_t H, int32_t W, int32_t C, int32_t act, const void* x,
                     const int64_t x_stride[3], const void* gamma, void* y, const int64_t y_stride[3], void* stream);

/* Measurement aid with no counterpart in the reference: runs a stream of independent 32x32x16 bf16 MFMAs (two waves
 * per SIMD, `iters` x 16 per wave) on `stream`, waits for it and returns the sustained rate in TFLOP/s.  bench.py
 * reports the dense kernel against it beside the nominal peak. */
int sfm_probe_mfma_bf16(int32_t iters, void* stream, float* tflops);

/* Measurement aid with no counterpart in the reference: the memory traffic of the Monarch forward's step 1 and nothing
 * else.  `tiles` work items in equal contiguous shares over two workgroups per compute unit; item t reads 2 x rows_in
 * rows of row_bytes (contiguous) and writes rows_out rows of row_bytes to each of two matrices, row r of item t at row
 * index r * tiles + t (the scatter of step 1's scratch), with non-temporal stores if `nontemporal` != 0.  The caller
 * supplies `workspace` (device memory, 16-byte aligned, >= tiles * (2 rows_in + 2 rows_out) * row_bytes bytes; its
 * contents are read and overwritten).  A workspace with room for several copies of the input (up to 8 are used:
 * tiles * (2 rows_in * copies + 2 rows_out) * row_bytes bytes) makes consecutive passes read different copies; with a
 * single copy below the size of the memory-side cache (256 MB) the reads are served from that cache and cost nothing,
 * which the operator's own reads in a model are not.  Runs on `stream`, waits, and returns the mean duration of one
 * pass in microseconds: the floor for this traffic on this machine, which bench.py reports beside step 1's duration. */
int sfm_probe_tile_traffic(int32_t tiles, int32_t rows_in, int32_t rows_out, int32_t row_bytes, int32_t nontemporal,
                           void* workspace, size_t workspace_bytes, void* stream, float* us);

/* Measurement aid with no counterpart in the reference: the memory traffic of the Monarch forward's step 2 and nothing
 * else.  `waves` waves (four per workgroup), each reading two contiguous blocks of kb_per_block KB of `workspace`
 * (device memory, 16-byte aligned, >= 2 * waves * kb_per_block KB; only read), 16 bytes per lane, 8 KB of each block
 * per batch and the next batch requested as soon as the current one is consumed.  Runs on `stream`, waits, and returns
 * the mean duration of one pass in microseconds, which bench.py reports beside step 2's own duration. */
int sfm_probe_row_stream(int32_t waves, int32_t kb_per_block, const void* workspace, size_t workspace_bytes, void* stream,
                         float* us);

/* Measurement aid with no counterpart in the reference: the rate at which the compute units can be fed from L2.
 * `workgroups` workgroups each stream `stages` (4..64) stages of 32 KB of one shared 2 MB window of `workspace`
 * (device memory, 256-byte aligned, >= 2 MiB + 256 bytes; read, plus 4 bytes written behind the window) into LDS.
 * Runs on `stream`, waits, and returns the mean duration of one launch in microseconds: workgroups * stages * 32 KiB
 * per that time is the aggregate L2 -> CU read rate (about 16 TB/s with one workgroup per compute unit on MI355X,
 * twice that per compute unit when only an eighth of them ask). */
int sfm_probe_l2_read(int32_t workgroups, int32_t stages, void* workspace, size_t workspace_bytes, void* stream, float* us);

/* Implementation switches for measurements and tests; no counterpart in the reference.  The environment is read
 * ONCE, when the library is loaded: a variable of the same name as a bit below that is set to anything but "0" turns
 * the bit on (SFM_BWD_SIMT=1 ...), SFM_NO_ROCBLAS makes the library behave as where rocBLAS is absent, and SFM_S1_WGS=n
 * overrides the step-1 workgroup count.  No entry point reads the environment afterwards; sfm_set_switches replaces the
 * mask for the whole process (returns the previous one; unknown bits are rejected with (unsigned)-1 and leave it
 * unchanged), which is how the tests reach every path from one process.  Workspace queries follow the mask: do not
 * change it between a workspace query and the call that uses that size. */
#define SFM_SW_BWD_SIMT        0x01u  /* backward on the fp32 SIMT kernels */
#define SFM_SW_BWD_LEFT_GEMM   0x02u  /* backward parts on the batched library GEMMs instead of their fused kernels: */
#define SFM_SW_BWD_FWD_GEMM    0x04u
#define SFM_SW_BWD_DQA_GEMM    0x08u
#define SFM_SW_BWD_RIGHT_GEMM  0x10u
#define SFM_SW_BWD_DQK_GEMM    0x20u
#define SFM_SW_ITER_SIMT       0x40u  /* num_iters > 1 on the fp32 SIMT kernels also where the MFMA kernels apply */
#define SFM_SW_ALL             0x7fu
unsigned sfm_set_switches(unsigned mask);
unsigned sfm_get_switches(void);

/* Thread-local description of the last error returned on this thread ("" if none). */
const char* sfm_last_error(void);

/* ABI version (bumped on any signature change). */
int sfm_version(void);

#ifdef __cplusplus
}
#endif
#endif /* SFM_ATTN_H */
