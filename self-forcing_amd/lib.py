"""ctypes binding of `libsfm_attn.so` (declared in include/sfm_attn.h).

The library is the only compute path: if it cannot be loaded this module raises, it never
falls back to another implementation.
"""
import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libsfm_attn.so")

SFM_BF16, SFM_F16, SFM_F32 = 0, 1, 2
SFM_MONARCH_ONE_KERNEL = 1
STATIC_SCRATCH_BYTES = 128 << 20      # SFM_STATIC_SCRATCH_BYTES of include/sfm_attn.h
# SFM_SW_* of include/sfm_attn.h: process-wide implementation switches (sfm_set_switches)
SW_BWD_SIMT, SW_BWD_LEFT_GEMM, SW_BWD_FWD_GEMM, SW_BWD_DQA_GEMM, SW_BWD_RIGHT_GEMM, SW_BWD_DQK_GEMM, SW_ITER_SIMT = (1 << i for i in range(7))

ERR_NAMES = {
    -1: "SFM_ERR_NULL", -2: "SFM_ERR_DTYPE", -3: "SFM_ERR_SHAPE", -4: "SFM_ERR_RANGE", -5: "SFM_ERR_STRIDE",
    -6: "SFM_ERR_WORKSPACE", -7: "SFM_ERR_ALIGN", -8: "SFM_ERR_HIP", -9: "SFM_ERR_UNSUPPORTED",
}

# every symbol include/sfm_attn.h declares
SYMBOLS = [
    "sfm_monarch_workspace_bytes", "sfm_monarch_fwd", "sfm_monarch_fwd_timed", "sfm_kv_cache_write", "sfm_monarch_attn_with_kv_cache",
    "sfm_monarch_attn_with_kv_cache_static",
    "sfm_dense_fwd", "sfm_full_attention_with_kv_cache", "sfm_qk_prologue", "sfm_ln_modulate", "sfm_gate_residual",
    "sfm_rms_norm", "sfm_gate_residual_ln", "sfm_linear", "sfm_monarch_bwd_workspace_bytes", "sfm_monarch_bwd", "sfm_monarch_bwd_uses_gemm",
    "sfm_monarch_stats_bytes", "sfm_monarch_fwd_stats", "sfm_monarch_bwd_saved", "sfm_dense_bwd_workspace_bytes", "sfm_dense_bwd", "sfm_probe_mfma_bf16", "sfm_probe_tile_traffic", "sfm_probe_row_stream", "sfm_probe_l2_read", "sfm_conv3d_cl", "sfm_vae_norm_act", "sfm_set_switches", "sfm_get_switches", "sfm_last_error", "sfm_version",
]


class ConvDesc(C.Structure):
    _fields_ = [("dtype", C.c_int32), ("T", C.c_int32), ("H", C.c_int32), ("W", C.c_int32), ("Cin", C.c_int32),
                ("Cout", C.c_int32), ("Cout_pad", C.c_int32), ("kt", C.c_int32), ("kh", C.c_int32), ("kw", C.c_int32),
                ("up2x", C.c_int32), ("reserved", C.c_int32), ("x_stride", C.c_int64 * 3), ("y_stride", C.c_int64 * 3)]


class LinearDesc(C.Structure):
    _fields_ = [("dtype", C.c_int32), ("epilogue", C.c_int32), ("M", C.c_int64), ("N", C.c_int32), ("K", C.c_int32),
                ("x_stride", C.c_int64), ("out_stride", C.c_int64), ("res_stride", C.c_int64), ("gate_stride", C.c_int64),
                ("rows_per_frame", C.c_int32), ("tile_rows", C.c_int32)]


EPI_NONE, EPI_GELU_TANH, EPI_GATE_RESIDUAL = 0, 1, 2


class Tiling(C.Structure):
    _fields_ = [("f_tied", C.c_int32), ("h_reduce", C.c_int32), ("w_reduce", C.c_int32), ("h", C.c_int32),
                ("w", C.c_int32)]


class MonarchDesc(C.Structure):
    _fields_ = [("dtype", C.c_int32), ("B", C.c_int32), ("H", C.c_int32), ("D", C.c_int32),
                ("q_tokens", C.c_int32), ("kv_tokens", C.c_int32), ("tiling", Tiling),
                ("kv_block_order", C.c_int32), ("causal_block_frames", C.c_int32), ("sm_scale", C.c_float),
                ("num_iters", C.c_int32), ("flags", C.c_int32),
                ("q_stride", C.c_int64 * 3), ("k_stride", C.c_int64 * 3), ("v_stride", C.c_int64 * 3),
                ("o_stride", C.c_int64 * 3)]


class MonarchBwdDesc(C.Structure):
    _fields_ = [("fwd", MonarchDesc), ("dq_stride", C.c_int64 * 3), ("dkv_stride", C.c_int64 * 3),
                ("kv_grad_frame_start", C.c_int32), ("kv_grad_frame_end", C.c_int32)]


class DenseDesc(C.Structure):
    _fields_ = [("dtype", C.c_int32), ("B", C.c_int32), ("H", C.c_int32), ("D", C.c_int32),
                ("q_tokens", C.c_int32), ("kv_tokens", C.c_int32), ("sm_scale", C.c_float),
                ("q_stride", C.c_int64 * 3), ("k_stride", C.c_int64 * 3), ("v_stride", C.c_int64 * 3),
                ("o_stride", C.c_int64 * 3)]


class DenseBwdDesc(C.Structure):
    _fields_ = [("fwd", DenseDesc), ("dq_stride", C.c_int64 * 3), ("dkv_stride", C.c_int64 * 3),
                ("kv_grad_start", C.c_int64), ("kv_grad_end", C.c_int64)]


class PrologueDesc(C.Structure):
    _fields_ = [("dtype", C.c_int32), ("B", C.c_int32), ("S", C.c_int32), ("H", C.c_int32), ("D", C.c_int32),
                ("F", C.c_int32), ("h", C.c_int32), ("w", C.c_int32), ("start_frame", C.c_int32),
                ("eps", C.c_float), ("tiling", Tiling), ("x_stride", C.c_int64 * 2), ("q_stride", C.c_int64 * 3),
                ("cache_stride", C.c_int64 * 3), ("cache_tokens", C.c_int64), ("start_idx", C.c_int64)]


_lib = None


def load():
    """Returns the loaded library; raises RuntimeError when it is missing or incomplete."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing: build it with `python self-forcing_amd/build.py` "
            "(there is no fallback implementation)")
    lib = C.CDLL(LIB_PATH)
    for name in SYMBOLS:
        if not hasattr(lib, name):
            raise RuntimeError(f"{LIB_PATH} does not export {name}")
    P, I64 = C.c_void_p, C.c_int64
    S3 = C.POINTER(C.c_int64)
    lib.sfm_version.restype = C.c_int
    lib.sfm_last_error.restype = C.c_char_p
    lib.sfm_monarch_workspace_bytes.argtypes = [C.POINTER(MonarchDesc), C.c_int32, C.POINTER(C.c_size_t)]
    lib.sfm_monarch_fwd.argtypes = [C.POINTER(MonarchDesc), P, P, P, P, P, C.c_size_t, P]
    lib.sfm_monarch_fwd_timed.argtypes = [C.POINTER(MonarchDesc), P, P, P, P, P, C.c_size_t, P,
                                          C.POINTER(C.c_float), C.POINTER(C.c_float)]
    lib.sfm_monarch_bwd_workspace_bytes.argtypes = [C.POINTER(MonarchBwdDesc), C.c_int32, C.POINTER(C.c_size_t)]
    lib.sfm_monarch_bwd.argtypes = [C.POINTER(MonarchBwdDesc), P, P, P, P, P, P, P, P, C.c_size_t, P]
    lib.sfm_dense_bwd_workspace_bytes.argtypes = [C.POINTER(DenseBwdDesc), C.POINTER(C.c_size_t)]
    lib.sfm_dense_bwd.argtypes = [C.POINTER(DenseBwdDesc), P, P, P, P, P, P, P, P, P, P, C.c_size_t, P]
    lib.sfm_monarch_stats_bytes.argtypes = [C.POINTER(MonarchDesc), C.POINTER(C.c_size_t)]
    lib.sfm_monarch_fwd_stats.argtypes = [C.POINTER(MonarchDesc), P, P, P, P, P, P, C.c_size_t, P]
    lib.sfm_monarch_bwd_saved.argtypes = [C.POINTER(MonarchBwdDesc), P, P, P, P, P, P, P, P, P, P, C.c_size_t, P]
    lib.sfm_kv_cache_write.argtypes = [C.c_int32, C.c_int32, C.c_int32, C.c_int32, C.POINTER(Tiling), P, P, S3, P, P,
                                       S3, I64, I64, I64, P]
    lib.sfm_monarch_attn_with_kv_cache.argtypes = [C.POINTER(MonarchDesc), P, P, P, P, P, S3, I64, I64, P, P,
                                                   C.c_size_t, P]
    lib.sfm_monarch_attn_with_kv_cache_static.argtypes = [C.POINTER(MonarchDesc), P, P, P, P, P, S3, I64, I64, P, P]
    lib.sfm_dense_fwd.argtypes = [C.POINTER(DenseDesc), P, P, P, P, P, P]
    lib.sfm_full_attention_with_kv_cache.argtypes = [C.POINTER(DenseDesc), P, P, P, P, P, S3, I64, I64, P, P, P]
    lib.sfm_qk_prologue.argtypes = [C.POINTER(PrologueDesc), P, P, P, P, P, P, C.c_int32, P, P, P, P]
    lib.sfm_ln_modulate.argtypes = [C.c_int32, I64, C.c_int32, C.c_float, P, I64, P, I64, P, P, I64, C.c_int32, P, P, P]
    lib.sfm_gate_residual.argtypes = [C.c_int32, I64, C.c_int32, P, I64, P, I64, P, I64, C.c_int32, P]
    lib.sfm_gate_residual_ln.argtypes = [C.c_int32, I64, C.c_int32, C.c_float, P, I64, P, I64, P, I64, C.c_int32, P, I64, P, P, I64,
                                         C.c_int32, P, P, P]
    lib.sfm_linear.argtypes = [C.POINTER(LinearDesc), P, P, P, P, P, P, P]
    lib.sfm_rms_norm.argtypes = [C.c_int32, I64, C.c_int32, C.c_float, P, I64, P, I64, P, P]
    lib.sfm_conv3d_cl.argtypes = [C.POINTER(ConvDesc), P, P, P, P, P, P]
    lib.sfm_vae_norm_act.argtypes = [C.c_int32] * 6 + [P, S3, P, P, S3, P]
    lib.sfm_probe_mfma_bf16.argtypes = [C.c_int32, P, C.POINTER(C.c_float)]
    lib.sfm_probe_tile_traffic.argtypes = [C.c_int32, C.c_int32, C.c_int32, C.c_int32, C.c_int32, P, C.c_size_t, P, C.POINTER(C.c_float)]
    lib.sfm_probe_row_stream.argtypes = [C.c_int32, C.c_int32, P, C.c_size_t, P, C.POINTER(C.c_float)]
    lib.sfm_probe_l2_read.argtypes = [C.c_int32, C.c_int32, P, C.c_size_t, P, C.POINTER(C.c_float)]
    lib.sfm_set_switches.argtypes = [C.c_uint]
    lib.sfm_set_switches.restype = lib.sfm_get_switches.restype = C.c_uint
    for name in SYMBOLS:
        if name not in ("sfm_version", "sfm_last_error", "sfm_set_switches", "sfm_get_switches"):
            getattr(lib, name).restype = C.c_int
    _lib = lib
    return lib


class SfmError(ValueError):
    """An entry point returned a negative status.  `.code` holds it."""

    def __init__(self, code, message):
        super().__init__(f"{ERR_NAMES.get(code, code)}: {message}")
        self.code = code


def check(rc):
    if rc != 0:
        raise SfmError(rc, load().sfm_last_error().decode())


def strides3(t):
    """(batch, token, head) element strides of a [B, S, H, D] tensor as a C array."""
    return (C.c_int64 * 3)(t.stride(0), t.stride(1), t.stride(2))
