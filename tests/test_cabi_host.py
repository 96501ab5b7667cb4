"""CPU-only checks of the C-ABI boundary: the library loads, exports every symbol the header
declares, and rejects bad arguments with error codes before touching any device."""
import ctypes as C
import os
import re

import pytest

from self_forcing_amd import lib as L

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "sfm_attn.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(sfm_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = L.load()
    names = _declared_symbols()
    assert len(names) >= 9 and set(names) == set(L.SYMBOLS)
    for n in names:
        assert hasattr(lib, n), n
    assert lib.sfm_version() == 9


def test_switches_are_a_process_wide_mask_set_through_the_abi():
    """The implementation switches: header constants == binding constants, set returns the previous mask, unknown bits
    are refused and leave the mask alone, and the workspace query of the backward follows the mask."""
    lib = L.load()
    text = open(os.path.join(ROOT, "include", "sfm_attn.h")).read()
    for i, name in enumerate(("BWD_SIMT", "BWD_LEFT_GEMM", "BWD_FWD_GEMM", "BWD_DQA_GEMM", "BWD_RIGHT_GEMM", "BWD_DQK_GEMM", "ITER_SIMT")):
        assert re.search(rf"#define\s+SFM_SW_{name}\s+0x{1 << i:02x}u", text), name
        assert getattr(L, "SW_" + name) == 1 << i
    old = lib.sfm_get_switches()
    try:
        assert lib.sfm_set_switches(L.SW_BWD_SIMT) == old
        assert lib.sfm_get_switches() == L.SW_BWD_SIMT and lib.sfm_monarch_bwd_uses_gemm() == 0
        assert lib.sfm_set_switches(0x80) == 0xFFFFFFFF and b"unknown switch" in lib.sfm_last_error()
        assert lib.sfm_get_switches() == L.SW_BWD_SIMT
    finally:
        lib.sfm_set_switches(old)
    assert lib.sfm_get_switches() == old


def test_environment_is_read_once_at_load():
    """A process started with SFM_BWD_SIMT=1 has the bit set from the start; changing the variable afterwards does
    nothing (no entry point reads the environment)."""
    import subprocess
    import sys
    code = ("import os, sys; sys.path.insert(0, %r); import importlib; L = importlib.import_module('self_forcing_amd').lib; "
            "lib = L.load(); a = lib.sfm_get_switches(); os.environ['SFM_BWD_SIMT'] = '0'; os.environ['SFM_BWD_DQK_GEMM'] = '1'; "
            "print('MASK', a, lib.sfm_get_switches(), lib.sfm_monarch_bwd_uses_gemm())") % ROOT
    env = dict(os.environ, SFM_BWD_SIMT="1")
    r = subprocess.run([sys.executable, "-c", code], env=env, capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-1500:]
    assert [ln for ln in r.stdout.splitlines() if ln.startswith("MASK")][0] == "MASK 1 1 0"


def test_struct_sizes_match_header_layout():
    # int32 x 6, tiling (5 x int32), 2 x int32, float, pad to 8, 12 x int64
    assert C.sizeof(L.Tiling) == 20
    assert C.sizeof(L.MonarchDesc) == 64 + 12 * 8
    assert C.sizeof(L.DenseDesc) == 32 + 12 * 8
    assert C.sizeof(L.PrologueDesc) == 64 + 8 * 8 + 16


def _desc(**kw):
    d = L.MonarchDesc()
    d.dtype, d.B, d.H, d.D = L.SFM_BF16, 1, 2, 128
    d.q_tokens, d.kv_tokens = 3 * 30 * 52, 21 * 30 * 52
    d.tiling = L.Tiling(1, 1, 1, 30, 52)
    d.kv_block_order, d.causal_block_frames, d.sm_scale, d.num_iters = 1, 0, 128 ** -0.5, 1
    for name in ("q_stride", "k_stride", "v_stride", "o_stride"):
        toks = d.kv_tokens if name[0] in "kv" else d.q_tokens
        setattr(d, name, (C.c_int64 * 3)(toks * 256, 256, 128))
    for k, v in kw.items():
        setattr(d, k, v)
    return d


def _ws(d, hpp=0):
    n = C.c_size_t(0)
    rc = L.load().sfm_monarch_workspace_bytes(C.byref(d), hpp, C.byref(n))
    return rc, n.value


def _fused_bytes(na, nf, b1, b2, units, cus=256):
    """Scratch of the one-kernel forward for a pass over `units` units: one output block [b1, 128] (16 bit) and 32
    floats per (unit, stream slot, column); streams = compute units // column groups of (up to) 12."""
    ncols, tpu = na * b2, nf * b1
    nj = min(12, ncols)
    ngroups = -(-ncols // nj)
    total = tpu * units
    ns = max(1, min(cus // ngroups, total))
    tps = -(-total // ns)
    nstreams = -(-total // tps)
    nslots = min(nstreams, (tpu - 1) // tps + 2)
    blocks = units * nslots * ncols
    r256 = lambda n: (n + 255) // 256 * 256
    return r256(r256(blocks * b1 * 256) + blocks * 32 * 4)


def test_workspace_bytes_accounting():
    # per unit: 2 matrices of a*b2*r_pad rows x D bf16 + one fp32 per row, r_pad = round_up(21*30, 32)
    rc, n1 = _ws(_desc(), 1)
    assert rc == 0
    rows = 3 * 52 * 640
    assert n1 == rows * 128 * 2 * 2 + rows * 4
    rc, n2 = _ws(_desc(), 2)
    assert rc == 0 and n2 == 2 * n1
    rc, nall = _ws(_desc(), 99)
    assert rc == 0 and nall == 2 * n1          # clamped to B*H units
    # the one-kernel forward (16-bit tensors, head_dim 128, b1 <= 32, b2 <= 64) and its per-pass scratch
    one = dict(flags=L.SFM_MONARCH_ONE_KERNEL)
    rc, f1 = _ws(_desc(**one), 1)
    assert rc == 0 and f1 == _fused_bytes(3, 21, 30, 52, 1)
    rc, f2 = _ws(_desc(**one), 0)
    assert rc == 0 and f2 == _fused_bytes(3, 21, 30, 52, 2)
    rc, f12 = _ws(_desc(H=12, **one), 0)
    assert rc == 0 and f12 == _fused_bytes(3, 21, 30, 52, 12) and f12 < 48 << 20
    assert _ws(_desc(flags=2), 1)[0] == -3
    # where the one-kernel forward does not apply the flag changes nothing
    assert _ws(_desc(tiling=L.Tiling(1, 1, 1, 60, 26), **one), 1) == _ws(_desc(tiling=L.Tiling(1, 1, 1, 60, 26)), 1)
    # fp32 tensors take the generic path, which keeps its scratch rows in float
    rc, nf32 = _ws(_desc(dtype=L.SFM_F32), 1)
    assert rc == 0 and nf32 == rows * 128 * 4 * 2 + rows * 4
    # iterated refinement on the MFMA kernels: 16-bit Kbar, Y and representatives, two fp32 scalars per row, and the left
    # factor's statistics (32 floats per (a, j) column); on the fp32 kernels (switch, or shapes the MFMA kernels do not
    # take: b1 = 180 below) everything in float and no statistics
    rc, nit = _ws(_desc(num_iters=3), 1)
    assert rc == 0 and nit == rows * 128 * 2 * 3 + rows * 4 * 2 + 3 * 52 * 32 * 4
    lib = L.load()
    old = lib.sfm_get_switches()
    try:
        lib.sfm_set_switches(L.SW_ITER_SIMT)
        rc, nsimt = _ws(_desc(num_iters=3), 1)
    finally:
        lib.sfm_set_switches(old)
    assert rc == 0 and nsimt == rows * 128 * 4 * 3 + rows * 4 * 2
    # three frames tied (b1 = 90): still the MFMA kernels, statistics rows padded to three 32-row query tiles
    rows3 = 1 * 52 * ((7 * 90 + 31) // 32 * 32)
    rc, ntied = _ws(_desc(num_iters=3, tiling=L.Tiling(3, 1, 1, 30, 52)), 1)
    assert rc == 0 and ntied == rows3 * 128 * 2 * 3 + rows3 * 4 * 2 + 52 * 96 * 4
    # b1 = 180 is beyond them: the fp32 kernels
    rows6 = 1 * 26 * ((7 * 180 + 31) // 32 * 32)
    rc, nwide = _ws(_desc(num_iters=3, tiling=L.Tiling(3, 1, 1, 60, 26)), 1)
    assert rc == 0 and nwide == (rows6 * 128 * 4 * 3 + rows6 * 4 * 2 + 255) // 256 * 256


@pytest.mark.parametrize("kw,code", [
    (dict(dtype=7), -2),
    (dict(num_iters=0), -3),
    (dict(num_iters=2, causal_block_frames=1, kv_block_order=0, q_tokens=21 * 30 * 52), -9),
    (dict(D=100), -3),
    (dict(q_tokens=1000), -3),
    (dict(kv_tokens=30 * 52 + 1), -3),
    (dict(tiling=L.Tiling(1, 4, 1, 30, 52)), -3),
    (dict(tiling=L.Tiling(0, 1, 1, 30, 52)), -3),
    (dict(sm_scale=0.0), -3),
    (dict(causal_block_frames=3), -3),                 # needs q_tokens == kv_tokens
    (dict(q_stride=(C.c_int64 * 3)(0, 256, 64)), -5),  # head stride < D
    (dict(v_stride=(C.c_int64 * 3)(1 << 20, 512, 128)), -5),   # differs from k_stride
    (dict(k_stride=(C.c_int64 * 3)(1 << 20, 257, 128), v_stride=(C.c_int64 * 3)(1 << 20, 257, 128)), -5),
])
def test_monarch_desc_validation(kw, code):
    rc, _ = _ws(_desc(**kw))
    assert rc == code
    assert L.load().sfm_last_error() != b""


def test_monarch_fwd_pointer_and_workspace_checks():
    lib = L.load()
    d = _desc()
    _, need = _ws(d, 1)
    fake = 0x10000
    assert lib.sfm_monarch_fwd(C.byref(d), None, fake, fake, fake, fake, need, None) == -1
    assert lib.sfm_monarch_fwd(C.byref(d), fake + 2, fake, fake, fake, fake, need, None) == -7
    assert lib.sfm_monarch_fwd(C.byref(d), fake, fake, fake, fake, None, need, None) == -6
    assert lib.sfm_monarch_fwd(C.byref(d), fake, fake, fake, fake, fake + 16, need, None) == -6
    assert lib.sfm_monarch_fwd(C.byref(d), fake, fake, fake, fake, fake, need - 1, None) == -6
    assert lib.sfm_monarch_fwd(None, fake, fake, fake, fake, fake, need, None) == -1


def test_row_statistics_size_and_argument_checks():
    """sfm_monarch_stats_bytes: one float per (unit, a, j) and block row, rows padded to 32; 0 where the forward that
    would run keeps none.  The entry points that write / read them refuse NULL and misaligned pointers first."""
    lib = L.load()
    n = C.c_size_t(1)
    assert lib.sfm_monarch_stats_bytes(C.byref(_desc()), C.byref(n)) == 0 and n.value == 2 * 3 * 52 * 32 * 4
    assert lib.sfm_monarch_stats_bytes(C.byref(_desc(dtype=L.SFM_F32)), C.byref(n)) == 0 and n.value == 0
    assert lib.sfm_monarch_stats_bytes(C.byref(_desc(num_iters=2)), C.byref(n)) == 0 and n.value == 0
    assert lib.sfm_monarch_stats_bytes(C.byref(_desc()), None) == -1
    d = _desc()
    _, need = _ws(d, 1)
    fake = 0x10000
    assert lib.sfm_monarch_fwd_stats(C.byref(d), fake, fake, fake, fake, None, fake, need, None) == -1
    assert lib.sfm_monarch_fwd_stats(C.byref(_desc(dtype=L.SFM_F32)), fake, fake, fake, fake, fake, fake, 1 << 40, None) == -9
    bd = L.MonarchBwdDesc()
    bd.fwd = d
    bd.dq_stride = (C.c_int64 * 3)(d.q_tokens * 256, 256, 128)
    bd.dkv_stride = (C.c_int64 * 3)(d.kv_tokens * 256, 256, 128)
    bd.kv_grad_frame_start, bd.kv_grad_frame_end = 0, 21
    args = [fake] * 4
    assert lib.sfm_monarch_bwd_saved(C.byref(bd), fake, fake, fake, None, fake, *args, fake, 1 << 40, None) == -1
    assert lib.sfm_monarch_bwd_saved(C.byref(bd), fake, fake, fake, fake, None, *args, fake, 1 << 40, None) == -1
    assert lib.sfm_monarch_bwd_saved(C.byref(bd), fake, fake, fake, fake + 2, fake, *args, fake, 1 << 40, None) == -7
    assert lib.sfm_monarch_bwd_saved(C.byref(bd), fake, fake, fake, fake, fake + 2, *args, fake, 1 << 40, None) == -7
    assert lib.sfm_monarch_bwd_saved(C.byref(bd), fake, fake, fake, fake, fake, None, fake, fake, fake, fake, 1 << 40, None) == -1


def test_dense_backward_argument_checks():
    lib = L.load()
    bd = L.DenseBwdDesc()
    d = bd.fwd
    d.dtype, d.B, d.H, d.D, d.q_tokens, d.kv_tokens, d.sm_scale = L.SFM_BF16, 1, 2, 128, 100, 300, 128 ** -0.5
    for name, toks in (("q_stride", 100), ("k_stride", 300), ("v_stride", 300), ("o_stride", 100)):
        setattr(d, name, (C.c_int64 * 3)(toks * 256, 256, 128))
    bd.dq_stride = (C.c_int64 * 3)(100 * 256, 256, 128)
    bd.dkv_stride = (C.c_int64 * 3)(300 * 256, 256, 128)
    bd.kv_grad_start, bd.kv_grad_end = 0, 300
    n = C.c_size_t(0)
    assert lib.sfm_dense_bwd_workspace_bytes(C.byref(bd), C.byref(n)) == 0 and n.value == 1792      # 2 x 2 x 100 floats, rounded to 256
    fake = 0x10000
    ok = [fake] * 9
    call = lambda args, ws=fake, nb=1792: lib.sfm_dense_bwd(C.byref(bd), *args, ws, nb, None)
    for i in range(9):
        args = list(ok)
        args[i] = None
        assert call(args) == -1
    args = list(ok)
    args[0] = fake + 2
    assert call(args) == -7
    assert call(ok, None) == -6 and call(ok, fake, 1599) == -6 and call(ok, fake + 16) == -6
    bd.kv_grad_end = 301
    assert call(ok) == -4
    bd.kv_grad_start, bd.kv_grad_end = 200, 100
    assert call(ok) == -4
    bd.kv_grad_start, bd.kv_grad_end = 0, 300
    d.D = 32
    for name, toks in (("q_stride", 100), ("k_stride", 300), ("v_stride", 300), ("o_stride", 100)):
        setattr(d, name, (C.c_int64 * 3)(toks * 64, 64, 32))
    assert call(ok) == -9                              # head_dim 32 has a forward only
    d.D, d.dtype = 128, L.SFM_F32
    for name, toks in (("q_stride", 100), ("k_stride", 300), ("v_stride", 300), ("o_stride", 100)):
        setattr(d, name, (C.c_int64 * 3)(toks * 256, 256, 128))
    assert call(ok) == -9


def test_kv_cache_op_range_checks_happen_before_any_write():
    lib = L.load()
    d = _desc()
    _, need = _ws(d, 1)
    fake = 0x10000
    ns = (C.c_int64 * 3)(4680 * 256, 256, 128)
    blk = 30 * 52
    call = lambda s, e, **kw: lib.sfm_monarch_attn_with_kv_cache(
        C.byref(_desc(**kw)), fake, fake, fake, fake, fake, ns, s, e, fake, fake, need, None)
    assert call(18 * blk + 1, 21 * blk) == -4          # not aligned to a block-frame
    assert call(18 * blk, 22 * blk) == -4              # past the end of the view
    assert call(-blk, 2 * blk) == -4
    assert call(3 * blk, 2 * blk) == -4
    assert call(18 * blk, 21 * blk, kv_block_order=0) == -9


def test_dense_and_prologue_validation():
    lib = L.load()
    fake = 0x10000
    d = L.DenseDesc()
    d.dtype, d.B, d.H, d.D, d.q_tokens, d.kv_tokens, d.sm_scale = L.SFM_BF16, 1, 2, 128, 10, 20, 0.1
    for name in ("q_stride", "k_stride", "v_stride", "o_stride"):
        setattr(d, name, (C.c_int64 * 3)(20 * 256, 256, 128))
    assert lib.sfm_dense_fwd(C.byref(d), fake, fake, None, fake, None, None) == -1
    d.D = 12
    assert lib.sfm_dense_fwd(C.byref(d), fake, fake, fake, fake, None, None) == -3
    d.D = 128
    ns = (C.c_int64 * 3)(5 * 256, 256, 128)
    assert lib.sfm_full_attention_with_kv_cache(C.byref(d), fake, fake, fake, fake, fake, ns, 18, 23, fake, None, None) == -4

    p = L.PrologueDesc()
    p.dtype, p.B, p.S, p.H, p.D = L.SFM_BF16, 1, 24, 2, 128
    p.F, p.h, p.w, p.start_frame, p.eps = 1, 4, 6, 0, 1e-6
    p.tiling = L.Tiling(1, 1, 1, 4, 6)
    p.x_stride = (C.c_int64 * 2)(24 * 256, 256)
    p.q_stride = (C.c_int64 * 3)(24 * 256, 256, 128)
    p.cache_stride = (C.c_int64 * 3)(48 * 256, 256, 128)
    p.cache_tokens, p.start_idx = 48, 24
    args = [fake] * 6
    assert lib.sfm_qk_prologue(C.byref(p), *args, 1024, fake, fake, None, None) == -1
    p.start_idx = 30
    assert lib.sfm_qk_prologue(C.byref(p), *args, 1024, fake, fake, fake, None) == -4
    p.start_idx, p.start_frame = 24, 1024
    assert lib.sfm_qk_prologue(C.byref(p), *args, 1024, fake, fake, fake, None) == -4
    p.start_frame, p.S = 0, 25
    assert lib.sfm_qk_prologue(C.byref(p), *args, 1024, fake, fake, fake, None) == -3


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    monkeypatch.setattr(L, "_lib", None)
    monkeypatch.setattr(L, "LIB_PATH", str(tmp_path / "nope.so"))
    with pytest.raises(RuntimeError, match="no fallback"):
        L.load()


def test_mfma_probe_rejects_bad_arguments_before_any_launch():
    lib = L.load()
    out = C.c_float(0)
    assert lib.sfm_probe_mfma_bf16(0, None, C.byref(out)) == -4
    assert lib.sfm_probe_mfma_bf16(100, None, None) == -4
    assert b"iters" in lib.sfm_last_error()


def test_traffic_probe_rejects_bad_arguments_before_any_launch():
    lib = L.load()
    out = C.c_float(0)
    fake = C.c_void_p(4096)                                   # never dereferenced: every call below fails the checks
    assert lib.sfm_probe_tile_traffic(0, 52, 156, 256, 1, fake, 1 << 30, None, C.byref(out)) == -4
    assert lib.sfm_probe_tile_traffic(10, 52, 156, 250, 1, fake, 1 << 30, None, C.byref(out)) == -4
    assert lib.sfm_probe_tile_traffic(10, 52, 156, 256, 1, None, 1 << 30, None, C.byref(out)) == -4
    assert lib.sfm_probe_tile_traffic(10, 52, 156, 256, 1, fake, 1 << 30, None, None) == -4
    need = 10 * (2 * 52 + 2 * 156) * 256
    assert lib.sfm_probe_tile_traffic(10, 52, 156, 256, 1, fake, need - 1, None, C.byref(out)) == -6
    assert str(need).encode() in lib.sfm_last_error()
    assert lib.sfm_probe_tile_traffic(10, 52, 156, 256, 1, C.c_void_p(4100), need, None, C.byref(out)) == -6


def test_row_stream_probe_rejects_bad_arguments_before_any_launch():
    lib = L.load()
    out = C.c_float(0)
    fake = C.c_void_p(4096)                                   # never dereferenced: every call below fails the checks
    assert lib.sfm_probe_row_stream(0, 8, fake, 1 << 30, None, C.byref(out)) == -4
    assert lib.sfm_probe_row_stream(4, 0, fake, 1 << 30, None, C.byref(out)) == -4
    assert lib.sfm_probe_row_stream(4, 8, None, 1 << 30, None, C.byref(out)) == -4
    assert lib.sfm_probe_row_stream(4, 8, fake, 1 << 30, None, None) == -4
    need = 2 * 4 * 8 * 1024
    assert lib.sfm_probe_row_stream(4, 8, fake, need - 1, None, C.byref(out)) == -6
    assert str(need).encode() in lib.sfm_last_error()
    assert lib.sfm_probe_row_stream(4, 8, C.c_void_p(4100), need, None, C.byref(out)) == -6


def test_static_scratch_entry_point_rejects_a_unit_beyond_its_size():
    """sfm_monarch_attn_with_kv_cache_static: one (batch, head) unit of a 63-frame cache at the 480p block shape needs
    155 MB of scratch, more than the library's 128 MiB array: SFM_ERR_WORKSPACE before any device is touched."""
    h, w, H, D = 30, 52, 1, 128
    d = _desc(H=H, kv_tokens=63 * h * w)
    d.k_stride = d.v_stride = (C.c_int64 * 3)(63 * h * w * H * D, H * D, D)
    d.q_stride = d.o_stride = (C.c_int64 * 3)(3 * h * w * H * D, H * D, D)
    rc, one = _ws(d, 1)
    assert rc == 0 and one > L.STATIC_SCRATCH_BYTES
    rc = L.load().sfm_monarch_attn_with_kv_cache_static(C.byref(d), 16, 16, 16, 16, 16, (C.c_int64 * 3)(3 * h * w * H * D, H * D, D),
                                                        60 * h * w, 63 * h * w, 16, None)
    assert rc == -6 and b"static scratch" in L.load().sfm_last_error()
    text = open(os.path.join(ROOT, "include", "sfm_attn.h")).read()
    assert re.search(r"#define\s+SFM_STATIC_SCRATCH_BYTES\s+\(128u\s*<<\s*20\)", text)


def test_fp32_kernel_limits_are_reported_before_anything_is_written():
    """Blocks 208 columns wide do not fit the LDS of the fp32 kernels that take them (b2 > 64 is beyond the MFMA kernels):
    every entry point, the workspace query included, answers SFM_ERR_UNSUPPORTED from the descriptor alone, i.e. before
    the KV-cache entry point could have written the new rows."""
    h, w = 30, 208
    for kw in (dict(), dict(num_iters=2), dict(dtype=L.SFM_F32)):
        d = _desc(q_tokens=3 * h * w, kv_tokens=6 * h * w, tiling=L.Tiling(1, 1, 1, h, w), **kw)
        d.q_stride = d.o_stride = (C.c_int64 * 3)(3 * h * w * 256, 256, 128)
        d.k_stride = d.v_stride = (C.c_int64 * 3)(6 * h * w * 256, 256, 128)
        assert _ws(d, 1)[0] == -9 and b"LDS budget" in L.load().sfm_last_error()
        rc = L.load().sfm_monarch_attn_with_kv_cache(C.byref(d), 16, 16, 16, 16, 16, (C.c_int64 * 3)(3 * h * w * 256, 256, 128),
                                                     3 * h * w, 6 * h * w, 16, 256, 1 << 40, None)
        assert rc == -9
    # 104 columns (the 720p grid halved) still run
    d = _desc(q_tokens=3 * 30 * 104, kv_tokens=6 * 30 * 104, tiling=L.Tiling(1, 1, 1, 30, 104))
    d.q_stride = d.o_stride = (C.c_int64 * 3)(3 * 30 * 104 * 256, 256, 128)
    d.k_stride = d.v_stride = (C.c_int64 * 3)(6 * 30 * 104 * 256, 256, 128)
    assert _ws(d, 1)[0] == 0


def test_linear_descriptor_errors():
    """sfm_linear validates before any launch: these calls return their error codes without a GPU."""
    lib = L.load()
    d = L.LinearDesc()
    d.dtype, d.epilogue, d.M, d.N, d.K = L.SFM_BF16, L.EPI_NONE, 256, 64, 128
    d.x_stride, d.out_stride = 128, 64
    call = lambda **kw: lib.sfm_linear(C.byref(d), kw.get("x", 0x10000), kw.get("w", 0x200000), None, kw.get("res"), None,
                                       kw.get("out", 0x400000), None)
    assert call(x=None) == -1
    d.dtype = L.SFM_F32
    assert call() == -2
    d.dtype, d.K = L.SFM_BF16, 96
    assert call() == -3 and b"multiple of 64" in lib.sfm_last_error()
    d.K, d.epilogue = 128, 7
    assert call() == -3
    d.epilogue = L.EPI_GATE_RESIDUAL
    assert call() == -1 and b"needs res" in lib.sfm_last_error()
    d.epilogue, d.x_stride = L.EPI_NONE, 100
    assert call() == -5
    d.x_stride = 128
    assert call(out=0x10000 + 256) == -4 and b"overlaps" in lib.sfm_last_error()  # out inside x
    assert call(out=0x200000 - 64) == -4                                          # out runs into w
    assert call(x=0x10008) == -7
