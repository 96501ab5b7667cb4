#!/usr/bin/env python3
"""Benchmark of the causal Wan-1.3B generator and its attention hot path on one MI355X.

Headline (one step = one 21-latent-frame video): latent frames/s of the random-init causal Wan-1.3B DiT at
480x832 (latents 21x16x60x104), 7 chunks of 3 frames x (4 denoising passes + 1 cache-refresh pass), Monarch
framewise attention with per-layer KV cache, bf16, synthetic text context — BASELINE.json configs[2].
Alongside, the attention op alone at the chunk shape (configs[1]): ms/call, per-kernel HIP-event durations,
roofline of the dominant hot-path kernel, dense fallback, and a CPU baseline.  Prints ONE JSON line.
"""
import argparse
import gc
import ctypes as C
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

# MI355X published peaks
HBM_PEAK_GBS = 8000.0
MFMA_BF16_PEAK_TFLOPS = 2500.0

B, H, D, A, F, B1, B2 = 1, 12, 128, 3, 21, 30, 52
SQ, SKV = A * B1 * B2, F * B1 * B2
MONARCH_FLOPS = B * H * (6 * A * F * B1 * B2 * B2 * D + 4 * A * B2 * F * B1 * B1 * D)
DENSE_FLOPS = 4 * B * H * SQ * SKV * D
# algorithmic bytes of the two kernels (bf16 tensors, fp32 entropy term)
ROWS = B * H * A * B2 * F * B1                        # rows of Kbar / Y
STEP1_BYTES = (2 * SKV + SQ) * H * D * 2 + 2 * ROWS * D * 2 + ROWS * 4      # read K,V,Q; write Kbar,Y,cl
STEP2_BYTES = 2 * ROWS * D * 2 + ROWS * 4 + 2 * SQ * H * D * 2              # read Kbar,Y,cl,Q; write O

LAYERS, CHUNKS, PASSES = 30, 7, 5

# the rollouts --config selects: (BASELINE.json entry, model size, attention flags, description)
ROLLOUTS = {
    "c3": ("configs[2]", "1.3B", dict(use_framewise=True),
           "random-init causal Wan-1.3B (30 layers, dim 1536, 12x128 heads, FFN 8960), Monarch framewise attention"),
    "c4": ("configs[3]", "1.3B", dict(use_framewise=True, h_reduce=2, use_dense_init=True),
           "random-init causal Wan-1.3B, Monarch framewise attention on the reduce2xh tiling (h_reduce=2: a=6, f=42, "
           "b1=15, b2=52) with dense attention on the first chunk (USE_DENSE_INIT)"),
    "c5": ("configs[4]", "14B", dict(use_framewise=True),
           "random-init causal Wan-14B (40 layers, dim 5120, 40x128 heads, FFN 13824), Monarch framewise attention"),
    "dense": ("configs[2] with DISABLE_MONARCH_ATTN=1", "1.3B", dict(disable_monarch=True),
              "random-init causal Wan-1.3B, every layer on the dense chunk-vs-cache fallback"),
}


def measured_traffic():
    """HBM bytes per launch of the two forward kernels from rocprofv3 counters (FETCH_SIZE, WRITE_SIZE scaled by what
    the same counters read for a 1 GiB device copy), with the commit they were measured at: profiles/traffic.json,
    rewritten whenever the counters are collected again.  Missing file or kernel: traffic is reported as null."""
    try:
        with open(os.path.join(ROOT, "profiles", "traffic.json")) as f:
            return json.load(f)
    except (OSError, ValueError):
        return {"commit": None, "kernels": {}}


def write_traffic(fetch_csv, write_csv):
    """Turns the counter_collection CSVs of two rocprofv3 runs of `bench.py --op-only --skip-simt --skip-shapes --no-cpu-baseline --copy-probe`
    (`--pmc FETCH_SIZE`, then `--pmc WRITE_SIZE`; KiB per dispatch) into profiles/traffic.json.  Each counter is scaled
    by what it reads for the run's own 1 GiB device-to-device copies, whose traffic is known (1 GiB read, 1 GiB written)."""
    import collections
    import csv
    import subprocess

    def read(path, counter):
        """kernel name -> list of per-dispatch values"""
        per = collections.defaultdict(lambda: collections.defaultdict(float))
        with open(path) as f:
            for row in csv.DictReader(f):
                if row["Counter_Name"] == counter:
                    per[row["Kernel_Name"]][row["Dispatch_Id"]] += float(row["Counter_Value"])
        return {k: list(v.values()) for k, v in per.items()}

    fetch, write = read(fetch_csv, "FETCH_SIZE"), read(write_csv, "WRITE_SIZE")
    mean = lambda v: sum(v) / len(v)

    def pick(table, key):
        """(name, mean) of the instantiation of `key` with the most dispatches (the forward's own: the backward leg
        launches a statistics-keeping instantiation a few times)."""
        name = max((k for k in table if key + "<" in k), key=lambda k: len(table[k]))
        return name, mean(table[name])

    def copy_factor(table):
        """The run's 1 GiB device copies are the largest dispatches of the runtime's buffer-copy kernel."""
        v = table["__amd_rocclr_copyBuffer"]
        big = [x for x in v if x > 0.5 * max(v)]
        return float(1 << 20) / mean(big), len(big)

    (f_fac, n_f), (w_fac, n_w) = copy_factor(fetch), copy_factor(write)
    kernels = {}
    for key in ("monarch_step1_kernel", "monarch_step2_kernel", "monarch_fused_kernel", "monarch_fused_merge_kernel"):
        if any(key + "<" in k for k in fetch):
            (name, fk), (_, wk) = pick(fetch, key), pick(write, key)
            kernels[key] = {"instantiation": name.split("(")[0], "dispatches": len(fetch[name]), "fetch_size_kib": fk,
                            "write_size_kib": wk, "traffic_bytes": round((fk * f_fac + wk * w_fac) * 1024)}
    commit = subprocess.run(["git", "-C", ROOT, "rev-parse", "--short", "HEAD"], capture_output=True, text=True).stdout.strip()
    dirty = subprocess.run(["git", "-C", ROOT, "status", "--porcelain", "--", "self-forcing_amd/csrc"], capture_output=True,
                           text=True).stdout.strip()
    rec = {"commit": (commit + ("+uncommitted kernel changes" if dirty else "")) or None,
           "command": "rocprofv3 --pmc FETCH_SIZE|WRITE_SIZE --output-format csv -- python3 bench.py --op-only --skip-simt "
                      "--skip-shapes --no-cpu-baseline --copy-probe, then python bench.py --write-traffic FETCH.csv WRITE.csv",
           "copy_kernel": "__amd_rocclr_copyBuffer", "copy_dispatches": [n_f, n_w], "fetch_factor": f_fac,
           "write_factor": w_fac, "kernels": kernels}
    with open(os.path.join(ROOT, "profiles", "traffic.json"), "w") as f:
        json.dump(rec, f, indent=1)
        f.write("\n")
    print(json.dumps(rec, indent=1))


def cpu_baseline(torch):
    """The same module code with the oracle's attention operators on the host cores, bf16 weights: ONE of the 30
    transformer blocks through all 7 x 5 passes of a video (3-frame chunks against the cache as it grows from 3 to 21
    frames, the fifth pass of a chunk being the cache refresh), scaled by the 30 layers."""
    import self_forcing_amd as sfa
    from oracle.ops import OracleOps
    cm = sfa.causal_model
    torch.set_num_threads(os.cpu_count())
    torch.manual_seed(0)
    blk = cm.CausalWanAttentionBlock(1536, 8960, 12, block_num=0, flags=cm.AttentionFlags(0, use_framewise=True),
                                     ops=OracleOps()).to(torch.bfloat16).eval()
    g = torch.Generator().manual_seed(0)
    x = torch.randn(1, SQ, 1536, generator=g).to(torch.bfloat16)
    e = torch.randn(1, 3, 6, 1536, generator=g).to(torch.bfloat16) * 0.1
    ctx = torch.randn(1, 512, 1536, generator=g).to(torch.bfloat16)
    kv = {"k": torch.zeros(1, SKV, 12, 128, dtype=torch.bfloat16), "v": torch.zeros(1, SKV, 12, 128, dtype=torch.bfloat16),
          "global_end_index": torch.tensor([0]), "local_end_index": torch.tensor([0])}
    ca = {"k": None, "v": None, "is_init": False}

    def one_pass(chunk):
        # a chunk's later passes overwrite its own cache rows: the counters go back to the chunk's start first
        kv["global_end_index"].fill_(chunk * SQ)
        kv["local_end_index"].fill_(chunk * SQ)
        kv["_global_end"] = kv["_local_end"] = chunk * SQ
        blk(x, e, (3, 30, 52), ctx, kv, ca, chunk * SQ)

    with torch.no_grad():
        one_pass(0)                                   # untimed: first-touch of the weights, text K/V of the cross-attention
        reps = 2                                      # about 13 s on 16 cores
        t0 = time.perf_counter()
        for _ in range(reps):
            for chunk in range(CHUNKS):
                for _ in range(PASSES):
                    one_pass(chunk)
        per_layer = (time.perf_counter() - t0) / reps
    return {"value": 21.0 / (per_layer * LAYERS), "unit": "latent frames/s", "cores": os.cpu_count(), "kind": "port",
            "sample": f"1 of {LAYERS} layers through all {CHUNKS * PASSES} passes of a video (bf16 torch-CPU block with oracle "
                      f"Monarch attention, 4680 tokens vs a cache of 3 to 21 frames), mean of {reps} runs = {per_layer:.1f} s, "
                      f"scaled x{LAYERS}"}


def op_level(torch, sfa, args):
    """Attention op alone at the chunk shape (BASELINE.json configs[1])."""
    from self_forcing_amd import lib as L
    from self_forcing_amd.monarch_attn import _desc
    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(0)
    bf = torch.bfloat16
    # configs[1]: Q, K RMS-normalised + 3-D RoPE'd, V ~ N(0,1).  The projections' outputs are drawn ~ N(0,1) and go
    # through the fused prologue chunk by chunk, which fills the 21-frame cache (block order = token order for the
    # framewise tiling) and leaves the last chunk's query.
    kc = torch.empty(B, SKV, H, D, dtype=bf, device=dev)
    vc = torch.empty(B, SKV, H, D, dtype=bf, device=dev)
    ones = torch.ones(H * D, dtype=bf, device=dev)
    rope = sfa.prologue.rope_table(D, device=dev)
    for c in range(F // A):
        xq, xk, xv = (torch.randn(B, SQ, H * D, generator=g).to(bf).to(dev) for _ in range(3))
        q = sfa.prologue.qk_prologue(xq, xk, xv, ones, ones, H, (A, B1, B2), A * c, rope, kc, vc, c * SQ)
    nk, nv = kc[:, SKV - SQ:].clone(), vc[:, SKV - SQ:].clone()
    start, end = SKV - SQ, SKV

    def step():
        return sfa.monarch_attn.monarch_attn_with_kv_cache(q, kc, vc, nk, nv, start, end, 1, 1, 1, B1, B2,
                                                           heads_per_pass=args.heads_per_pass, one_kernel=args.one_kernel)

    for _ in range(10):
        out = step()
    torch.cuda.synchronize()
    n = 50
    t0 = time.perf_counter()
    for _ in range(n):
        out = step()
    torch.cuda.synchronize()
    ms_call = (time.perf_counter() - t0) * 1e3 / n

    # per-kernel durations, HIP events on the launch stream (inside the library)
    lib = L.load()
    d = _desc(q, kc, vc, out, 1, 1, 1, B1, B2, D ** -0.5, 1, 0, 1, args.one_kernel)
    nbytes = sfa.monarch_attn.monarch_workspace_bytes(d, args.heads_per_pass)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    t1s, t2s = [], []
    for _ in range(20):
        a1, a2 = C.c_float(0), C.c_float(0)
        L.check(lib.sfm_monarch_fwd_timed(C.byref(d), q.data_ptr(), kc.data_ptr(), vc.data_ptr(), out.data_ptr(),
                                          ws.data_ptr(), nbytes, stream, C.byref(a1), C.byref(a2)))
        t1s.append(a1.value)
        t2s.append(a2.value)
    s1_ms, s2_ms = sum(t1s) / len(t1s), sum(t2s) / len(t2s)

    for _ in range(2):
        sfa.attention.attention(q, kc, vc)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(5):
        sfa.attention.attention(q, kc, vc)
    torch.cuda.synchronize()
    dense_ms = (time.perf_counter() - t0) * 1e3 / 5

    # iterated refinement (num_iters = 8, the reference's "slow" quality setting) at the same shape: on the MFMA kernels
    # and, once, on the fp32 SIMT kernels the same call runs on where the MFMA kernels do not apply
    def iter_call():
        return sfa.monarch_attn.monarch_attn(q, kc, vc, 1, 1, 1, B1, B2, kv_block_order=True, num_iters=8)

    iter_call()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(5):
        iter_call()
    torch.cuda.synchronize()
    iter_ms = (time.perf_counter() - t0) * 1e3 / 5
    iter_simt_ms = None
    if not args.skip_simt:
        old_sw = lib.sfm_set_switches(L.SW_ITER_SIMT)
        try:
            iter_call()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            iter_call()
            torch.cuda.synchronize()
            iter_simt_ms = (time.perf_counter() - t0) * 1e3
        finally:
            lib.sfm_set_switches(old_sw)

    # backward of the same op: with the output and row statistics the forward keeps under autograd, and recomputing
    # them; three timed calls after one warm-up each
    from self_forcing_amd.monarch_attn import _monarch_bwd, _monarch_fwd_stats
    do = torch.randn(B, SQ, H, D, generator=g).to(bf).to(dev)
    out_kept, stats = _monarch_fwd_stats(q, kc, vc, (1, 1, 1, B1, B2), D ** -0.5, 1, 0)
    bwd = {}
    for name, kept in (("recompute", {}), ("saved", {"out": out_kept, "stats": stats})):
        _monarch_bwd(q, kc, vc, do, (1, 1, 1, B1, B2), D ** -0.5, 1, 0, **kept)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(3):
            _monarch_bwd(q, kc, vc, do, (1, 1, 1, B1, B2), D ** -0.5, 1, 0, **kept)
        torch.cuda.synchronize()
        bwd[name] = (time.perf_counter() - t0) * 1e3 / 3
    bwd_ms = bwd["saved"]

    # backward of the dense fallback at the same shape (all keys, and the new chunk's keys only)
    from self_forcing_amd.attention import _dense_bwd, _dense_fwd
    dout_kept, dlse = _dense_fwd(q, kc, vc, D ** -0.5, True)
    dense_bwd = {}
    for name, rng in (("all_keys", (0, SKV)), ("new_chunk_keys", (SKV - SQ, SKV))):
        _dense_bwd(q, kc, vc, dout_kept, dlse, do, D ** -0.5, *rng)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(3):
            _dense_bwd(q, kc, vc, dout_kept, dlse, do, D ** -0.5, *rng)
        torch.cuda.synchronize()
        dense_bwd[name] = (time.perf_counter() - t0) * 1e3 / 3

    # what the matrix pipes sustain on this machine (independent MFMAs only), to read the dense figure against
    probe = C.c_float(0)
    L.check(lib.sfm_probe_mfma_bf16(20000, stream, C.byref(probe)))
    dense_tfl = DENSE_FLOPS / (dense_ms * 1e-3) / 1e12

    # device-to-device copy of 1 GiB: the rate this machine's HBM sustains for a plain stream, read + write
    # (with --copy-probe the copies are also what the rocprofv3 counters are scaled against)
    src = torch.empty(1 << 30, dtype=torch.uint8, device=dev)
    dst = torch.empty_like(src)
    dst.copy_(src)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(5):
        dst.copy_(src)
    e1.record()
    torch.cuda.synchronize()
    copy_gbs = 5 * 2 * (1 << 30) / (e0.elapsed_time(e1) * 1e-3) / 1e9
    del src, dst

    # step 1's memory traffic with nothing else (same tile count, rows and scatter, non-temporal stores): what this
    # machine's memory system takes for the bytes alone.  Six copies of the input, read in turn: a single 201 MB copy
    # stays in the 256 MB memory-side cache between passes and its reads then cost nothing (`cached_reads_us`), which
    # the K / V reads of the operator inside a model never are.
    tiles, rows_in, rows_out, row_bytes = B * H * B1 * F, B2, A * B2, 2 * D
    one_copy = tiles * (2 * rows_in + 2 * rows_out) * row_bytes
    ws = torch.empty(tiles * (2 * rows_in * 6 + 2 * rows_out) * row_bytes, dtype=torch.uint8, device=dev)
    ws.zero_()
    floor_us, cached_us = C.c_float(0), C.c_float(0)
    L.check(lib.sfm_probe_tile_traffic(tiles, rows_in, rows_out, row_bytes, 1, ws.data_ptr(), one_copy, stream, C.byref(cached_us)))
    L.check(lib.sfm_probe_tile_traffic(tiles, rows_in, rows_out, row_bytes, 1, ws.data_ptr(), ws.numel(), stream, C.byref(floor_us)))
    # step 2's: one wave per (unit, a, j) reading its Kbar rows and its Y rows
    s2_waves, s2_kb = B * H * A * B2, (F * B1 * 2 * D + 1023) // 1024
    read_us = C.c_float(0)
    L.check(lib.sfm_probe_row_stream(s2_waves, s2_kb, ws.data_ptr(), ws.numel(), stream, C.byref(read_us)))
    # the rate at which all compute units together can be fed from L2 (one workgroup per CU streaming a shared 2 MB window)
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    l2_us = C.c_float(0)
    L.check(lib.sfm_probe_l2_read(cus, 64, ws.data_ptr(), ws.numel(), stream, C.byref(l2_us)))
    l2_tbs = cus * 64 * 32768 / (l2_us.value * 1e-6) / 1e12
    del ws

    traffic = measured_traffic()
    t_of = lambda k: traffic["kernels"].get(k, {}).get("traffic_bytes")
    s1_gbs = STEP1_BYTES / (s1_ms * 1e-3) / 1e9
    s2_gbs = STEP2_BYTES / (s2_ms * 1e-3) / 1e9
    tfl = MONARCH_FLOPS / (ms_call * 1e-3) / 1e12
    return {
        "monarch_attn": {"workload": "configs[1]: monarch_attn_with_kv_cache, B1 H12 D128, a=3 f=21 b1=30 b2=52 "
                                     "(4680 q x 32760 kv), new chunk written at tokens 28080..32760; Q, K RMS-normalised + 3-D "
                                     "RoPE'd (N(0,1) projections through qk_prologue), V ~ N(0,1), seed 0",
                         "ms_per_call": ms_call, "tflops": tfl, "mfma_frac": tfl / MFMA_BF16_PEAK_TFLOPS,
                         "kernel_ms": {"monarch_step1": s1_ms, "monarch_step2": s2_ms}},
        "monarch_iter": {"workload": "monarch_attn, num_iters = 8 (monarch_attn_slow), same shape and cache",
                         "ms_per_call": iter_ms, "ms_per_call_fp32_simt_kernels": iter_simt_ms,
                         "tflops": 8 * MONARCH_FLOPS / (iter_ms * 1e-3) / 1e12},
        "monarch_bwd": {"workload": "gradients of q and of all 21 cached K/V frames at the same shape",
                        "ms_per_call": bwd_ms, "ms_per_call_recomputing_statistics": bwd["recompute"]},
        "l2_read_probe_tbs": l2_tbs,
        "dense_fallback": {"ms_per_call": dense_ms, "tflops": dense_tfl, "mfma_frac": dense_tfl / MFMA_BF16_PEAK_TFLOPS,
                           "mfma_probe_tflops": probe.value, "frac_of_probe": dense_tfl / probe.value,
                           "bwd_ms_per_call": dense_bwd["all_keys"], "bwd_ms_per_call_new_chunk_keys": dense_bwd["new_chunk_keys"]},
        "roofline": {"kernel": "monarch_step1_kernel (configs[1] shape)", "bound": "hbm", "achieved": s1_gbs,
                     "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": s1_gbs / HBM_PEAK_GBS,
                     "algorithmic_bytes": STEP1_BYTES, "traffic": t_of("monarch_step1_kernel"),
                     "traffic_measured_at_commit": traffic["commit"],
                     "copy_probe_gbs": copy_gbs, "frac_of_copy_probe": s1_gbs / copy_gbs,
                     "traffic_only_us": floor_us.value, "frac_of_traffic_only": floor_us.value / (s1_ms * 1e3),
                     "traffic_only_cached_reads_us": cached_us.value},
        "roofline_step2": {"kernel": "monarch_step2_kernel (configs[1] shape)", "bound": "hbm", "achieved": s2_gbs,
                           "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": s2_gbs / HBM_PEAK_GBS,
                           "algorithmic_bytes": STEP2_BYTES, "traffic": t_of("monarch_step2_kernel"),
                           "traffic_measured_at_commit": traffic["commit"],
                           "copy_probe_gbs": copy_gbs, "frac_of_copy_probe": s2_gbs / copy_gbs,
                           "traffic_only_us": read_us.value, "frac_of_traffic_only": read_us.value / (s2_ms * 1e3)},
    }


def gemm_legs(torch, sfa):
    """The block's four GEMM shapes at M = 4680 (1.3B and 14B widths), each with its element-wise tail: hipBLASLt
    (TunableOp's pick) alone and followed by the separate tail kernel, against `linear.linear` with the tail in the
    epilogue.  HIP-event means of 30 calls after 5 warm-up calls."""
    dev, bf = "cuda:0", torch.bfloat16
    sfa.pipeline.use_tuned_gemms()
    shapes = [("qkv", 4680, 4608, 1536, "none"), ("o_proj", 4680, 1536, 1536, "gate_residual"),
              ("ffn_up", 4680, 8960, 1536, "gelu_tanh"), ("ffn_down", 4680, 1536, 8960, "gate_residual"),
              ("14b_qkv", 4680, 15360, 5120, "none"), ("14b_ffn_up", 4680, 13824, 5120, "gelu_tanh"),
              ("14b_ffn_down", 4680, 5120, 13824, "gate_residual")]

    def timeit(f, n=30):
        for _ in range(5):
            f()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(n):
            f()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e3 / n

    out = {}
    g = torch.Generator().manual_seed(0)
    with torch.no_grad():
        for name, M, N, K, epi in shapes:
            x = torch.randn(1, M, K, generator=g).to(bf).to(dev)
            lin = torch.nn.Linear(K, N, device=dev, dtype=bf)
            w, b = lin.weight.detach(), lin.bias.detach()
            res = torch.randn(1, M, N, generator=g).to(bf).to(dev)
            gate = torch.randn(1, 3, 1, N, generator=g).to(bf).to(dev)
            rec = {"M": M, "N": N, "K": K, "epilogue": epi, "library_gemm_us": timeit(lambda: lin(x))}
            if epi == "gelu_tanh":
                rec["library_plus_tail_us"] = timeit(lambda: torch.nn.functional.gelu(lin(x), approximate="tanh"))
                rec["library_fused_gelu_us"] = timeit(lambda: torch._addmm_activation(b, x[0], w.t(), use_gelu=True))
                rec["own_us"] = timeit(lambda: sfa.linear.linear(x, w, b, epilogue="gelu_tanh"))
            elif epi == "gate_residual":
                rec["library_plus_tail_us"] = timeit(lambda: sfa.block_ops.gate_residual_(res, lin(x), gate))
                rec["own_us"] = timeit(lambda: sfa.linear.linear(x, w, b, epilogue="gate_residual", res=res, gate=gate))
            else:
                rec["own_us"] = timeit(lambda: sfa.linear.linear(x, w, b))
            rec["own_tflops"] = 2.0 * M * N * K / rec["own_us"] / 1e6
            out[name] = rec
    return out


def forward_shapes_leg(torch, sfa):
    """ms per call of the two Monarch forwards (two kernels with Kbar / Y in HBM; one kernel with them in LDS) at the
    chunk shapes of the rollout configurations: 3 query frames against a 21-frame cache in block order, bf16, random
    operands.  The one-kernel forward covers b1 <= 32, b2 <= 64; elsewhere its column is null."""
    dev, bf = "cuda:0", torch.bfloat16
    shapes = [("c2: H12, 30x52 framewise (a=3 f=21 b1=30 b2=52)", 12, 30, 52, (1, 1, 1)),
              ("c4: H12, 30x52 reduce2xh (a=6 f=42 b1=15 b2=52)", 12, 30, 52, (1, 2, 1)),
              ("c5: H40, 30x52 framewise", 40, 30, 52, (1, 1, 1)),
              ("reference default tiling: H12, 30x52, three frames tied (a=1 f=7 b1=90 b2=52)", 12, 30, 52, (3, 1, 1)),
              ("720p: H12, 45x80 framewise (a=3 f=21 b1=45 b2=80)", 12, 45, 80, (1, 1, 1))]
    out = {}
    g = torch.Generator().manual_seed(1)
    for name, heads, h, w, tiling in shapes:
        q = torch.randn(1, 3 * h * w, heads, 128, generator=g).to(bf).to(dev)
        k = torch.randn(1, 21 * h * w, heads, 128, generator=g).to(bf).to(dev)
        v = torch.randn(1, 21 * h * w, heads, 128, generator=g).to(bf).to(dev)
        b1, b2 = tiling[0] * h // tiling[1], w // tiling[2]
        rec = {}
        for key, one in (("two_kernels_ms", False), ("one_kernel_ms", True)):
            if one and (b1 > 32 or b2 > 64):
                rec[key] = None
                continue
            f = lambda: sfa.monarch_attn.monarch_attn(q, k, v, *tiling, h, w, kv_block_order=True, one_kernel=one)
            for _ in range(3):
                f()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(10):
                f()
            e1.record()
            torch.cuda.synchronize()
            rec[key] = e0.elapsed_time(e1) / 10
        out[name] = rec
        del q, k, v
    sfa.monarch_attn.release_scratch()
    torch.cuda.empty_cache()
    return out


def rollout_leg(torch, sfa, name, steps, warmup, own_gemm):
    """Seconds per video of the rollout configuration `name`: `warmup` untimed videos, then `steps` timed ones between
    device synchronisations.  The generator and its caches are freed afterwards."""
    _, size, flags, _ = ROLLOUTS[name]
    pl = sfa.pipeline
    pl.use_tuned_gemms()          # hipBLASLt solution per GEMM shape (shipped selections; unknown shapes tuned in warm-up)
    gen = pl.build_generator(size, attention_flags=flags, ops=sfa.causal_model.HipAttentionOps(own_gemm=own_gemm),
                             init_on_device=size == "14B")
    pipe = pl.CausalInferencePipeline(gen)
    g = torch.Generator().manual_seed(0)
    noise = torch.randn(1, 21, 16, 60, 104, generator=g).to(torch.bfloat16).cuda()
    ctx = torch.randn(1, 512, 4096, generator=g).to(torch.bfloat16).cuda()
    for _ in range(warmup):
        pipe.inference(noise, ctx)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        out = pipe.inference(noise, ctx)
    torch.cuda.synchronize()
    sec = (time.perf_counter() - t0) / steps
    assert torch.isfinite(out).all()
    del pipe, gen, out
    gc.collect()
    torch.cuda.empty_cache()
    torch.cuda.tunable.tuning_enable(False)       # later legs keep the selections made so far and tune nothing new
    return sec


def vae_decode_leg(torch, sfa):
    """Streaming decode of one video's latents (outside the headline metric, which excludes the VAE): random-init
    decoder of the Wan 2.1 VAE shape, bf16, 21 latent frames in 7 chunks of 3 -> 81 frames of 480x832."""
    vae = sfa.vae_decode.WanVAEDecoder().eval().to("cuda", torch.bfloat16)
    g = torch.Generator().manual_seed(0)
    lat = torch.randn(1, 21, 16, 60, 104, generator=g).to(torch.bfloat16).cuda()
    sec = None
    for _ in range(2):                         # the first pass warms up
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        st, frames = vae.new_state(), 0
        for c in range(7):
            frames += vae.decode_to_pixel(lat[:, 3 * c:3 * c + 3], use_cache=True, state=st).shape[1]
        torch.cuda.synchronize()
        sec = time.perf_counter() - t0
    return {"workload": "WanVAEDecoder (dim 96, z 16), 21 latent frames 60x104 in 7 chunks -> 81 frames 480x832, bf16, "
                        "HIP channels-last convolutions", "ms_per_video": sec * 1e3, "pixel_frames_per_s": frames / sec,
            "latent_frames_per_s": 21.0 / sec}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=3, help="timed videos (21 latent frames each)")
    ap.add_argument("--warmup", type=int, default=1)
    ap.add_argument("--config", choices=sorted(ROLLOUTS), default="c3",
                    help="the rollout that `value` measures: c3 = BASELINE.json configs[2] (the headline), c4 = configs[3] "
                         "(reduce2xh + dense first chunk), c5 = configs[4] (14B), dense = the 1.3B model with Monarch "
                         "disabled.  The op-level legs are the same for all; the VAE leg and the CPU baseline belong to c3")
    ap.add_argument("--heads-per-pass", type=int, default=0)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--op-only", action="store_true", help="skip the model; time the attention op only")
    ap.add_argument("--rollout-only", action="store_true",
                    help="for kernel traces: the rollout alone, without the op-level legs, the VAE leg and the CPU baseline "
                         "(the line then carries no roofline)")
    ap.add_argument("--own-gemm", choices=("auto", "all", "none"), default="none",
                    help="which linear layers of the rollout run on the library's own kernel (sfm_linear): none = hipBLASLt "
                         "everywhere (fastest), auto = the block's square projections, all = also the FFN with GELU / gated "
                         "residual in the epilogue")
    ap.add_argument("--no-extra-rollouts", action="store_true",
                    help="skip the short legs of the other rollout configurations (c4, dense, c5) that follow the c3 headline")
    ap.add_argument("--one-kernel", action="store_true",
                    help="op-level figures of the opt-in one-kernel Monarch forward (Kbar / Y kept in LDS) instead of the default "
                         "two kernels; kernel_ms then holds the fused kernel and its merge kernel")
    ap.add_argument("--skip-simt", action="store_true", help="leave out the 0.7 s of fp32 SIMT refinement calls (profile runs)")
    ap.add_argument("--skip-shapes", action="store_true",
                    help="leave out the leg that times both forwards at other chunk shapes (counter runs: the per-dispatch "
                         "averages of profiles/traffic.json must cover the configs[1] shape only)")
    ap.add_argument("--copy-probe", action="store_true",
                    help="accepted for the profile commands; the 1 GiB device copies (known HBM traffic, for scaling rocprof "
                         "counters) always run")
    ap.add_argument("--vae-only", action="store_true", help="the streaming VAE decode leg alone (profile runs)")
    ap.add_argument("--gemm-legs", action="store_true",
                    help="only the table of the block's GEMM shapes: hipBLASLt (+ tail kernel) against sfm_linear with the tail fused")
    ap.add_argument("--write-traffic", nargs=2, metavar=("FETCH_CSV", "WRITE_CSV"),
                    help="no GPU work: rewrite profiles/traffic.json from two rocprofv3 counter_collection CSVs")
    args = ap.parse_args()
    if args.write_traffic:
        write_traffic(*args.write_traffic)
        return
    if args.gpus != 1:
        print("bench.py measures one GPU only: this build has no multi-GPU path (--gpus must be 1)", file=sys.stderr)
        sys.exit(2)

    import torch
    import self_forcing_amd as sfa

    torch.cuda.set_device(0)
    if args.gemm_legs:
        print(json.dumps({"metric": "block GEMM shapes, us per call", "gemm": gemm_legs(torch, sfa)}))
        return
    if args.vae_only:
        print(json.dumps({"metric": "streaming VAE decode", "vae_decode": vae_decode_leg(torch, sfa)}))
        return
    entry, size, flags, what = ROLLOUTS[args.config]
    rec = {"metric": f"latent frames/s, causal Wan-{size} 480x832 bf16 (+ Monarch attn ms/call, MFMA %)",
           "unit": "latent frames/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
           "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
           "config": {"workload": f"{entry}: {what}, latents 21x16x60x104 in 7 chunks of 3 frames, 4 denoising steps + 1 "
                                  "cache-refresh pass per chunk, per-layer KV cache, text context [1,512,4096] ~ N(0,1); "
                                  "VAE and text encoder excluded",
                      "name": args.config, "heads_per_pass": args.heads_per_pass}}
    own = {"auto": "auto", "all": True, "none": False}[args.own_gemm]
    if not args.op_only:
        sec = rollout_leg(torch, sfa, args.config, args.steps, args.warmup, own)
        rec["config"]["own_gemm"] = args.own_gemm
        rec["value"] = 21.0 / sec
        rec["ms_per_step"] = sec * 1e3
    if args.rollout_only:
        print(json.dumps(rec))
        return
    if not args.op_only and args.config == "c3" and not args.no_extra_rollouts:
        # the other rollout configurations, 1 warm-up + 2 timed videos each (the headline fields above are c3's)
        rec["rollouts"] = {}
        for name in ("c4", "dense", "c5"):
            sec = rollout_leg(torch, sfa, name, 2, 1, own)
            entry, size, _, what = ROLLOUTS[name]
            rec["rollouts"][name] = {"workload": f"{entry}: {what}", "value": 21.0 / sec, "unit": "latent frames/s",
                                     "ms_per_step": sec * 1e3, "steps": 2, "warmup": 1}
    rec.update(op_level(torch, sfa, args))
    if not args.skip_shapes:
        rec["monarch_forward_shapes"] = forward_shapes_leg(torch, sfa)
    if args.config == "c3":
        rec["vae_decode"] = vae_decode_leg(torch, sfa)
    if args.op_only:
        rec["metric"] = "Monarch attn ms/call, causal Wan-1.3B 480x832 chunk shape, bf16"
        rec["unit"], rec["higher_is_better"] = "ms/call", False
        rec["value"] = rec["ms_per_step"] = rec["monarch_attn"]["ms_per_call"]
    if not args.no_cpu_baseline and args.config == "c3":
        rec["cpu_baseline"] = cpu_baseline(torch)
    print(json.dumps(rec))


if __name__ == "__main__":
    main()
