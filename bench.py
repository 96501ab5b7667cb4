#!/usr/bin/env python3
"""Benchmark of the attention hot path on one MI355X.

One step = one call of monarch_attn_with_kv_cache (cache write of the new 3-frame chunk + two-step
Monarch attention) at the Wan-1.3B 480x832 chunk shape: B=1, H=12, D=128, 4680 queries against a
21-frame (32760-token) KV cache, bf16, inputs resident in HBM.  Prints ONE JSON line.
"""
import argparse
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


# HBM bytes per launch measured with rocprofv3 (FETCH_SIZE x 2.0 + WRITE_SIZE x 1.0, factors from a 1 GiB
# device copy in the same run); the runs and raw counters are in profiles/monarch_step{1,2}_c2.md.
MEASURED_TRAFFIC = {"monarch_step1_kernel": 868.7e6, "monarch_step2_kernel": 647.2e6}


def cpu_baseline(torch):
    """The reference's CPU torch formulation restated by the oracle, fp32, on ONE of the 12 heads of the
    same workload; scaled by 12 to a per-call figure."""
    from oracle import monarch
    torch.set_num_threads(os.cpu_count())
    g = torch.Generator().manual_seed(0)
    q = torch.randn(1, A, B1, B2, 1, D, generator=g)
    k = torch.randn(1, F, B1, B2, 1, D, generator=g)
    v = torch.randn(1, F, B1, B2, 1, D, generator=g)
    monarch.monarch_1iter(q[:, :, :, :, :, :], k[:, :3], v[:, :3], D ** -0.5, dtype=torch.float32)   # warm-up
    times = []
    for _ in range(3):
        t0 = time.perf_counter()
        monarch.monarch_1iter(q, k, v, D ** -0.5, dtype=torch.float32)
        times.append(time.perf_counter() - t0)
    ms_call = sorted(times)[1] * 1e3 * H
    return {"value": ms_call, "unit": "ms/call", "cores": os.cpu_count(), "kind": "port",
            "sample": "1 of 12 heads of the same call (fp32 torch einsum oracle), median of 3, scaled x12"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--heads-per-pass", type=int, default=0)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--copy-probe", action="store_true",
                    help="also run a plain 1 GiB device copy (known HBM traffic, for scaling rocprof counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU only: this build has no multi-GPU path (--gpus must be 1)", file=sys.stderr)
        sys.exit(2)

    import torch
    import self_forcing_amd as sfa
    from self_forcing_amd import lib as L
    from self_forcing_amd.monarch_attn import _desc

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    g = torch.Generator().manual_seed(0)
    bf = torch.bfloat16
    q = torch.randn(B, SQ, H, D, generator=g).to(bf).to(dev)
    kc = torch.randn(B, SKV, H, D, generator=g).to(bf).to(dev)
    vc = torch.randn(B, SKV, H, D, generator=g).to(bf).to(dev)
    nk = torch.randn(B, SQ, H, D, generator=g).to(bf).to(dev)
    nv = torch.randn(B, SQ, H, D, generator=g).to(bf).to(dev)
    start, end = SKV - SQ, SKV

    def step():
        return sfa.monarch_attn.monarch_attn_with_kv_cache(q, kc, vc, nk, nv, start, end, 1, 1, 1, B1, B2,
                                                           heads_per_pass=args.heads_per_pass)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        out = step()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps

    # per-kernel durations, HIP events on the launch stream (inside the library)
    lib = L.load()
    d = _desc(q, kc, vc, out, 1, 1, 1, B1, B2, D ** -0.5, 1, 0)
    nbytes = sfa.monarch_attn.monarch_workspace_bytes(d, args.heads_per_pass)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    t1s, t2s = [], []
    for _ in range(max(5, min(args.steps, 20))):
        a1, a2 = C.c_float(0), C.c_float(0)
        L.check(lib.sfm_monarch_fwd_timed(C.byref(d), q.data_ptr(), kc.data_ptr(), vc.data_ptr(), out.data_ptr(),
                                          ws.data_ptr(), nbytes, stream, C.byref(a1), C.byref(a2)))
        t1s.append(a1.value)
        t2s.append(a2.value)
    s1_ms, s2_ms = sum(t1s) / len(t1s), sum(t2s) / len(t2s)

    # dense fallback on the same tensors (for the record)
    for _ in range(2):
        sfa.attention.attention(q, kc, vc)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(5):
        sfa.attention.attention(q, kc, vc)
    torch.cuda.synchronize()
    dense_ms = (time.perf_counter() - t0) * 1e3 / 5

    if args.copy_probe:
        src = torch.empty(1 << 30, dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()

    s1_gbs = STEP1_BYTES / (s1_ms * 1e-3) / 1e9
    s2_gbs = STEP2_BYTES / (s2_ms * 1e-3) / 1e9
    rec = {
        "metric": "Monarch attn ms/call, causal Wan-1.3B 480x832 chunk shape (4680 q x 32760 kv, H12 D128), bf16",
        "value": ms_per_step, "unit": "ms/call", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "configs[1]: monarch_attn_with_kv_cache, B1 H12 D128, a=3 f=21 b1=30 b2=52, "
                               "new chunk written at tokens 28080..32760", "heads_per_pass": args.heads_per_pass},
        "monarch_tflops": MONARCH_FLOPS / (ms_per_step * 1e-3) / 1e12,
        "monarch_mfma_frac": MONARCH_FLOPS / (ms_per_step * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS,
        "kernel_ms": {"monarch_step1": s1_ms, "monarch_step2": s2_ms},
        "dense_fallback": {"ms_per_call": dense_ms, "tflops": DENSE_FLOPS / (dense_ms * 1e-3) / 1e12,
                           "mfma_frac": DENSE_FLOPS / (dense_ms * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS},
        "roofline": {"kernel": "monarch_step1_kernel", "bound": "hbm", "achieved": s1_gbs, "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": s1_gbs / HBM_PEAK_GBS, "algorithmic_bytes": STEP1_BYTES,
                     "traffic": MEASURED_TRAFFIC["monarch_step1_kernel"]},
        "roofline_step2": {"kernel": "monarch_step2_kernel", "bound": "hbm", "achieved": s2_gbs,
                           "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": s2_gbs / HBM_PEAK_GBS,
                           "algorithmic_bytes": STEP2_BYTES, "traffic": MEASURED_TRAFFIC["monarch_step2_kernel"]},
    }
    if not args.no_cpu_baseline:
        rec["cpu_baseline"] = cpu_baseline(torch)
    print(json.dumps(rec))


if __name__ == "__main__":
    main()
