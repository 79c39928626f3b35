"""Benchmark of the nmg sparse x dense matmul on one MI355X.

Workload (BASELINE config 2): fp16 weight 4096x4096 ~ N(0, 0.02), grouped 2:4 (group 16) along
the reduction dim; fp16 activations 2048 tokens x 4096 ~ N(0,1); forward only, fp32 accumulate.
A "step" is one nmg x dense matmul over that batch with every operand resident in HBM.

Prints one JSON line.  value = dense-equivalent TFLOP/s (2*M*K*N / step time).
roofline.achieved counts the effective (non-zero) flops 2*M*K*N*n/m per launch over the kernel's
average launch duration, measured with HIP events on the stream the kernel is launched on, against
the dense fp16 MFMA peak -- i.e. the fraction of the density-scaled MFMA roofline.
roofline.traffic is read from the committed rocprofv3 --pmc summary of this same command.
cpu_baseline = the CPU restatement of the reference's AVX/OpenMP kernel (oracle/nmg_cpu_simd.cpp)
on the host cores, same shape, fp32.

Other modes: --workload picks another BASELINE shape for ad-hoc measurement; --calibrate-copy
runs a plain device copy of known size (the counter calibration for FETCH_SIZE / WRITE_SIZE).
"""
import argparse
import json
import os
import re
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_FP16_TFLOPS = 2500.0   # MI355X dense fp16 MFMA
PEAK_HBM_GBS = 8000.0

WORKLOADS = {
    # name: (M, K, tokens, n, m, g, description)
    "c2": (4096, 4096, 2048, 2, 4, 16, "configs[1]: W 4096x4096 fp16 2:4:16 along K x 2048 tokens, forward"),
    "target_2_4": (4096, 11008, 2048, 2, 4, 16, "north_star: W 4096x11008 fp16 2:4:16 x 2048 tokens, forward"),
    "c3_1_8": (8192, 8192, 4096, 1, 8, 32, "configs[2]: W 8192x8192 fp16 1:8:32 x 4096 tokens, forward"),
    "c3_2_8": (8192, 8192, 4096, 2, 8, 32, "configs[2]: W 8192x8192 fp16 2:8:32 x 4096 tokens, forward"),
    "c3_4_8": (8192, 8192, 4096, 4, 8, 32, "configs[2]: W 8192x8192 fp16 4:8:32 x 4096 tokens, forward"),
    "c5_fwd": (16384, 4096, 4096, 2, 4, 16, "configs[4]: W 16384x4096 fp16 2:4:16 x 4096 tokens, forward"),
}


def cpu_baseline(M, K, N, n, m, g, seconds=15.0):
    import numpy as np
    from oracle import nmg_oracle as O
    rng = np.random.default_rng(0)
    # bounded sample: the reference kernel works on fp32 with the n:m blocks along M; a slab of
    # M_s rows of the same weight shape keeps the per-row work identical
    M_s = min(M, 1024)
    W = (rng.standard_normal((M_s, K)) * 0.02).astype(np.float32)
    X = rng.standard_normal((K, N)).astype(np.float32)
    val, idx, lay = O.sparsify(W, n, m, 0, g, 1)
    O.simd_spmm(val, idx, lay, X)
    t0 = time.perf_counter()
    it = 0
    while True:
        O.simd_spmm(val, idx, lay, X)
        it += 1
        if time.perf_counter() - t0 > seconds or it >= 50:
            break
    dt = (time.perf_counter() - t0) / it
    info = O.simd_info()
    return {
        "value": 2.0 * M_s * K * N / dt / 1e12,
        "unit": "TFLOP/s dense-equiv",
        "cores": info["threads"],
        "kind": "port",
        "sample": f"{M_s}x{K} fp32 slab of the weight x {N} tokens, {it} passes, kernel {info['kernel']}",
    }


def committed_traffic(workload):
    """HBM bytes per launch from profiles/ (FETCH_SIZE + WRITE_SIZE, calibrated), or None."""
    path = os.path.join(ROOT, "profiles", f"spmm_{workload}_pmc.txt")
    try:
        text = open(path).read()
    except OSError:
        return None
    mt = re.search(r"^traffic_bytes_per_launch:\s*([0-9.eE+]+)", text, re.M)
    return float(mt.group(1)) if mt else None


def calibrate_copy():
    import torch
    n = 64 * 1024 * 1024
    src = torch.empty(n, dtype=torch.uint8, device="cuda:0").random_(0, 255)
    dst = torch.empty_like(src)
    for _ in range(5):
        dst.copy_(src)
    torch.cuda.synchronize()
    print(json.dumps({"calibration": "device copy", "bytes_read": n, "bytes_written": n}))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="c2", choices=sorted(WORKLOADS))
    ap.add_argument("--kernel", default="auto")
    ap.add_argument("--variant", type=int, default=-1)
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--calibrate-copy", action="store_true")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU; multi-GPU runs are not part of this build", file=sys.stderr)
        sys.exit(2)
    if args.calibrate_copy:
        calibrate_copy()
        return

    import torch
    import sten_amd as sten

    dev = "cuda:0"
    M, K, N, n, m, g, desc = WORKLOADS[args.workload]
    torch.manual_seed(0)
    W = (torch.randn(M, K) * 0.02).half().to(dev)
    X = torch.randn(N, K).half().to(dev)
    w = sten.GroupedNMTensor.from_dense(W, n, m, sparse_dim=1, group_size=g, group_dim=0)
    w.spmm_opt["variant"] = args.variant
    del W
    for _ in range(args.warmup):
        y = sten.spmm(w, X, reduce_dim=1, kernel=args.kernel)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        y = sten.spmm(w, X, reduce_dim=1, kernel=args.kernel)
    torch.cuda.synchronize()
    wall = (time.perf_counter() - t0) / args.steps

    # average launch duration of the kernel: one HIP event pair around K back-to-back launches,
    # recorded on the stream the kernel is launched on (torch's current stream)
    stream = torch.cuda.current_stream()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record(stream)
    for _ in range(args.steps):
        sten.spmm(w, X, reduce_dim=1, kernel=args.kernel)
    e1.record(stream)
    torch.cuda.synchronize()
    kern_ms = e0.elapsed_time(e1) / args.steps

    dense_flops = 2.0 * M * K * N
    eff_flops = dense_flops * n / m
    achieved = eff_flops / (kern_ms * 1e-3) / 1e12
    out = {
        "metric": "nmg sparse x dense GEMM TFLOP/s (dense-equiv)",
        "value": dense_flops / wall / 1e12,
        "unit": "TFLOP/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": wall * 1e3,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16", "data": "synthetic",
        "config": {"workload": desc, "kernel": args.kernel, "variant": args.variant,
                   "effective_tflops": eff_flops / wall / 1e12, "kernel_ms": kern_ms},
        "roofline": {"bound": "mfma", "achieved": achieved, "peak": PEAK_FP16_TFLOPS,
                     "unit": "TFLOP/s", "frac": achieved / PEAK_FP16_TFLOPS,
                     "traffic": committed_traffic(args.workload),
                     "flops": "effective non-zero (2*M*K*N*n/m); dense-equivalent is m/n times this"},
    }
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(M, K, N, n, m, g)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
