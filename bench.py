"""Benchmark of the grouped n:m (nmg) hot path on one MI355X.

Default (headline) workload: the north-star shape, fp16 weight 4096x11008 ~ N(0, 0.02), grouped
2:4 (group 16) along the reduction dim; fp16 activations 2048 tokens x 11008 ~ N(0,1); forward
only, fp32 accumulate.  A "step" is one pass of the measured operation over that batch with every
operand resident in HBM.

Prints one JSON line.  For the matmul workloads value = dense-equivalent TFLOP/s (2*M*K*N / step
time) and roofline.achieved counts the effective (non-zero) flops 2*M*K*N*n/m per launch over the
kernel's launch duration (the median over the timed steps, one HIP event pair per step on the
stream the kernel is launched on), against the dense fp16 MFMA peak -- i.e. the fraction of the
density-scaled MFMA roofline.
For the bandwidth-bound workloads (decode shapes, sparsifier) value = GB/s of algorithmic bytes
(weight values + int16 indices + activations + output; dense input + val + idx for the
sparsifier) and the roofline is HBM.  roofline.traffic is the HBM bytes per launch that the
committed rocprofv3 counter summary of the workload reports (its `traffic_bytes_per_launch` line:
FETCH_SIZE and WRITE_SIZE runs, scaled by a copy of known size; roofline.traffic_source names the
file under profiles/ and says that the figure is not measured by this run), null for a workload
without such a summary -- the counters cannot be read from inside this process.
With the default workload the same run also measures the other benchmark rows (config 2, config 3
at 1:8 / 2:8 / 4:8, the decode shapes at 1, 4, 8 and 16 tokens, config 4 at 1, 4 and 16 tokens, the
config 2 sparsifier and the config 5 training step without and with the optimizer update) with the
same protocol and reports them under config.also as
{us, value, unit, frac}; --no-also skips them.
cpu_baseline (headline and config 2) = the CPU restatement of the reference's AVX/OpenMP kernel
(oracle/nmg_cpu_simd.cpp) on the host cores, same shape, fp32, on a 1024-row slab of the weight;
for the sparsifier workloads the restatement of the reference's single-threaded sort-and-scan on
a slab of the weight.

Timing protocol: `warmup` untimed steps, more untimed steps until 80 ms of load have passed, then
the K timed steps back to back between two synchronisations, cut by HIP events into groups that
last about 0.5 ms each (one step where a step is longer; see measure()).  Reported are the median,
the minimum and the maximum over the groups of duration / steps in the group (the roofline uses the
median), the mean from the first to the last event, and ms_per_step = wall clock of the K steps /
K.  The decode shapes replay their steps from a HIP graph (events cannot be recorded into one): a
timed iteration is one replay of a graph of GRAPH_STEPS steps, divided by GRAPH_STEPS.

Other modes: --workload picks another benchmark shape; --calibrate-copy runs a plain device copy
of known size (the counter calibration for FETCH_SIZE / WRITE_SIZE).
"""
import argparse
import gc
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_FP16_TFLOPS = 2500.0   # MI355X dense fp16 MFMA
PEAK_FP32_TFLOPS = 157.3    # MI355X dense fp32 MFMA
ROTATE_BYTES = 512 * 1024 * 1024
PEAK_HBM_GBS = 8000.0
SETTLE_S = 0.08                # untimed load before the timed steps (see measure())
GRAPH_STEPS = 20               # steps per replayed HIP graph (decode shapes)
FP32_WORKLOADS = ("c1", "ref_f32", "big_f32")
BF16_WORKLOADS = ("target_2_4_bf16",)

WORKLOADS = {
    # name: (kind, M, K, tokens, n, m, g, description)
    "c1": ("fwd", 768, 768, 256, 2, 4, 16, "configs[0]: W 768x768 fp32 2:4:16 x 256 tokens, forward (the reference's own CPU-runnable case; fp32 matrix cores)"),
    "ref_f32": ("fwd", 768, 3072, 4096, 3, 6, 12, "the reference's matmul-test shape in its own dtype: W 768x3072 fp32 3:6:12 x 4096 tokens, forward (fp32 matrix cores on the expanded weight)"),
    "big_f32": ("fwd", 8192, 8192, 4096, 2, 4, 16, "W 8192x8192 fp32 2:4:16 x 4096 tokens, forward (fp32 matrix cores on the expanded weight)"),
    "c2": ("fwd", 4096, 4096, 2048, 2, 4, 16, "configs[1]: W 4096x4096 fp16 2:4:16 along K x 2048 tokens, forward"),
    "target_2_4": ("fwd", 4096, 11008, 2048, 2, 4, 16, "north_star: W 4096x11008 fp16 2:4:16 x 2048 tokens, forward"),
    "target_2_4_4k": ("fwd", 4096, 11008, 4096, 2, 4, 16, "north_star: W 4096x11008 fp16 2:4:16 x 4096 tokens, forward"),
    # the same product in bf16: three mantissa bits fewer toggle in the multipliers, and the power limit leaves more
    "target_2_4_bf16": ("fwd", 4096, 11008, 2048, 2, 4, 16, "W 4096x11008 bf16 2:4:16 x 2048 tokens, forward"),
    "target_2_4_64": ("fwd", 4096, 11008, 64, 2, 4, 16, "W 4096x11008 fp16 2:4:16 x 64 tokens, forward (split reduction)"),
    "target_2_4_256": ("fwd", 4096, 11008, 256, 2, 4, 16, "W 4096x11008 fp16 2:4:16 x 256 tokens, forward (split reduction)"),
    "target_2_4_512": ("fwd", 4096, 11008, 512, 2, 4, 16, "W 4096x11008 fp16 2:4:16 x 512 tokens, forward (split reduction)"),
    "c3_1_8": ("fwd", 8192, 8192, 4096, 1, 8, 32, "configs[2]: W 8192x8192 fp16 1:8:32 x 4096 tokens, forward"),
    "c3_2_8": ("fwd", 8192, 8192, 4096, 2, 8, 32, "configs[2]: W 8192x8192 fp16 2:8:32 x 4096 tokens, forward"),
    "c3_4_8": ("fwd", 8192, 8192, 4096, 4, 8, 32, "configs[2]: W 8192x8192 fp16 4:8:32 x 4096 tokens, forward"),
    "c5_fwd": ("fwd", 16384, 4096, 4096, 2, 4, 16, "configs[4]: W 16384x4096 fp16 2:4:16 x 4096 tokens, forward"),
    "c5_grad_x": ("grad_x", 16384, 4096, 4096, 2, 4, 16, "configs[4]: dY 4096x16384 x W 16384x4096 fp16 2:4:16, grad_input"),
    "c5_grad_w_dense": ("gw_dense", 16384, 4096, 4096, 2, 4, 16, "configs[4] shapes: the dense weight gradient dY^T X (default gradient format), dY 4096x16384, X 4096x4096, fp16, nmg_gemm_tn (the kernel of the masked product without its mask)"),
    "c5_step": ("step", 16384, 4096, 4096, 2, 4, 16, "configs[4]: training step of a sparse linear 4096 -> 16384, 4096 tokens: forward, grad_input, masked grad_weight in val layout"),
    "c5_train": ("train", 16384, 4096, 4096, 2, 4, 16, "configs[4] + optimizer: the training step of c5_step followed by an SGD update of the compressed weight (pattern kept) and the re-derivation of the matmul operands"),
    "c2_grad_x": ("grad_x", 4096, 4096, 2048, 2, 4, 16, "configs[1] shape: dY 2048x4096 x W 4096x4096 fp16 2:4:16, grad_input"),
    "decode_1": ("decode", 4096, 11008, 1, 2, 4, 16, "north_star: W 4096x11008 fp16 2:4:16 x 1 token"),
    "decode_4": ("decode", 4096, 11008, 4, 2, 4, 16, "north_star: W 4096x11008 fp16 2:4:16 x 4 tokens"),
    "decode_8": ("decode", 4096, 11008, 8, 2, 4, 16, "north_star: W 4096x11008 fp16 2:4:16 x 8 tokens"),
    "decode_16": ("decode", 4096, 11008, 16, 2, 4, 16, "north_star: W 4096x11008 fp16 2:4:16 x 16 tokens"),
    "decode_gdim_1": ("decode_g", 4096, 11008, 1, 2, 4, 16, "W 4096x11008 fp16 2:4:16 with the n:m blocks along the outputs (the reference's default orientation) x 1 token: the reduction runs along the group dim, the compressed lines are streamed and expanded in registers"),
    "decode_gdim_4": ("decode_g", 4096, 11008, 4, 2, 4, 16, "the same x 4 tokens"),
    "decode_gdim_8": ("decode_g", 4096, 11008, 8, 2, 4, 16, "the same x 8 tokens"),
    "decode_gdim_16": ("decode_g", 4096, 11008, 16, 2, 4, 16, "the same x 16 tokens"),
    "decode_2_8_1": ("decode", 8192, 8192, 1, 2, 8, 32, "north_star: W 8192x8192 fp16 2:8:32 x 1 token"),
    "decode_2_8_16": ("decode", 8192, 8192, 16, 2, 8, 32, "north_star: W 8192x8192 fp16 2:8:32 x 16 tokens"),
    "decode_up_1": ("decode", 11008, 4096, 1, 2, 4, 16, "W 11008x4096 fp16 2:4:16 x 1 token (the up-projection beside the north_star shape)"),
    "decode_up_16": ("decode", 11008, 4096, 16, 2, 4, 16, "W 11008x4096 fp16 2:4:16 x 16 tokens"),
    "c4_b1": ("w4", 11008, 4096, 1, 2, 4, 1, "configs[3]: W 11008x4096 2:4 + int4 (scale per 128) x 1 token"),
    "c4_b4": ("w4", 11008, 4096, 4, 2, 4, 1, "configs[3]: W 11008x4096 2:4 + int4 (scale per 128) x 4 tokens"),
    "c4_b16": ("w4", 11008, 4096, 16, 2, 4, 1, "configs[3]: W 11008x4096 2:4 + int4 (scale per 128) x 16 tokens"),
    "sparsify_c2": ("sparsify", 4096, 4096, 0, 2, 4, 16, "configs[1]: sparsify W 4096x4096 fp16 to 2:4:16"),
    "sparsify_c3_2_8": ("sparsify", 8192, 8192, 0, 2, 8, 32, "configs[2]: sparsify W 8192x8192 fp16 to 2:8:32"),
}


# committed rocprofv3 --pmc summaries (FETCH_SIZE / WRITE_SIZE) of the workloads that have one
PMC_SUMMARIES = {
    "target_2_4": "spmm_target_2_4_pmc.txt",
    "c5_step": "train_step_c5_kernel_trace_pmc.txt",
    "c2": "spmm_c2_pmc.txt",
    "decode_1": "spmm_decode_1_pmc.txt",
    "c4_b1": "w4_linear_c4_b1_pmc.txt",
    "sparsify_c2": "sparsify_rounds_sparsify_c2_pmc.txt",
}

# measured beside the headline workload in the default run: (workload, steps, warm-up)
ALSO = [("c1", 50, 10), ("ref_f32", 80, 5), ("target_2_4_bf16", 100, 10), ("c2", 240, 10), ("c3_1_8", 40, 5), ("c3_2_8", 40, 5), ("c3_4_8", 40, 5),
        ("decode_1", 50, 10), ("decode_4", 50, 10), ("decode_8", 50, 10), ("decode_16", 50, 10),
        ("decode_gdim_1", 50, 10), ("decode_gdim_16", 50, 10), ("decode_2_8_1", 50, 10), ("decode_2_8_16", 50, 10),
        ("c4_b1", 50, 10), ("c4_b4", 50, 10), ("c4_b16", 50, 10),
        ("sparsify_c2", 100, 5), ("sparsify_c3_2_8", 20, 5), ("c5_step", 20, 3), ("c5_train", 20, 3)]


def profile_traffic(name):
    """HBM bytes per launch from the `traffic_bytes_per_launch:` line of a committed counter summary."""
    if not name:
        return None
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "profiles", name)
    try:
        with open(path) as f:
            for line in f:
                if line.startswith("traffic_bytes_per_launch:"):
                    return float(line.split(":", 1)[1].split()[0])
    except OSError:
        pass
    return None


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


def cpu_baseline_sparsify(M, K, n, m, g, seconds=10.0):
    """The CPU restatement of the reference's sort-and-scan sparsifier (oracle/nmg_oracle.c), single
    thread as the reference's (no OpenMP there), on a slab of whole chunks of the same weight."""
    import math
    import numpy as np
    from oracle import nmg_oracle as O
    cols = math.comb(m, n) * g
    rows = min(M, max(cols, (256 // cols) * cols))
    rng = np.random.default_rng(0)
    W = (rng.standard_normal((rows, K)) * 0.02).astype(np.float16)
    t0 = time.perf_counter()
    it = 0
    while True:
        val, idx, _ = O.sparsify(W, n, m, 1, g, 0)
        it += 1
        if time.perf_counter() - t0 > seconds or it >= 20:
            break
    dt = (time.perf_counter() - t0) / it
    return {
        "value": (W.nbytes + val.nbytes + idx.nbytes) / dt / 1e9,
        "unit": "GB/s",
        "cores": 1,
        "kind": "port",
        "sample": f"{rows}x{K} fp16 slab of the weight ({rows // cols} chunks of {cols} lines), {it} passes",
    }


PROBE_KINDS = ["V_MFMA_F32_32X32X16_F16", "V_MFMA_F32_16X16X32_F16", "V_SMFMAC_F32_32X32X32_F16",
               "V_SMFMAC_F32_16X16X64_F16"]


def matrix_ceiling(iters=4000):
    """What the matrix cores sustain with nothing else going on (nmg_probe_matrix_rate: the
    instructions of a 128 x 128 x 64 slab per wavefront, issued from registers, no memory traffic in
    the loop), per instruction, on all-zero operands (the instruction's issue rate) and on N(0,1)
    operands (what the power limit leaves).  TFLOP/s, dense-equivalent for the sparse instructions."""
    import ctypes
    import torch
    from sten_amd import native

    path = os.path.join(ROOT, "sten_amd", "libnmg_probe.so")
    if not os.path.exists(path):
        raise RuntimeError(f"{path} is missing: build it with `python -m sten_amd.build`")
    lib = ctypes.CDLL(path)
    lib.nmg_probe_matrix_rate.restype = ctypes.c_int
    lib.nmg_probe_matrix_rate.argtypes = [ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p]
    lib.nmg_probe_matrix_rate_flops.restype = ctypes.c_int64
    lib.nmg_probe_matrix_rate_flops.argtypes = [ctypes.c_int, ctypes.c_int]
    dev = "cuda:0"
    torch.manual_seed(0)
    ops = {"random": torch.randn(512 * 1024, device=dev).half(), "zero": torch.zeros(512 * 1024, device=dev).half()}
    out = torch.empty(256 * 1024, dtype=torch.float32, device=dev)
    stream = native.stream_ptr(out.device)
    res = {}
    for kind, name in enumerate(PROBE_KINDS):
        res[name] = {}
        flops = lib.nmg_probe_matrix_rate_flops(kind, iters)
        for label, src in ops.items():
            def launch():
                if lib.nmg_probe_matrix_rate(kind, native.ptr(src), native.ptr(out), iters, stream) != 0:
                    raise RuntimeError(f"nmg_probe_matrix_rate refused kind {kind}")
            settle_end = time.perf_counter() + SETTLE_S
            while time.perf_counter() < settle_end:
                launch()
                torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(3):
                launch()
            e1.record()
            torch.cuda.synchronize()
            res[name][label] = flops / (e0.elapsed_time(e1) / 3 * 1e-3) / 1e12
    return res


def calibrate_copy():
    import torch
    n = 64 * 1024 * 1024
    src = torch.empty(n, dtype=torch.uint8, device="cuda:0").random_(0, 255)
    dst = torch.empty_like(src)
    for _ in range(5):
        dst.copy_(src)
    torch.cuda.synchronize()
    print(json.dumps({"calibration": "device copy", "bytes_read": n, "bytes_written": n}))


def measure(workload, steps, warmup, kernel="auto", variant=-1, eager=False, graph_large=False, copies_arg=0):
    """Run one workload: `warmup` untimed steps, then `steps` timed ones between two synchronisations.
    Returns the row of that workload (times, value, roofline)."""
    import torch
    import sten_amd as sten

    dev = "cuda:0"
    kind, M, K, N, n, m, g, desc = WORKLOADS[workload]
    # Decode shapes are bound by the stream of the weight from HBM, and a weight of 18-54 MB
    # would stay in the 256 MB memory-side cache between two steps: the steps take separate
    # copies of it in turn, more than 512 MiB in all.
    copies, turn = 1, [0]
    torch.manual_seed(0)
    dt = torch.float32 if workload in FP32_WORKLOADS else (torch.bfloat16 if workload in BF16_WORKLOADS else torch.float16)
    W = (torch.randn(M, K) * 0.02).to(dt).to(dev)

    if kind in ("step", "train"):
        # the registered F.linear through the dispatch layer, compressed weight gradient
        lin = torch.nn.Linear(K, M, bias=False).half().to(dev)
        with torch.no_grad():
            lin.weight.copy_(W)
        del W
        sb = sten.SparsityBuilder()
        sb.set_weight("weight", initial_sparsifier=sten.GroupedNMSparsifier(n, m, g, sparse_dim=1, group_dim=0),
                      out_format=sten.GroupedNMTensor)
        sb.set_weight_grad("weight", tmp_format=sten.GroupedNMTensor, out_format=sten.GroupedNMTensor)
        slin = sb.get_sparse_model(lin)
        X = torch.randn(N, K, dtype=torch.float16, device=dev, requires_grad=True)
        dY = torch.randn(N, M, dtype=torch.float16, device=dev)

        if kind == "train":
            opt = torch.optim.SGD(slin.parameters(), lr=1e-3)

            def step():
                opt.zero_grad(set_to_none=True)
                X.grad = None
                slin(X).backward(dY)
                opt.step()
        else:
            def step():
                slin.weight.grad = None
                X.grad = None
                slin(X).backward(dY)
        algo_bytes = 0
    elif kind == "gw_dense":
        from sten_amd.impls import _dense_product
        del W
        X = torch.randn(N, K).half().to(dev)
        dY = torch.randn(N, M).half().to(dev)

        def step():
            return _dense_product("tn", dY, X)
        algo_bytes = 0
    elif kind == "w4":
        # int4 kept values + 2-bit positions + fp16 scales + activations + output
        algo_bytes = M * K // 4 + M * K // 8 + (K // 128) * M * 2 + N * K * 2 + N * M * 2
        copies = copies_arg or -(-ROTATE_BYTES // algo_bytes)
        ws = [sten.SparseMarlinTensor.from_dense(W) for _ in range(copies)]
        del W
        X = torch.randn(N, K).half().to(dev)

        def step():
            turn[0] += 1
            return ws[turn[0] % copies].linear(X)
    elif kind == "sparsify":
        def step():
            return sten.GroupedNMTensor.from_dense(W, n, m, sparse_dim=1, group_size=g, group_dim=0)
        w = step()
        algo_bytes = M * K * 2 + w.val.numel() * 2 + w.idx.numel() * 2
    else:
        # weight values + one int16 index per (line, block) + activations + output
        algo_bytes = M * K * n // m * 2 + M * K // m * 2 + N * K * 2 + N * M * 2
        if kind in ("decode", "decode_g"):
            copies = copies_arg or -(-ROTATE_BYTES // algo_bytes)
        sdim, gdim = (0, 1) if kind == "decode_g" else (1, 0)
        ws = [sten.GroupedNMTensor.from_dense(W, n, m, sparse_dim=sdim, group_size=g, group_dim=gdim)
              for _ in range(copies)]
        for w in ws:
            w.spmm_opt["variant"] = variant
        del W
        if kind == "grad_x":
            X = torch.randn(N, M).half().to(dev)      # upstream gradient dY [tokens, out features]
            rd = 0
        else:
            X = torch.randn(N, K).to(dt).to(dev)
            rd = 1

        def step():
            turn[0] += 1
            return sten.spmm(ws[turn[0] % copies], X, reduce_dim=rd, kernel=kernel)

    # every copy of the weight derives its kernel operands before anything is timed or captured
    for _ in range(max(warmup, copies)):
        step()
    torch.cuda.synchronize()

    # Decode shapes: the K timed steps are recorded once into a HIP graph and replayed, as a
    # serving loop would launch them -- a step lasts 6-13 us on the device, less than one launch
    # through Python and ctypes costs on the host (about 15 us).  The same holds for products on up
    # to 1024 tokens (20-70 us on the device, two kernels and two allocations per call).  The large
    # shapes keep the host busy for less than a step and are launched eagerly (--graph replays
    # them too).
    graph = None
    per = 1                      # steps per timed iteration
    short = kind in ("decode", "decode_g", "w4") or (kind == "fwd" and N <= 1024)
    if (short and not eager) or (graph_large and kind not in ("step", "train", "sparsify", "gw_dense")):
        per = max(GRAPH_STEPS, copies)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            for _ in range(per):
                step()
        graph.replay()
        torch.cuda.synchronize()
    run_once = graph.replay if graph is not None else step

    # Settling: after an idle spell the chip's power management overshoots -- the headline kernel
    # runs at 104 us for its first 2 ms, at 118-125 us for the next 10 ms and at 104 us from then
    # on; the training step needs 60-80 ms to come down from 1.5-1.7 ms to 1.29 ms.  The untimed
    # steps are therefore repeated until SETTLE_S of load have passed, so that the K timed steps
    # see the clocks a workload that keeps running sees.
    gc.collect()
    gc.disable()            # no collector pause of the host between the settling and the timed steps, or inside them
    settle_end = time.perf_counter() + SETTLE_S
    settle_steps = 0
    est = 1.0
    while time.perf_counter() < settle_end:
        ts = time.perf_counter()
        for _ in range(steps):
            run_once()
        torch.cuda.synchronize()
        est = (time.perf_counter() - ts) / steps      # seconds per timed iteration, roughly
        settle_steps += steps * per

    # The timed region: K back-to-back iterations between two synchronisations.  HIP events on the
    # stream the kernels are launched on (torch's current stream) cut the region into groups of
    # consecutive iterations, every group between its own pair of events: event g+1 closes group g
    # and opens group g+1, so the durations add up to the whole region.  A group is one iteration
    # where an iteration lasts 0.5 ms or more and as many as fill about 0.5 ms otherwise (at most a
    # quarter of K): an event marker between two kernels keeps the second from starting under the
    # tail of the first and costs 5-7 us, which a 0.1 ms kernel shows as 7 % (measured: headline
    # 102 us with a marker after every launch, 95 us back to back, 95.5 us in the rocprofv3 kernel
    # trace).  The median over the groups is what the roofline uses -- one stall of the host or the
    # allocator lands in one group and does not move it -- min and max are reported beside it.
    group = max(1, min(int(round(0.5e-3 / max(est, 1e-9))), max(1, steps // 4)))
    bounds = list(range(0, steps, group))
    if len(bounds) > 1 and steps - bounds[-1] < group:
        bounds.pop()                                   # the last group takes the leftover iterations
    bounds.append(steps)
    stream = torch.cuda.current_stream()
    events = [torch.cuda.Event(enable_timing=True) for _ in bounds]
    t0 = time.perf_counter()
    events[0].record(stream)
    for gi in range(len(bounds) - 1):
        for _ in range(bounds[gi], bounds[gi + 1]):
            run_once()
        events[gi + 1].record(stream)
    torch.cuda.synchronize()
    wall = (time.perf_counter() - t0) / (steps * per)
    gc.enable()
    durs = sorted(events[g].elapsed_time(events[g + 1]) / ((bounds[g + 1] - bounds[g]) * per)
                  for g in range(len(bounds) - 1))
    kern_ms = durs[len(durs) // 2] if len(durs) % 2 else 0.5 * (durs[len(durs) // 2 - 1] + durs[len(durs) // 2])
    kern_mean = events[0].elapsed_time(events[-1]) / (steps * per)
    launch = (f"hip graph of {per} steps, replayed once per timed iteration" if graph is not None else "eager")

    traffic = profile_traffic(PMC_SUMMARIES.get(workload))
    traffic_source = (f"profiles/{PMC_SUMMARIES[workload]} (committed rocprofv3 --pmc summary of this workload; "
                      "not measured by this run)") if traffic is not None else None
    row = {"ms_per_step": wall * 1e3, "kernel_ms": kern_ms, "kernel_ms_min": durs[0], "kernel_ms_max": durs[-1],
           "kernel_ms_mean": kern_mean, "timed_groups": len(durs), "steps_per_group": group * per,
           "launch": launch, "desc": desc, "kind": kind, "settle_steps": settle_steps,
           "shape": (M, K, N, n, m, g), "traffic_profile": PMC_SUMMARIES.get(workload)}
    if kind in ("fwd", "grad_x", "step", "train", "gw_dense"):
        dense_flops = 2.0 * M * K * N * (3 if kind in ("step", "train") else 1)
        eff_flops = dense_flops if kind == "gw_dense" else dense_flops * n / m
        achieved = eff_flops / (kern_ms * 1e-3) / 1e12
        peak = PEAK_FP32_TFLOPS if workload in FP32_WORKLOADS else PEAK_FP16_TFLOPS
        row.update({
            "metric": "nmg sparse x dense GEMM TFLOP/s (dense-equiv)",
            "value": dense_flops / wall / 1e12, "unit": "TFLOP/s",
            "effective_tflops": eff_flops / wall / 1e12,
            "roofline": {"bound": "mfma", "achieved": achieved, "peak": peak,
                         "unit": "TFLOP/s", "frac": achieved / peak, "traffic": traffic, "traffic_source": traffic_source,
                         "flops": "effective non-zero (2*M*K*N*n/m); dense-equivalent is m/n times this"},
        })
    else:
        achieved = algo_bytes / (kern_ms * 1e-3) / 1e9
        row.update({
            "metric": "nmg sparsifier GB/s" if kind == "sparsify" else "nmg sparse x dense decode GB/s",
            "value": algo_bytes / wall / 1e9, "unit": "GB/s",
            "algorithmic_bytes": algo_bytes, "weight_copies": copies,
            "roofline": {"bound": "hbm", "achieved": achieved, "peak": PEAK_HBM_GBS, "unit": "GB/s",
                         "frac": achieved / PEAK_HBM_GBS, "traffic": traffic, "traffic_source": traffic_source},
        })
    del step
    torch.cuda.empty_cache()
    return row


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="target_2_4", choices=sorted(WORKLOADS))
    ap.add_argument("--kernel", default="auto")
    ap.add_argument("--variant", type=int, default=-1)
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--no-also", action="store_true", help="headline workload only")
    ap.add_argument("--eager", action="store_true", help="launch every step from Python, decode shapes too")
    ap.add_argument("--graph", action="store_true", help="replay the timed steps from a HIP graph, large shapes too")
    ap.add_argument("--calibrate-copy", action="store_true")
    ap.add_argument("--matrix-ceiling", action="store_true",
                    help="only measure what the matrix cores sustain from registers, per instruction")
    ap.add_argument("--no-ceiling", action="store_true", help="skip that measurement in the default run")
    ap.add_argument("--copies", type=int, default=0,
                    help="decode shapes: separate copies of the weight that the steps take in turn "
                         "(0: as many as exceed 512 MiB, so that no step finds its weight in a cache)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU; multi-GPU runs are not part of this build", file=sys.stderr)
        sys.exit(2)
    if args.calibrate_copy:
        calibrate_copy()
        return
    if args.matrix_ceiling:
        print(json.dumps({"matrix_ceiling_tflops": matrix_ceiling()}))
        return

    row = measure(args.workload, args.steps, args.warmup, args.kernel, args.variant, args.eager, args.graph,
                  args.copies)
    kind, M, K, N, n, m, g, desc = WORKLOADS[args.workload]
    out = {
        "metric": row["metric"], "value": row["value"], "unit": row["unit"],
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": row["ms_per_step"],
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32" if args.workload in FP32_WORKLOADS else ("bf16" if args.workload in BF16_WORKLOADS else "f16"), "data": "synthetic",
        "config": {"workload": desc, "kernel": args.kernel, "variant": args.variant, "launch": row["launch"],
                   "settle": f"{row['settle_steps']} more untimed steps ({SETTLE_S * 1e3:.0f} ms of load) between the "
                             "warm-up and the timed steps: the clocks dip for 10-60 ms after an idle spell",
                   "kernel_ms": row["kernel_ms"], "kernel_ms_min": row["kernel_ms_min"],
                   "kernel_ms_max": row["kernel_ms_max"],
                   "kernel_ms_mean": row["kernel_ms_mean"], "timed_groups": row["timed_groups"],
                   "steps_per_group": row["steps_per_group"],
                   "timing": "the timed steps are cut into groups by HIP events (a group lasts about 0.5 ms, one step "
                             "where a step is longer); kernel_ms = median over the groups of duration / steps in "
                             "the group, min / max beside it, kernel_ms_mean = first to last event / steps; "
                             "ms_per_step = wall clock of the timed steps / steps"},
        "roofline": row["roofline"],
    }
    for key in ("effective_tflops", "algorithmic_bytes", "weight_copies"):
        if key in row:
            out["config"][key] = row[key]
    if kind in ("fwd", "grad_x") and not args.no_ceiling and args.workload not in FP32_WORKLOADS:
        # The instruction of the dominant kernel, issued from registers with nothing else going on:
        # the 2.5 PFLOP/s behind `peak` assume 2.4 GHz, which random operands do not sustain, and the
        # 32x32x32 sparse instruction stays below its nominal rate even on zeros.
        ceil = matrix_ceiling()
        sparse_cores = args.kernel in ("auto", "smfmac") and kind == "fwd" and (n, m) in ((2, 4), (1, 4), (1, 8), (2, 8))
        inst = "V_SMFMAC_F32_32X32X32_F16" if sparse_cores else "V_MFMA_F32_32X32X16_F16"
        issued = 2.0 * M * K * N / (row["kernel_ms"] * 1e-3) / 1e12      # flops the instruction stream carries
        out["roofline"]["ceiling"] = {
            "instruction": inst, "unit": "TFLOP/s issued (dense-equivalent for the sparse instruction)",
            "random_operands": ceil[inst]["random"], "zero_operands": ceil[inst]["zero"],
            "achieved_issued": issued, "frac_of_random_ceiling": issued / ceil[inst]["random"]}
        out["config"]["matrix_ceiling_tflops"] = ceil
    if args.workload == "target_2_4" and not args.no_also:
        also = {}
        for name, steps, warmup in ALSO:
            r = measure(name, steps, warmup)
            also[name] = {"us": r["kernel_ms"] * 1e3, "us_min": r["kernel_ms_min"] * 1e3,
                          "us_max": r["kernel_ms_max"] * 1e3, "us_mean": r["kernel_ms_mean"] * 1e3,
                          "groups": r["timed_groups"], "steps_per_group": r["steps_per_group"], "value": r["value"], "unit": r["unit"],
                          "frac": r["roofline"]["frac"], "bound": r["roofline"]["bound"]}
        out["config"]["also"] = also
    if not args.no_cpu and args.workload in ("c1", "c2", "target_2_4"):
        out["cpu_baseline"] = cpu_baseline(M, K, N, n, m, g)
    if not args.no_cpu and kind == "sparsify":
        out["cpu_baseline"] = cpu_baseline_sparsify(M, K, n, m, g)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
