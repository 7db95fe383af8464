#!/usr/bin/env python3
"""Benchmark of the quantized-inference custom calls on one MI355X.

A *step* is one pass of the decode hot path over the configuration-2 workload: the weight-only
s4 group-128 dequantize-dot [M,8192] x [8192,28672] (+bias, SiLU) for M = 1, 8, 32 and 64, one
custom call each, all through the library's XLA FFI handler symbols.  Inputs are synthetic, of
the benchmark's shapes and distributions, and resident in HBM before the timed region.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--skip-other] [--skip-cpu]

Prints ONE JSON line: `value` = algorithmic bytes of a step / wall time per step (GB/s), over exactly
K steps between two synchronisations, after the W warm-up steps and `settle_steps` further untimed
steps that bring the clocks of a GPU that has idled back up;
`roofline` = the step's slowest kernel against the 8 TB/s HBM peak, timed with events on the
launch stream (every per-kernel `ms` is the median over 21 event-bracketed batches of back-to-back
launches, `ms_best` the fastest batch); `cpu_baseline` = the CPU oracle on the same workload; `kernels` = every kernel of
the step; `other_configs` = the four other configurations, each with a `roofline` and a
`cpu_baseline` of its own (the oracle on a stated sample of the same shape); `launch_floor_us` =
what a kernel that does nothing costs per launch in the same back-to-back measurement.

`traffic` figures (HBM bytes per launch from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs) are read
from profiles/hbm_traffic_per_launch.md, which names the hash of the kernel sources it was measured
on; when the sources here hash differently the figures are stale and `traffic` is null.
"""
import argparse
import hashlib
import json
import os
import re
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E
HBM_PEAK_XLA_GBS = 6810.0      # what XLA's own device file assumes (mi350.txtpb:28)
MFMA_PEAK_TFLOPS = {"bf16": 2500.0, "fp8": 5000.0}
TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "hbm_traffic_per_launch.md")


def kernel_sources_hash():
    """sha256 over the device sources and headers, in path order: identifies what a profile measured."""
    h = hashlib.sha256()
    csrc = os.path.join(ROOT, "xla_amd", "csrc")
    files = sorted(os.path.join(csrc, f) for f in os.listdir(csrc) if f.endswith((".hip", ".h")))
    for f in files:
        h.update(os.path.basename(f).encode() + b"\0")
        h.update(open(f, "rb").read())
    return h.hexdigest()


def measured_traffic():
    """workload -> HBM bytes per launch from the committed profile summary; {} when that summary
    was measured on other kernel sources (or is missing)."""
    try:
        text = open(TRAFFIC_PROFILE).read()
    except OSError:
        return {}
    m = re.search(r"kernel sources sha256: `?([0-9a-f]{64})`?", text)
    if not m or m.group(1) != kernel_sources_hash():
        return {}
    table = {}
    for line in text.splitlines():
        cells = [c.strip() for c in line.strip().strip("|").split("|")]
        if len(cells) >= 5 and re.fullmatch(r"\d+", cells[-1]):
            table[cells[0]] = int(cells[-1])
    return table


K2, N2, GROUP2 = 8192, 28672, 128
MS2 = (1, 8, 32, 64)


def c2_bytes(m):
    return K2 * N2 // 2 + (K2 // GROUP2) * N2 * 2 + N2 * 2 + m * K2 * 2 + m * N2 * 2


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--skip-other", action="store_true", help="only the headline workload")
    ap.add_argument("--skip-cpu", action="store_true", help="no CPU baseline leg")
    ap.add_argument("--reps", type=int, default=20, help="launches per event-timed batch")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run a plain 256 MiB device copy a few times, so that a rocprofv3 --pmc run of this "
                         "command shows what FETCH_SIZE / WRITE_SIZE read for a known number of bytes")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU (the path shards by output channels with no "
                 "exchange step, so more GPUs would only run independent column slices); --gpus %d is not supported" % args.gpus)

    import torch
    from xla_amd import ffi, ops

    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible; the kernels have no CPU fallback")
    dev = torch.device("cuda:0")
    torch.manual_seed(0)

    BATCHES = 21

    def ev_time(fn, reps, warm=1):
        """Device time of fn() per launch: `BATCHES` batches of `reps` back-to-back launches, each batch
        bracketed by events on the launch stream.  Returns (median, best) of the batch means in ms."""
        for _ in range(warm):
            fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        ts = []
        for _ in range(BATCHES):
            e0.record()
            for _ in range(reps):
                fn()
            e1.record()
            e1.synchronize()
            ts.append(e0.elapsed_time(e1) / reps)
        ts.sort()
        return ts[len(ts) // 2], ts[0]  # ms

    # ---- what a plain copy reaches on this machine (context for every HBM fraction below) ------
    ca = torch.empty(1 << 30, dtype=torch.uint8, device=dev)
    cb = torch.empty_like(ca)
    st = torch.cuda.current_stream().cuda_stream
    copy_ms, _ = ev_time(lambda: ffi.debug_stream(cb.data_ptr(), ca.data_ptr(), ca.numel(), st), 4, warm=3)
    copy_gbs = 2 * ca.numel() / (copy_ms * 1e-3) / 1e9
    read_ms, _ = ev_time(lambda: ffi.debug_stream(None, ca.data_ptr(), ca.numel(), st), 4, warm=3)
    read_gbs = ca.numel() / (read_ms * 1e-3) / 1e9
    if args.calibrate_copy:
        for _ in range(3):
            cb[:1 << 28].copy_(ca[:1 << 28])     # 256 MiB read + 256 MiB written per launch
        torch.cuda.synchronize()
    del ca, cb

    # ---- configuration 2 on the device -------------------------------------------------------
    w_packed = torch.randint(0, 256, (K2 * N2 // 2,), dtype=torch.uint8, device=dev)   # nibbles ~U{-8..7}
    scales = torch.empty((K2 // GROUP2, N2), device=dev).uniform_(1e-3, 2e-2).to(torch.bfloat16)
    bias = torch.randn((N2,), device=dev).to(torch.bfloat16)
    calls = []
    for m in MS2:
        lhs = torch.randn((m, K2), device=dev).to(torch.bfloat16)
        calls.append(ops.dequant_dot(lhs, w_packed, scales, bias, weight_dtype="s4", weight_shape=(K2, N2),
                                     epilogue="BIAS_SILU", dequant_type="bf16", build_only=True))
    for c in calls:
        c.frame.host.stream = torch.cuda.current_stream().cuda_stream
    step = ffi.Replay([(c.target, c.frame) for c in calls])

    step.run(max(args.warmup, 1))
    # The GPU has idled while the operands were made and its clocks take tens of milliseconds of work to
    # come back: more untimed steps (about 40 ms) until the rate is the steady one that a serving loop
    # sees.  The timed region below is still exactly args.steps steps between two synchronisations.
    settle_steps = 300 if args.steps >= 10 else 0   # (profiling runs with a handful of steps skip it)
    step.run(settle_steps)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    step.run(args.steps)
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms_per_step = wall * 1e3 / args.steps
    step_bytes = sum(c2_bytes(m) for m in MS2)
    value = step_bytes / (ms_per_step * 1e-3) / 1e9

    traffic = measured_traffic()
    kernels = []
    for m, c in zip(MS2, calls):
        one = ffi.Replay([(c.target, c.frame)])
        ms, ms_best = ev_time(lambda: one.run(args.reps), 1)   # a batch = args.reps native replays
        ms, ms_best = ms / args.reps, ms_best / args.reps
        c.run()
        gbs = c2_bytes(m) / (ms * 1e-3) / 1e9
        kernels.append({"workload": "C2 M=%d" % m, "kernel": ffi.last_kernel(), "ms": round(ms, 5), "ms_best": round(ms_best, 5),
                        "bytes": c2_bytes(m), "GB/s": round(gbs, 1), "frac": round(gbs / HBM_PEAK_GBS, 4),
                        "TFLOP/s": round(2 * m * K2 * N2 / (ms * 1e-3) / 1e12, 2),
                        "traffic": traffic.get("C2 M=%d" % m)})
    dom = max(kernels, key=lambda k: k["ms"])
    roofline = {"bound": "hbm", "kernel": dom["kernel"], "workload": dom["workload"],
                "achieved": dom["GB/s"], "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": dom["frac"],
                "frac_of_xla_device_file_peak": round(dom["GB/s"] / HBM_PEAK_XLA_GBS, 4),
                "traffic": dom["traffic"], "launch_ms": dom["ms"], "launch_ms_best": dom["ms_best"],
                "timing": "median of %d event-bracketed batches of %d launches" % (BATCHES, args.reps),
                "algorithmic_bytes": dom["bytes"],
                "device_copy_GB/s": round(copy_gbs, 1), "device_read_GB/s": round(read_gbs, 1),
                "frac_of_device_read_rate": round(dom["GB/s"] / read_gbs, 4)}

    # ---- the floor under every one-kernel figure: a kernel that does nothing, launched the same way
    st = torch.cuda.current_stream().cuda_stream
    floor_ms = ev_time(lambda: ffi.launch_empty(st, 50, 256), 4, warm=2)[0] / 50

    # ---- the other four configurations, each with its own roofline and CPU baseline ---------------
    import numpy as np
    other = []
    cpu_legs = {}   # workload -> function returning the cpu_baseline dict (run after the GPU part)
    if not args.skip_other:
        def entry(key, name, call, bytes_, flops, bound, dtype=None):
            # replayed natively from the prebuilt call frame, like the C2 calls; the half-millisecond
            # kernels get 20 ms of launches to settle the clocks before timing and 5 launches per batch
            call.frame.host.stream = torch.cuda.current_stream().cuda_stream
            one = ffi.Replay([(call.target, call.frame)])
            n = max(3, args.reps // 4) if bound == "mfma" else args.reps
            one.run(40 if bound == "mfma" else 2)
            ms, ms_best = ev_time(lambda: one.run(n), 1, warm=1)
            ms, ms_best = ms / n, ms_best / n
            call.run()   # (sets the kernel name this thread reads below)
            e = {"workload": name, "key": key, "kernel": ffi.last_kernel(), "ms": round(ms, 5), "ms_best": round(ms_best, 5),
                 "GB/s": round(bytes_ / (ms * 1e-3) / 1e9, 1)}
            e["frac_hbm"] = round(e["GB/s"] / HBM_PEAK_GBS, 4)
            if flops:
                e["TFLOP/s"] = round(flops / (ms * 1e-3) / 1e12, 2)
                if dtype:
                    e["frac_mfma"] = round(e["TFLOP/s"] / MFMA_PEAK_TFLOPS[dtype], 4)
            e["bound"] = bound
            if bound == "hbm":
                e["roofline"] = {"bound": "hbm", "achieved": e["GB/s"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
                                 "frac": e["frac_hbm"], "traffic": traffic.get(key), "algorithmic_bytes": bytes_}
            else:
                e["roofline"] = {"bound": "mfma", "achieved": e["TFLOP/s"], "peak": MFMA_PEAK_TFLOPS[dtype],
                                 "unit": "TFLOP/s", "frac": e["frac_mfma"], "traffic": traffic.get(key),
                                 "algorithmic_flops": flops}
            e["cpu_baseline"] = None
            other.append(e)

        # C2's weights at a prefill-sized token count (informational: the tiled s4 kernel)
        lhs2k = torch.randn((2048, K2), device=dev).to(torch.bfloat16)
        entry("C2 prefill", "C2 weights, 2048 tokens (s4 prefill)",
              ops.dequant_dot(lhs2k, w_packed, scales, bias, weight_dtype="s4", weight_shape=(K2, N2),
                              epilogue="BIAS_SILU", dequant_type="bf16", build_only=True),
              c2_bytes(2048), 2 * 2048 * K2 * N2, "mfma", "bf16")
        del lhs2k
        # C1: s8 per-channel decode
        a = torch.randn((16, 4096), device=dev).to(torch.bfloat16)
        w8 = torch.randint(-127, 128, (4096, 4096), dtype=torch.int8, device=dev)
        sc = torch.empty((4096,), device=dev).uniform_(1e-3, 1e-2)
        entry("C1", "C1 s8 [16,4096]x[4096,4096]", ops.dequant_dot(a, w8, sc, build_only=True),
              4096 * 4096 + 2 * 16 * 4096 * 2 + 4096 * 4, 2 * 16 * 4096 * 4096, "hbm")
        # a mixture-of-experts decode step: 32 tokens sorted by expert over 8 experts' s8 weights
        # (ragged dot, group sizes read on the device; informational -- not one of the five configurations)
        ar = torch.randn((32, 4096), device=dev).to(torch.bfloat16)
        wr = torch.randint(-127, 128, (8, 4096, 4096), dtype=torch.int8, device=dev)
        sr = torch.empty((8, 4096), device=dev).uniform_(1e-3, 1e-2)
        gsz = torch.tensor([4, 4, 4, 4, 4, 4, 4, 4], dtype=torch.int32, device=dev)
        entry("ragged", "ragged s8 [32,4096] x [8,4096,4096], 8 groups of 4 rows",
              ops.dequant_dot(ar, wr, sr, scale_group_size=0, group_sizes=gsz, build_only=True),
              8 * 4096 * 4096 + 8 * 4096 * 4 + 32 * 4096 * 2 + 32 * 4096 * 2, 2 * 32 * 4096 * 4096, "hbm")
        del wr
        # C4: RMSNorm + rowwise fp8 quantize
        x = torch.randn((16384, 8192), device=dev)
        x = torch.where(torch.rand_like(x) < 0.01, x * 50, x).to(torch.bfloat16)
        g = torch.empty((8192,), device=dev).uniform_(0.5, 1.5).to(torch.bfloat16)
        entry("C4", "C4 rmsnorm+quantize [16384,8192]", ops.rowwise_quantize_fp8(x, g, build_only=True),
              16384 * 8192 * 3 + 16384 * 4 + 8192 * 2, 0, "hbm")
        del x
        # C3: fp8 scaled dot + bias + GELU
        a8 = (torch.randn((8192, 8192), device=dev) * 64).clamp(-448, 448).to(torch.float8_e4m3fn)
        b8 = (torch.randn((8192, 8192), device=dev) * 64).clamp(-448, 448).to(torch.float8_e4m3fn)
        s64 = torch.full((), 1 / 64, device=dev)
        b3 = torch.randn((8192,), device=dev).to(torch.bfloat16)
        c3_bytes, c3_flops = 2 * 8192 * 8192 + 8192 * 8192 * 2 + 8192 * 2, 2 * 8192 ** 3
        entry("C3", "C3 fp8 [8192,8192]x[8192,8192] (rhs [K,N], as in the HLO)",
              ops.fp8_scaled_dot(a8, b8, s64, s64, b3, epilogue="BIAS_GELU", build_only=True),
              c3_bytes, c3_flops, "mfma", "fp8")
        entry("C3 nk", "C3 fp8, rhs given as [N,K]",
              ops.fp8_scaled_dot(a8, b8, s64, s64, b3, epilogue="BIAS_GELU", rhs_contracting_dim=1,
                                 build_only=True),
              c3_bytes, c3_flops, "mfma", "fp8")
        # the reference's own test spelling: every op bf16-typed (gemm_rewriter_fp8_test.cc:1110-1141);
        # power-of-two scales keep it on the tiled kernel, with an extra rounding per epilogue op
        s64b = torch.full((), 1 / 64, device=dev)
        entry("C3 bf16-typed", "C3 fp8 with bf16-typed dequantise, dot and epilogue ops",
              ops.fp8_scaled_dot(a8, b8, s64b, s64b, b3, epilogue="BIAS_GELU", dequant_type="bf16", dot_type="bf16",
                                 epilogue_type="bf16", build_only=True),
              c3_bytes, c3_flops, "mfma", "fp8")
        # the same call with GELU from its closed form (opt-in: the far negative tail then differs
        # from the reference's own cancellation by more than 2 bf16 ulp of results below 1e-5)
        ffi.set_option("tiled_epilogue", 1)
        try:
            entry("C3 closed form", "C3 fp8 (rhs [K,N]), opt-in closed-form GELU: fails the 2-ulp rule in the far tail",
                  ops.fp8_scaled_dot(a8, b8, s64, s64, b3, epilogue="BIAS_GELU", build_only=True),
                  c3_bytes, c3_flops, "mfma", "fp8")
        finally:
            ffi.set_option("tiled_epilogue", 0)
        del a8, b8
        # the decode end of the same call: 16 rows of a against an f8 matrix of C2's shape, streamed once
        # (informational -- not one of the five configurations)
        a8d = (torch.randn((16, K2), device=dev) * 64).clamp(-448, 448).to(torch.float8_e4m3fn)
        b8d = (torch.randn((K2, N2), device=dev) * 64).clamp(-448, 448).to(torch.float8_e4m3fn)
        b3d = torch.randn((N2,), device=dev).to(torch.bfloat16)
        f8d_bytes = K2 * N2 + 16 * K2 + 16 * N2 * 2 + N2 * 2
        entry("fp8 decode", "fp8 [16,8192]x[8192,28672] + bias + GELU (rhs [K,N])",
              ops.fp8_scaled_dot(a8d, b8d, s64, s64, b3d, epilogue="BIAS_GELU", build_only=True),
              f8d_bytes, 2 * 16 * K2 * N2, "hbm")
        # every op bf16-typed and scales that are no powers of two: each scaled operand is rounded to bf16
        s03 = torch.full((), 0.30078125, device=dev)
        entry("fp8 decode bf16-typed", "fp8 [16,8192]x[8192,28672] + bias + GELU, bf16-typed ops, scales 77/256 (operands rounded to bf16)",
              ops.fp8_scaled_dot(a8d, b8d, s03, s03, b3d, epilogue="BIAS_GELU", dequant_type="bf16", dot_type="bf16",
                                 epilogue_type="bf16", build_only=True),
              f8d_bytes, 2 * 16 * K2 * N2, "hbm")
        b8dt = b8d.view(torch.uint8).t().contiguous()
        del b8d
        entry("fp8 decode nk", "fp8 [16,8192]x[28672,8192] + bias + GELU (rhs [N,K])",
              ops.fp8_scaled_dot(a8d, b8dt, s64, s64, b3d, epilogue="BIAS_GELU", rhs_contracting_dim=1, build_only=True),
              f8d_bytes, 2 * 16 * K2 * N2, "hbm")
        del a8d, b8dt
        # C5: batched s8 per-channel prefill
        a5 = torch.randn((8, 512, 4096), device=dev).to(torch.bfloat16)
        w5 = torch.randint(-127, 128, (8, 4096, 14336), dtype=torch.int8, device=dev)
        s5 = torch.empty((8, 14336), device=dev).uniform_(1e-3, 1e-2)
        entry("C5", "C5 s8 [8,512,4096]x[8,4096,14336]", ops.dequant_dot(a5, w5, s5, scale_group_size=0, build_only=True),
              8 * (4096 * 14336 + 512 * 4096 * 2 + 14336 * 4 + 512 * 14336 * 2),
              2 * 8 * 512 * 4096 * 14336, "mfma", "bf16")
        # the same experts with routing: 4096 tokens sorted by expert, uneven group sizes read on the device
        # (ragged dot as a grouped GEMM; informational -- not one of the five configurations)
        a5r = torch.randn((4096, 4096), device=dev).to(torch.bfloat16)
        gsz5 = torch.tensor([1024, 0, 512, 512, 100, 924, 512, 512], dtype=torch.int32, device=dev)
        entry("ragged prefill", "ragged s8 [4096,4096] x [8,4096,14336], groups of 1024/0/512/512/100/924/512/512 rows",
              ops.dequant_dot(a5r, w5, s5, scale_group_size=0, group_sizes=gsz5, build_only=True),
              8 * (4096 * 14336 + 14336 * 4) + 4096 * 4096 * 2 + 4096 * 14336 * 2,
              2 * 4096 * 4096 * 14336, "mfma", "bf16")
        # weights stored [N,K] (the contracting dimension minor, rhs_contracting_dim = 1; informational):
        # C5's experts through the tiled kernel's [N,K] loader, C2's matrix at 8 tokens through the
        # streaming kernel that takes K-minor rows as matrix operands
        w5t = w5.transpose(1, 2).contiguous()
        del w5, a5r
        entry("C5 k-minor", "C5 with the weights stored [8,14336,4096]",
              ops.dequant_dot(a5, w5t, s5, scale_group_size=0, rhs_contracting_dim=1, build_only=True),
              8 * (4096 * 14336 + 512 * 4096 * 2 + 14336 * 4 + 512 * 14336 * 2),
              2 * 8 * 512 * 4096 * 14336, "mfma", "bf16")
        del a5, w5t
        w2t = torch.randint(0, 256, (N2, K2 // 2), dtype=torch.uint8, device=dev)
        s2t = torch.empty((N2, K2 // GROUP2), device=dev).uniform_(1e-3, 2e-2).to(torch.bfloat16)
        lhs8 = torch.randn((8, K2), device=dev).to(torch.bfloat16)
        entry("C2 k-minor", "C2 at 8 tokens with the weights stored [28672,8192], scales [28672,64]",
              ops.dequant_dot(lhs8, w2t, s2t, bias, weight_dtype="s4", weight_shape=(N2, K2), epilogue="BIAS_SILU",
                              dequant_type="bf16", scale_group_size=GROUP2, rhs_contracting_dim=1, build_only=True),
              c2_bytes(8), 2 * 8 * K2 * N2, "hbm")
        del w2t, s2t, lhs8

    # ---- CPU baselines: the oracle on the same workload, or on a stated sample of it ------------
    cpu = None
    if not args.skip_cpu:
        from oracle import oracle
        from xla_amd import dtypes, workloads
        cores = oracle.num_threads()
        wl = workloads.c2_s4_group(M=max(MS2), K=K2, N=N2)  # weights, scales, bias: generated once
        t_cpu, b_cpu = 0.0, 0
        for m in MS2:
            lhs = np.ascontiguousarray(wl["lhs"][:m])
            t1 = time.perf_counter()
            oracle.dequant_dot(lhs, wl["weights_packed"], 4, wl["scales"], "bf16", "bf16",
                               bias=wl["bias"], group=GROUP2, epilogue="silu")
            t_cpu += time.perf_counter() - t1
            b_cpu += c2_bytes(m)
        cpu = {"value": round(b_cpu / t_cpu / 1e9, 3), "unit": "GB/s", "cores": cores,
               "kind": "port",
               "sample": "C2 at M=1,8,32,64 on all %d output channels (full K), %.2f s of "
                         "CPU time; scalar restatement of the XLA CPU backend's op-by-op semantics, "
                         "OpenMP over output channels" % (N2, t_cpu)}
        del wl

        def timed(fn):
            t1 = time.perf_counter()
            fn()
            return time.perf_counter() - t1

        def base(value, unit, sample):
            return {"value": value, "unit": unit, "cores": cores, "kind": "port", "sample": sample}

        by_key = {e["key"]: e for e in other}
        if "C2 k-minor" in by_key:   # the same arithmetic on re-laid-out weights
            by_key["C2 k-minor"]["cpu_baseline"] = base(cpu["value"], "GB/s", "as C2 (the oracle reads the weights [K,N]): " + cpu["sample"])
        if "C1" in by_key:
            w = workloads.c1_s8_channel()
            t = timed(lambda: oracle.dequant_dot(w["lhs"], w["weights"], 8, w["scales"], "f32", "f32"))
            by_key["C1"]["cpu_baseline"] = base(round(w["algorithmic_bytes"] / t / 1e9, 3), "GB/s",
                                                "the whole [16,4096]x[4096,4096] workload, %.2f s" % t)
        if "C2 prefill" in by_key:
            w = workloads.c2_s4_group(M=64, K=K2, N=4096)
            t = timed(lambda: oracle.dequant_dot(w["lhs"], w["weights_packed"], 4, w["scales"], "bf16", "bf16",
                                                 bias=w["bias"], group=GROUP2, epilogue="silu"))
            by_key["C2 prefill"]["cpu_baseline"] = base(round(2 * 64 * K2 * 4096 / t / 1e12, 4), "TFLOP/s",
                                                        "64 of 2048 tokens on 4096 of %d channels (full K), %.2f s" % (N2, t))
        if "ragged" in by_key:
            w = workloads.ragged_s8_experts(M=32, K=4096, N=4096, groups=8, sizes=[4] * 8)
            t = timed(lambda: oracle.ragged_dequant_dot(w["lhs"], w["weights"], 8, w["scales"], "f32", "f32",
                                                        w["group_sizes"]))
            by_key["ragged"]["cpu_baseline"] = base(round(w["algorithmic_bytes"] / t / 1e9, 3), "GB/s",
                                                    "the whole workload, %.2f s" % t)
        if "C4" in by_key:
            w = workloads.c4_quantize(rows=8192, cols=8192)
            t = timed(lambda: oracle.rmsnorm_quantize_fp8(w["x"], w["gamma"], eps=1e-6))
            by_key["C4"]["cpu_baseline"] = base(round(w["algorithmic_bytes"] / t / 1e9, 3), "GB/s",
                                                "8192 of 16384 rows (all 8192 columns), %.2f s" % t)
        c3_keys = [k for k in ("C3", "C3 nk", "C3 bf16-typed") if k in by_key]
        if c3_keys:
            w = workloads.c3_fp8(1024, 8192, 2048)
            t = timed(lambda: oracle.fp8_scaled_dot(w["a"], w["b"], w["a_scale"], w["b_scale"], bias=w["bias"],
                                                    epilogue="gelu_tanh"))
            for k in c3_keys:
                by_key[k]["cpu_baseline"] = base(round(2 * 1024 * 8192 * 2048 / t / 1e12, 4), "TFLOP/s",
                                                 "1024 of 8192 rows x 2048 of 8192 channels (full K), f32-typed ops, %.2f s" % t)
        f8d_keys = [k for k in ("fp8 decode", "fp8 decode nk", "fp8 decode bf16-typed") if k in by_key]
        if f8d_keys:
            w = workloads.c3_fp8(16, K2, 4096)
            t = timed(lambda: oracle.fp8_scaled_dot(w["a"], w["b"], w["a_scale"], w["b_scale"], bias=w["bias"],
                                                    epilogue="gelu_tanh"))
            for k in f8d_keys:
                by_key[k]["cpu_baseline"] = base(round(w["algorithmic_bytes"] / t / 1e9, 3), "GB/s",
                                                 "4096 of %d channels (16 rows, full K; the oracle reads the rhs [K,N]), %.2f s" % (N2, t))
        if "C5" in by_key:
            w = workloads.c5_s8_batched(B=1, M=64, K=4096, N=14336)
            t = timed(lambda: oracle.dequant_dot(w["lhs"], w["weights"], 8, w["scales"], "f32", "f32"))
            by_key["C5"]["cpu_baseline"] = base(round(2 * 64 * 4096 * 14336 / t / 1e12, 4), "TFLOP/s",
                                                "1 of 8 batches, 64 of 512 tokens (full K and N), %.2f s" % t)
            if "C5 k-minor" in by_key:   # the same arithmetic on re-laid-out weights
                by_key["C5 k-minor"]["cpu_baseline"] = base(round(2 * 64 * 4096 * 14336 / t / 1e12, 4), "TFLOP/s",
                                                            "as C5 (the oracle reads the weights [K,N]), %.2f s" % t)
            if "ragged prefill" in by_key:   # the same arithmetic per row and expert
                by_key["ragged prefill"]["cpu_baseline"] = base(round(2 * 64 * 4096 * 14336 / t / 1e12, 4), "TFLOP/s",
                                                                "64 rows of one expert (full K and N), %.2f s" % t)

    out = {
        "metric": "quant-dot HBM GB/s on the s4 group-128 decode dequantize-dot (% of MI355X roofline) "
                  "next to the XLA-CPU-semantics oracle",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "settle_steps": settle_steps,
        "ms_per_step": round(ms_per_step, 5), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": "C2: bf16 [M,8192] x s4 [8192,28672] group-128 bf16 scales + bias + SiLU, "
                               "M in {1,8,32,64}, one custom call per M per step",
                   "boundary": "XLA FFI handler xla_amd_dequant_dot via native call-frame replay"},
        "roofline": roofline, "cpu_baseline": cpu, "kernels": kernels, "other_configs": other,
        "frac_of_hbm_peak_whole_step": round(value / HBM_PEAK_GBS, 4),
        "launch_floor_us": round(floor_ms * 1e3, 3),
        "kernel_sources_sha256": kernel_sources_hash(),
        "traffic_source": os.path.relpath(TRAFFIC_PROFILE, ROOT) if traffic else None,
    }
    print(json.dumps(out))


if __name__ == "__main__":
    main()
