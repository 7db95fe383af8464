"""The handlers declare XLA_FFI_HANDLER_TRAITS_COMMAND_BUFFER_COMPATIBLE: XLA may record them
into a command buffer (a HIP graph) once and replay it step after step
(xla/ffi/api/c_api.h:428-437, 528-533; xla/backends/gpu/runtime/custom_call_thunk.cc:659-666).
That only works if a call enqueues the same kernels for the same shapes, never synchronises,
never reads device data on the host and allocates nothing.  Here decode steps of every kind
(two workgroups per strip handing over inside the kernel, K-slices adding up inside the kernel,
K-slices with a second launch, more than 64 tokens as several launches, prefill tiles split along K), a quantize and scaled dots
are captured into one graph through the native call-frame replay; the operands are then changed
in place, and every replay must equal what eager calls give on the same data AND what the oracle
computes from it."""
import sys

import numpy as np
import pytest
import torch

from tests.gpu_util import check_dot, dev_bf16, dev_f32, dev_s8, dev_u8, host_bf16
from tests.test_gpu_dequant_dot import compare
from tests.test_gpu_fp8_dot import floor_for as fp8_floor_for
from xla_amd import dtypes, ffi, ops, workloads

pytestmark = pytest.mark.gpu


def say(msg):
    print("[case] " + msg, flush=True)
    sys.stdout.flush()


def test_handlers_replay_from_a_hip_graph(oracle):
    say("graph capture of dequant_dot (pair hand-over, s8 in-kernel slices, split-K + finalize, 70 tokens, split tiles), "
        "rowwise_quantize_fp8, fp8_scaled_dot (bf16 and f8 + amax)")
    dev = torch.device("cuda:0")
    rng = np.random.default_rng(7)
    # the decode calls, each with the numpy workload the oracle reads
    dots = []
    for w, opts in ((workloads.c2_s4_group(M=8, K=2048, N=1024), {"dequant_dot_pair": 1}),  # pair hand-over
                    (workloads.c2_s4_group(M=20, K=2048, N=768, group=64), {"dequant_dot_slices": 2}),  # finalize launch
                    (workloads.c2_s4_group(M=70, K=1024, N=512), {}),                     # 64 + 6 tokens
                    (workloads.c1_s8_channel(M=16, K=2048, N=1024), {}),                  # slices inside the kernel
                    (workloads.c5_s8_batched(B=1, M=300, K=2048, N=700), {"dequant_dot_kernel": 3}),   # tiles split along K
                    (workloads.c2_s4_group(M=8, K=2048, N=512), {"nk": 1})):              # weights stored [N,K], K-slices
        nk = opts.pop("nk", 0)
        v = workloads.k_minor(w) if nk else w   # (the oracle keeps reading the [K,N] arrays)
        lhs = dev_bf16(v["lhs"])
        wt = dev_u8(v["weights_packed"]) if v["weight_dtype"] == "s4" else dev_s8(v["weights"])
        sc = dev_bf16(v["scales"]) if v["scales"].dtype == np.uint16 else dev_f32(v["scales"])
        bias = dev_bf16(v["bias"]) if v.get("bias") is not None else None
        for k, val in opts.items():
            ffi.set_option(k, val)
        try:
            call = ops.dequant_dot(lhs, wt, sc, bias, weight_dtype=v["weight_dtype"], weight_shape=v["weight_shape"],
                                   epilogue=v["epilogue"], dequant_type=v["dequant_type"],
                                   scale_group_size=0 if v["group"] == v["lhs"].shape[-1] else v["group"],
                                   rhs_contracting_dim=nk, build_only=True)
            call.run()   # eager warm-up with the options that pick the kernel; the frame keeps its scratch
            torch.cuda.synchronize()
            kern = ffi.last_kernel()
        finally:
            for k in opts:
                ffi.set_option(k, 0)
        dots.append((w, lhs, call, opts, kern))
    assert dots[0][4] == "dequant_dot_decode_s4x_m16_pair", dots[0][4]
    assert dots[2][4].endswith(":x64"), dots[2][4]
    assert dots[3][4].startswith("dequant_dot_decode_s8x_"), dots[3][4]
    assert dots[4][4] == "dequant_dot_tiled_s8_factored:tail2", dots[4][4]
    assert dots[5][4] == "dequant_dot_nk_s4_m16_rounded", dots[5][4]

    q4 = workloads.c4_quantize(rows=256, cols=1024)
    x, gamma = dev_bf16(q4["x"]), dev_bf16(q4["gamma"])
    c3 = workloads.c3_fp8(256, 512, 256)
    a8, b8 = dev_u8(c3["a"]), dev_u8(c3["b"])
    s64 = torch.full((), 1 / 64, device=dev)
    calls = [d[2] for d in dots] + [
        ops.rowwise_quantize_fp8(x, gamma, build_only=True),
        ops.fp8_scaled_dot(a8, b8, s64, s64, None, epilogue="GELU", build_only=True),
        # f8 result with its amax: a one-thread kernel zeroes the amax, then atomics fold into it
        ops.fp8_scaled_dot(a8, b8, s64, s64, None, epilogue="RELU", d_scale=torch.full((), 0.05, device=dev),
                           amax=True, build_only=True)]

    def results():
        out = []
        for c in calls:
            r = c.result if isinstance(c.result, (list, tuple)) else [c.result]
            out += [t.clone().view(torch.uint8) if t.dtype != torch.float32 else t.clone() for t in r]
        return out

    # options that steer a call's kernel choice are set around that call, eagerly and under capture alike
    def run_all_eager():
        for i, c in enumerate(calls):
            opts = dots[i][3] if i < len(dots) else {}
            for k, v in opts.items():
                ffi.set_option(k, v)
            try:
                c.run()
            finally:
                for k in opts:
                    ffi.set_option(k, 0)

    run_all_eager()   # first launches may set kernel attributes, which must not happen under capture
    torch.cuda.synchronize()

    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for c in calls:
            c.frame.host.stream = side.cuda_stream
        with torch.cuda.graph(graph, stream=side):
            for i, c in enumerate(calls):
                opts = dots[i][3] if i < len(dots) else {}
                for k, v in opts.items():
                    ffi.set_option(k, v)
                try:
                    ffi.Replay([(c.target, c.frame)]).run(1)
                finally:
                    for k in opts:
                        ffi.set_option(k, 0)
    torch.cuda.current_stream().wait_stream(side)

    for round_ in range(3):
        # new operand values in the same buffers, eager work and a synchronisation between replays
        new_lhs = []
        for w, lhs, _, _, _ in dots:
            a = dtypes.f32_to_bf16(rng.standard_normal(w["lhs"].shape).astype(np.float32))
            lhs.copy_(dev_bf16(a))
            new_lhs.append(a)
        xq = dtypes.f32_to_bf16((rng.standard_normal(q4["x"].shape) * (round_ + 1)).astype(np.float32))
        x.copy_(dev_bf16(xq))
        an = dtypes.f32_to_f8e4m3fn(np.clip(rng.standard_normal(c3["a"].shape) * 64, -448, 448).astype(np.float32))
        a8.copy_(dev_u8(an))
        torch.cuda.synchronize()
        run_all_eager()
        torch.cuda.synchronize()
        want = results()
        for c in calls:  # wipe the outputs so that a replay that does nothing cannot pass
            for t in (c.result if isinstance(c.result, (list, tuple)) else [c.result]):
                t.reshape(-1).view(torch.uint8).zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got = results()
        for i, (g, w) in enumerate(zip(got, want)):
            assert torch.equal(g, w), "replay %d: result %d differs from the eager call" % (round_, i)
        # ... and against the oracle, from the replay's own outputs
        for (w, _, call, _, kern), a in zip(dots, new_lhs):
            compare(oracle, dict(w, lhs=a), host_bf16(call.result), "replay %d %s" % (round_, kern))
        q_ref, s_ref = oracle.rmsnorm_quantize_fp8(xq, q4["gamma"], eps=1e-6)
        q_got, s_got = calls[len(dots)].result
        assert np.array_equal(q_got.cpu().numpy(), q_ref) and np.array_equal(s_got.cpu().numpy(), s_ref), round_
        ref = oracle.fp8_scaled_dot(an, c3["b"], 1 / 64, 1 / 64, epilogue="gelu_tanh")
        floor = fp8_floor_for(dict(c3, a=an))
        check_dot(host_bf16(calls[len(dots) + 1].result), ref, floor, "replay %d fp8 dot" % round_)
    assert ffi.last_kernel()  # the library recorded which kernels it chose
