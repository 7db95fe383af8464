"""Builds the native pieces of the package in-tree with hipcc, for gfx950 only.

``python -m xla_amd.build`` (or ``__graft_entry__.build()``) produces
  xla_amd/lib/libxla_amd_quant.so   kernels + launchers + XLA FFI handlers
  xla_amd/lib/libxla_amd_host.so    FFI call-frame host and HLO rewrite pass (host only)
  xla_amd/lib/libxla_amd_selfcheck.so  test and benchmark aids (exhaustive numerics checks, stream
                                    yardstick, empty kernel); not part of the product
Nothing is compiled at import time; loaders fail loudly if a library is missing.
"""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "xla_amd", "csrc")
LIB = os.path.join(ROOT, "xla_amd", "lib")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")

KERNEL_SOURCES = ["capi.hip", "rowwise_quantize.hip", "dequant_dot_decode.hip", "dequant_dot_decode_s4x.hip", "dequant_dot_decode_s8x.hip", "dequant_dot_nk.hip", "tiled_dot_mfma.hip", "fp8_dot_decode.hip",
                  "ffi_handlers.cc"]
SELFCHECK_SOURCES = ["self_check.hip"]
HOST_SOURCES = ["host/ffi_host.cc", "host/hlo_ir.cc", "host/quant_fusion_rewriter.cc",
                "host/host_capi.cc"]

# -ffp-contract=off: multiplies and adds round separately unless __builtin_fmaf is written out.
# packed-fp32 VALU forms are disabled (the compiler would otherwise form them from scalar code).
DEVICE_FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off",
                "-fvisibility=hidden", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
                "-Wno-unused-command-line-argument", "-Wno-unknown-warning-option",
                "-I" + os.path.join(ROOT, "include"), "-I" + CSRC]


def _run(cmd):
    print(" ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)


def build_kernels(jobs=8, sources=None, libname="libxla_amd_quant.so"):
    os.makedirs(LIB, exist_ok=True)
    objs, procs = [], []
    for src in (sources or KERNEL_SOURCES):
        obj = os.path.join(LIB, os.path.basename(src) + ".o")
        cmd = [HIPCC, "-c", os.path.join(CSRC, src), "-o", obj] + DEVICE_FLAGS
        if src.endswith(".cc"):
            cmd = [HIPCC, "-x", "hip", "-c", os.path.join(CSRC, src), "-o", obj] + DEVICE_FLAGS
        print(" ".join(cmd), flush=True)
        procs.append((subprocess.Popen(cmd), src))
        objs.append(obj)
        if len(procs) >= jobs:
            p, s = procs.pop(0)
            if p.wait() != 0:
                raise RuntimeError("hipcc failed on " + s)
    for p, s in procs:
        if p.wait() != 0:
            raise RuntimeError("hipcc failed on " + s)
    out = os.path.join(LIB, libname)
    _run([HIPCC, "-shared", "-o", out] + objs + ["--offload-arch=gfx950", "-fPIC"])
    return out


def build_selfcheck():
    return build_kernels(sources=SELFCHECK_SOURCES, libname="libxla_amd_selfcheck.so")


def build_host():
    os.makedirs(LIB, exist_ok=True)
    srcs = [os.path.join(CSRC, s) for s in HOST_SOURCES if os.path.exists(os.path.join(CSRC, s))]
    out = os.path.join(LIB, "libxla_amd_host.so")
    _run(["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-fvisibility=hidden", "-Wall",
          "-I" + os.path.join(ROOT, "include"), "-I" + CSRC, "-o", out] + srcs + ["-ldl"])
    return out


def build_all():
    return [build_kernels(), build_selfcheck(), build_host()]


if __name__ == "__main__":
    what = sys.argv[1] if len(sys.argv) > 1 else "all"
    {"all": build_all, "kernels": build_kernels, "host": build_host, "selfcheck": build_selfcheck}[what]()
