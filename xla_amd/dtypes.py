"""Host-side helpers for the narrow element types on the quantized path.

XLA literals carry bf16 / f8e4m3fn / s4 values that numpy has no dtype for, so
this package moves them as raw bit patterns: bf16 -> ``uint16``, f8e4m3fn ->
``uint8``, s4 -> two's-complement nibbles packed two per ``uint8``.  The
routines here are vectorised numpy and are used to *prepare inputs* (synthetic
workloads, literal files); device kernels do their own casts.

Element-type numbers are XLA's ``PrimitiveType`` / ``XLA_FFI_DataType`` values
(xla/ffi/api/c_api.h:233-266).
"""
import numpy as np

# XLA_FFI_DataType values (xla/ffi/api/c_api.h:233-266).
PRED, S8, S16, S32, S64 = 1, 2, 3, 4, 5
U8, U16, U32, U64 = 6, 7, 8, 9
F16, F32, F64, BF16 = 10, 11, 12, 16
F8E5M2, F8E4M3FN, S4, U4 = 19, 20, 21, 22
F8E8M0FNU = 33

DTYPE_NAMES = {PRED: "PRED", S8: "S8", S16: "S16", S32: "S32", S64: "S64", U8: "U8", U16: "U16",
               U32: "U32", U64: "U64", F16: "F16", F32: "F32", F64: "F64", BF16: "BF16",
               F8E5M2: "F8E5M2", F8E4M3FN: "F8E4M3FN", S4: "S4", U4: "U4", F8E8M0FNU: "F8E8M0FNU"}
HLO_NAMES = {k: v.lower() for k, v in DTYPE_NAMES.items()}
FROM_HLO_NAME = {v: k for k, v in HLO_NAMES.items()}


def f32_to_bf16(x):
    """Round-to-nearest-even f32 -> bf16 bit patterns; NaN -> quiet NaN, sign kept
    (same rule as xla/codegen/intrinsic/fptrunc.cc:88-110)."""
    u = np.ascontiguousarray(x, np.float32).view(np.uint32)
    lsb = (u >> 16) & 1
    rounded = (u + np.uint32(0x7FFF) + lsb) >> 16
    nan = (u & 0x7FFFFFFF) > 0x7F800000
    qnan = ((u & np.uint32(0xFFC00000)) | np.uint32(0x00400000)) >> 16
    return np.where(nan, qnan, rounded).astype(np.uint16)


def bf16_to_f32(h):
    return (np.ascontiguousarray(h, np.uint16).astype(np.uint32) << 16).view(np.float32)


def f8e4m3fn_to_f32(c):
    """Exact widening of e4m3fn codes (bias 7, no inf, 0x7F/0xFF = NaN)."""
    c = np.ascontiguousarray(c, np.uint8).astype(np.int32)
    e = (c >> 3) & 0xF
    m = c & 7
    mag = np.where(e == 0, m * 2.0 ** -9, (8 + m) * 2.0 ** (e - 10.0))
    mag = np.where((c & 0x7F) == 0x7F, np.nan, mag)
    return np.where(c & 0x80, -mag, mag).astype(np.float32)


def f32_to_f8e4m3fn(x):
    """f32 -> e4m3fn, round-to-nearest-even, overflow (|x| > 464) / inf / NaN -> 0x7F
    with the sign kept, no saturation (xla/codegen/intrinsic/fptrunc.cc:375-509)."""
    x = np.ascontiguousarray(x, np.float32)
    u = x.view(np.uint32)
    sign = ((u >> 31) << 7).astype(np.uint8)
    with np.errstate(invalid="ignore"):
        a = np.abs(x.astype(np.float64))
    fin = np.where(np.isfinite(a), a, 0.0)
    e = np.frexp(fin)[1] - 1.0               # exact floor(log2(a)); 0 -> -1, clipped below
    e = np.clip(e, -6, None)                 # subnormals share the exponent of 2^-6
    step = 2.0 ** (e - 3)
    q = np.rint(fin / step)                  # rint = ties to even; fin/step is exact
    v = q * step
    # re-derive the code from the rounded value (rounding may have bumped the exponent)
    ev = np.clip(np.frexp(v)[1] - 1.0, -6, None)
    mant = np.rint(v / 2.0 ** (ev - 3)).astype(np.int64)
    normal = mant >= 8
    code = np.where(normal, ((ev + 7).astype(np.int64) << 3) | (mant - 8), mant)
    bad = ~(a <= 464.0)                      # also catches NaN
    code = np.where(bad, 0x7F, code).astype(np.uint8)
    return code | sign


def pack_s4(values):
    """Pack s4 values (any int array in [-8, 7]) low nibble first over the flat row-major
    index (xla/service/llvm_ir/ir_array.cc:588-603).  Odd counts leave the last high nibble 0."""
    v = np.ascontiguousarray(values).reshape(-1).astype(np.int8).view(np.uint8) & 0xF
    if v.size & 1:
        v = np.concatenate([v, np.zeros(1, np.uint8)])
    return (v[0::2] | (v[1::2] << 4)).astype(np.uint8)


def unpack_s4(packed, n):
    b = np.ascontiguousarray(packed, np.uint8).reshape(-1)
    nib = np.empty(b.size * 2, np.uint8)
    nib[0::2] = b & 0xF
    nib[1::2] = b >> 4
    nib = nib[:n]
    return ((nib << 4).view(np.int8) >> 4).astype(np.int8)
