"""ctypes view of the CPU oracle (``xla_cpu_oracle.c``).

Test infrastructure only: imported by ``tests/``, by ``__graft_entry__.smoke``
and by the ``cpu_baseline`` leg of ``bench.py``; never by the ``xla_amd``
package.  Arrays are numpy; bf16 travels as ``uint16`` bit patterns,
f8e4m3fn as ``uint8`` codes, packed s4 as ``uint8`` bytes.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libxla_cpu_oracle.so")

F32, BF16 = 0, 1
EPI_NONE, EPI_RELU, EPI_GELU_TANH, EPI_SILU = 0, 1, 2, 3
EPILOGUES = {"none": EPI_NONE, "relu": EPI_RELU, "gelu_tanh": EPI_GELU_TANH, "silu": EPI_SILU}
TYPES = {"f32": F32, "bf16": BF16}


def build(force=False):
    """Compile the oracle with its Makefile (gcc, OpenMP)."""
    if force and os.path.exists(_LIB_PATH):
        os.remove(_LIB_PATH)
    subprocess.run(["make", "-s", "-C", _HERE], check=True)
    return _LIB_PATH


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = ctypes.CDLL(_LIB_PATH)
        c = ctypes
        vp, i64, i32, f32 = c.c_void_p, c.c_int64, c.c_int, c.c_float
        L.xo_f32_to_bf16.restype = c.c_uint16
        L.xo_f32_to_bf16.argtypes = [f32]
        L.xo_bf16_to_f32.restype = f32
        L.xo_bf16_to_f32.argtypes = [c.c_uint16]
        L.xo_f32_to_f8e4m3fn.restype = c.c_uint8
        L.xo_f32_to_f8e4m3fn.argtypes = [f32]
        L.xo_f16_to_f8e4m3fn.restype = c.c_uint8
        L.xo_f16_to_f8e4m3fn.argtypes = [c.c_uint16]
        L.xo_f8e4m3fn_to_f16.restype = c.c_uint16
        L.xo_f8e4m3fn_to_f16.argtypes = [c.c_uint8]
        L.xo_f8e4m3fn_to_f32.restype = f32
        L.xo_f8e4m3fn_to_f32.argtypes = [c.c_uint8]
        L.xo_f16_to_f32.restype = f32
        L.xo_f16_to_f32.argtypes = [c.c_uint16]
        L.xo_f32_to_f16.restype = c.c_uint16
        L.xo_f32_to_f16.argtypes = [f32]
        L.xo_tanh_f32.restype = f32
        L.xo_tanh_f32.argtypes = [f32]
        L.xo_exp_f32.restype = f32
        L.xo_exp_f32.argtypes = [f32]
        L.xo_mul_add_f32_n.restype = None
        L.xo_mul_add_f32_n.argtypes = [vp, vp, vp, c.c_size_t, vp]
        L.xo_set_fp_contract.restype = None
        L.xo_set_fp_contract.argtypes = [i32]
        L.xo_get_fp_contract.restype = i32
        L.xo_get_fp_contract.argtypes = []
        for name in ("xo_pack_s4", "xo_unpack_s4", "xo_unpack_u4", "xo_f32_to_bf16_n",
                     "xo_f32_to_f8e4m3fn_n", "xo_f8e4m3fn_to_f32_n", "xo_tanh_f32_n",
                     "xo_exp_f32_n"):
            fn = getattr(L, name)
            fn.restype = None
            fn.argtypes = [vp, c.c_size_t, vp]
        L.xo_tree32_sum.restype = f32
        L.xo_tree32_sum.argtypes = [vp, i64]
        L.xo_epilogue_one.restype = c.c_uint16
        L.xo_epilogue_one.argtypes = [f32, i32, i32, i32, f32, i32]
        L.xo_dequant_dot.restype = i32
        L.xo_dequant_dot.argtypes = [vp, vp, i32, vp, i32, i32, vp, i32, i64, i64, i64, i64,
                                     i64, i32, i32, i32, vp]
        L.xo_dequant_dot_zp.restype = i32
        L.xo_dequant_dot_zp.argtypes = [vp, vp, i32, i32, vp, vp, i32, i32, vp, i32, i64, i64, i64, i64,
                                        i64, i32, i32, i32, vp]
        L.xo_dequant_dot_f32.restype = i32
        L.xo_dequant_dot_f32.argtypes = L.xo_dequant_dot_zp.argtypes
        L.xo_fp8_scaled_dot.restype = i32
        L.xo_fp8_scaled_dot.argtypes = [vp, vp, i32, vp, i32, vp, i32, i32, vp, i32, i64, i64, i64,
                                        i32, i32, i32, vp, vp, i32, vp, vp]
        L.xo_f8e8m0fnu_to_f32.restype = f32
        L.xo_f8e8m0fnu_to_f32.argtypes = [c.c_uint8]
        L.xo_block_scaled_dot.restype = i32
        L.xo_block_scaled_dot.argtypes = [vp, vp, vp, vp, i64, vp, i32, i64, i64, i64, i32, i32, i32, vp]
        L.xo_rmsnorm_quantize_fp8.restype = i32
        L.xo_rmsnorm_quantize_fp8.argtypes = [vp, vp, f32, i64, i64, vp, vp]
        L.xo_num_threads.restype = i32
        _lib = L
    return _lib


def _ptr(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def _c(a, dtype):
    a = np.ascontiguousarray(a, dtype=dtype)
    return a


def num_threads():
    return lib().xo_num_threads()


# ---- array casts -----------------------------------------------------------

def f32_to_bf16(x):
    x = _c(x, np.float32)
    out = np.empty(x.shape, np.uint16)
    lib().xo_f32_to_bf16_n(_ptr(x), x.size, _ptr(out))
    return out


def bf16_to_f32(h):
    h = _c(h, np.uint16)
    return (h.astype(np.uint32) << 16).view(np.float32)


def f32_to_f8e4m3fn(x):
    x = _c(x, np.float32)
    out = np.empty(x.shape, np.uint8)
    lib().xo_f32_to_f8e4m3fn_n(_ptr(x), x.size, _ptr(out))
    return out


def f8e4m3fn_to_f32(c):
    c = _c(c, np.uint8)
    out = np.empty(c.shape, np.float32)
    lib().xo_f8e4m3fn_to_f32_n(_ptr(c), c.size, _ptr(out))
    return out


def pack_s4(v):
    v = _c(v, np.int8).reshape(-1)
    out = np.zeros((v.size + 1) // 2, np.uint8)
    lib().xo_pack_s4(_ptr(v), v.size, _ptr(out))
    return out


def unpack_s4(b, n):
    b = _c(b, np.uint8).reshape(-1)
    out = np.empty(n, np.int8)
    lib().xo_unpack_s4(_ptr(b), n, _ptr(out))
    return out


def unpack_u4(b, n):
    b = _c(b, np.uint8).reshape(-1)
    out = np.empty(n, np.uint8)
    lib().xo_unpack_u4(_ptr(b), n, _ptr(out))
    return out


class fp_contract:
    """`with fp_contract(False):` -- the f32 polynomials and the f32-typed GELU with every multiply
    and add rounded separately (a host without fma); the default fuses them, as the reference's
    CPU backend does wherever the host has the instruction (cpu_aot_loader.cc:49-55)."""

    def __init__(self, on):
        self.on = int(bool(on))

    def __enter__(self):
        self.before = lib().xo_get_fp_contract()
        lib().xo_set_fp_contract(self.on)

    def __exit__(self, *exc):
        lib().xo_set_fp_contract(self.before)


def mul_add_f32(a, b, c):
    """a * b + c elementwise with the rounding of one f32 kernel: fused when fp_contract is on."""
    a, b, c = np.broadcast_arrays(np.asarray(a, np.float32), np.asarray(b, np.float32), np.asarray(c, np.float32))
    a, b, c = _c(a, np.float32), _c(b, np.float32), _c(c, np.float32)
    out = np.empty_like(a)
    lib().xo_mul_add_f32_n(_ptr(a), _ptr(b), _ptr(c), a.size, _ptr(out))
    return out


def tanh_f32(x):
    x = _c(x, np.float32)
    out = np.empty_like(x)
    lib().xo_tanh_f32_n(_ptr(x), x.size, _ptr(out))
    return out


def exp_f32(x):
    x = _c(x, np.float32)
    out = np.empty_like(x)
    lib().xo_exp_f32_n(_ptr(x), x.size, _ptr(out))
    return out


def tree32_sum(v):
    v = _c(v, np.float32).reshape(-1)
    return float(lib().xo_tree32_sum(_ptr(v), v.size))


# ---- the three fused paths -------------------------------------------------

def dequant_dot(a_bf16, w, w_bits, scale, scale_ty, mul_ty, bias=None, bias_ty="bf16",
                group=None, dot_ty="f32", ep_ty="f32", epilogue="none", unsigned=False, zero_points=None,
                f32_result=False):
    """a_bf16: uint16 [B,M,K] or [M,K]; w: int8 [..,K,N] (w_bits=8) or packed uint8 (w_bits=4,
    with logical shape given by scale/N); scale: [..,K/group,N].  Returns uint16 bf16 [..,M,N].
    unsigned: the 4-bit weights are u4; zero_points: packed u4, one per scale: (w - z) * scale.
    f32_result: returns float32, the value before the final convert to bf16."""
    a = _c(a_bf16, np.uint16)
    batched = a.ndim == 3
    if not batched:
        a = a[None]
    B, M, K = a.shape
    scale = np.ascontiguousarray(scale)
    s = scale if scale.ndim == 3 else scale.reshape(B, -1, scale.shape[-1])
    G, N = s.shape[1], s.shape[2]
    if group is None:
        group = K // G
    assert G * group == K
    s = _c(s, np.uint16 if scale_ty == "bf16" else np.float32)
    if w_bits == 8:
        w = _c(w, np.int8)
        assert w.size == B * K * N
    else:
        w = _c(w, np.uint8)
        assert w.size == (B * K * N + 1) // 2
    bp = None
    if bias is not None:
        bias = _c(bias, np.uint16 if bias_ty == "bf16" else np.float32)
        assert bias.size == N
        bp = _ptr(bias)
    out = np.empty((B, M, N), np.float32 if f32_result else np.uint16)
    zp = None
    if zero_points is not None:
        zero_points = _c(zero_points, np.uint8)
        assert zero_points.size == (B * G * N + 1) // 2
        zp = _ptr(zero_points)
    fn = lib().xo_dequant_dot_f32 if f32_result else lib().xo_dequant_dot_zp
    rc = fn(_ptr(a), _ptr(w), w_bits, int(bool(unsigned)), zp, _ptr(s), TYPES[scale_ty],
            TYPES[mul_ty], bp, TYPES[bias_ty], B, M, K, N, group, TYPES[dot_ty],
            TYPES[ep_ty], EPILOGUES[epilogue], _ptr(out))
    assert rc == 0
    return out if batched else out[0]


def ragged_dequant_dot(a_bf16, w, w_bits, scale, scale_ty, mul_ty, group_sizes, **kw):
    """Ragged dot (xla ragged-dot, ragged dimension = rows of lhs; expanded by the reference into one
    masked dense dot per group, xla/hlo/transforms/expanders/ragged_dot_rewriter.cc:110-210):
    a_bf16 [M,K] with rows sorted by group, w [G,K,N] (int8, or packed 4-bit per group), scale
    [G,..,N]; row m of group g is lhs[m] . dequant(w[g]); rows past the last group are a dot of
    nothing, i.e. epilogue(0).  Built from dequant_dot, one call per group."""
    a = _c(a_bf16, np.uint16)
    M, K = a.shape
    sizes = [int(x) for x in np.asarray(group_sizes).reshape(-1)]
    G = len(sizes)
    scale = np.ascontiguousarray(scale)
    N = scale.shape[-1]
    w = np.ascontiguousarray(w)
    wg = w.reshape(G, -1)
    sg = scale.reshape(G, -1, N)
    zp = kw.pop("zero_points", None)
    zg = None if zp is None else np.ascontiguousarray(zp).reshape(G, -1)
    out = np.empty((M, N), np.uint16)
    start = 0
    for g in range(G):
        n = max(0, min(sizes[g], M - start))
        if n:
            out[start:start + n] = dequant_dot(a[start:start + n], wg[g], w_bits, sg[g], scale_ty, mul_ty,
                                               zero_points=None if zg is None else zg[g], **kw)
        start += n
    if start < M:   # a dot of nothing: zero activations give the same rows
        zero = np.zeros((M - start, K), np.uint16)
        out[start:] = dequant_dot(zero, wg[0], w_bits, sg[0], scale_ty, mul_ty,
                                  zero_points=None if zg is None else zg[0], **kw)
    return out


def fp8_scaled_dot(a8, b8, a_scale, b_scale, b_is_nk=False, mul_ty="f32", bias=None,
                   bias_ty="bf16", dot_ty="f32", ep_ty="f32", epilogue="none", d_scale=None,
                   d_scale_divides=True):
    """bf16 result [M,N]; with d_scale the f8e4m3fn result convert(clamp(v / d_scale)) (or
    v * d_scale) and the f32 values v before the scaling, as a pair."""
    a8 = _c(a8, np.uint8)
    b8 = _c(b8, np.uint8)
    M, K = a8.shape
    N = b8.shape[0] if b_is_nk else b8.shape[1]
    assert (b8.shape[1] if b_is_nk else b8.shape[0]) == K
    bp = None
    if bias is not None:
        bias = _c(bias, np.uint16 if bias_ty == "bf16" else np.float32)
        assert bias.size == N
        bp = _ptr(bias)
    # a scale is one value, or one per row of a (a_scale) / per output channel (b_scale)
    sa = _c(np.asarray(a_scale, np.float32).reshape(-1), np.float32)
    sb = _c(np.asarray(b_scale, np.float32).reshape(-1), np.float32)
    a_rows, b_cols = np.ndim(a_scale) == 1, np.ndim(b_scale) == 1
    assert sa.size == (M if a_rows else 1) and sb.size == (N if b_cols else 1)
    if d_scale is None:
        out = np.empty((M, N), np.uint16)
        tail = (_ptr(out), None, 0, None, None)
    else:
        assert dot_ty == "f32" and ep_ty == "f32"
        sd = _c(np.asarray(d_scale, np.float32).reshape(1), np.float32)
        out8, val = np.empty((M, N), np.uint8), np.empty((M, N), np.float32)
        tail = (None, _ptr(sd), int(bool(d_scale_divides)), _ptr(out8), _ptr(val))
    rc = lib().xo_fp8_scaled_dot(_ptr(a8), _ptr(b8), int(b_is_nk), _ptr(sa), int(a_rows), _ptr(sb),
                                 int(b_cols), TYPES[mul_ty], bp, TYPES[bias_ty], M, K, N, TYPES[dot_ty],
                                 TYPES[ep_ty], EPILOGUES[epilogue], *tail)
    assert rc == 0
    return out if d_scale is None else (out8, val)


def f8e8m0fnu_to_f32(codes):
    codes = np.asarray(codes, np.uint8)
    return np.array([lib().xo_f8e8m0fnu_to_f32(int(v)) for v in codes.reshape(-1)], np.float32).reshape(codes.shape)


def block_scaled_dot(a8, b8_nk, a_sc, b_sc, block=32, bias=None, bias_ty="bf16", dot_ty="f32", ep_ty="f32",
                     epilogue="none"):
    """bf16 [M,N] = epilogue(dot(a8 * 2^(a_sc-127), b8 * 2^(b_sc-127))): a8 [M,K], b8 [N,K] f8e4m3fn codes,
    scales f8e8m0fnu codes, one per `block` elements of K."""
    a8, b8 = _c(a8, np.uint8), _c(b8_nk, np.uint8)
    M, K = a8.shape
    N = b8.shape[0]
    assert b8.shape[1] == K and K % block == 0
    a_sc, b_sc = _c(a_sc, np.uint8), _c(b_sc, np.uint8)
    assert a_sc.shape == (M, K // block) and b_sc.shape == (N, K // block)
    bp = None
    if bias is not None:
        bias = _c(bias, np.uint16 if bias_ty == "bf16" else np.float32)
        bp = _ptr(bias)
    out = np.empty((M, N), np.uint16)
    rc = lib().xo_block_scaled_dot(_ptr(a8), _ptr(b8), _ptr(a_sc), _ptr(b_sc), block, bp, TYPES[bias_ty], M, K, N,
                                   TYPES[dot_ty], TYPES[ep_ty], EPILOGUES[epilogue], _ptr(out))
    assert rc == 0
    return out


def rmsnorm_quantize_fp8(x_bf16, gamma_bf16, eps=1e-6):
    x = _c(x_bf16, np.uint16)
    g = _c(gamma_bf16, np.uint16)
    rows, cols = x.shape
    assert g.size == cols
    q = np.empty((rows, cols), np.uint8)
    s = np.empty(rows, np.float32)
    rc = lib().xo_rmsnorm_quantize_fp8(_ptr(x), _ptr(g), float(np.float32(eps)), rows, cols,
                                       _ptr(q), _ptr(s))
    assert rc == 0
    return q, s
