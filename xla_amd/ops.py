"""The three custom calls as Python callables over device tensors.

Every function builds an XLA FFI call frame and goes through the library's exported
handler symbol -- the same entry XLA's CustomCallThunk would call -- on torch's current
HIP stream.  torch only supplies device memory and the stream.  bf16 operands are
``torch.bfloat16`` tensors, f8e4m3fn operands ``torch.float8_e4m3fn`` (or ``uint8`` codes),
s8 weights ``int8``, s4 weights ``uint8`` holding two values per byte (low nibble first)
with the logical shape passed separately.
"""
import torch

from . import dtypes, ffi

_host = None


def host():
    """The process-wide FFI host (function table in C++)."""
    global _host
    if _host is None:
        _host = ffi.NativeHost()
    return _host


def _stream():
    return torch.cuda.current_stream().cuda_stream


def _check_cuda(*tensors):
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise ValueError("operands must live on the GPU; this package has no CPU path")


_FLOAT = {torch.float32: dtypes.F32, torch.bfloat16: dtypes.BF16}
_NAMES = {dtypes.F32: "f32", dtypes.BF16: "bf16"}
_TYPE_ATTR = {"f32": dtypes.F32, "bf16": dtypes.BF16}


class Call:
    """A prepared custom call: the call frame, its result tensors, and references that keep every
    operand alive.  ``run()`` invokes it on torch's current stream; ``build_only=True`` on the
    functions below returns the Call so that ffi.Replay can re-invoke it natively."""

    def __init__(self, target, frame, result, keep=()):
        self.target, self.frame, self.result, self._keep = target, frame, result, keep

    def run(self):
        self.frame.host.stream = _stream()
        ffi.invoke(self.target, self.frame)
        return self.result


def _scratch(nbytes, device):
    return torch.empty(max(int(nbytes), 1), dtype=torch.uint8, device=device) if nbytes else None


def dequant_dot(lhs, weights, scales, bias=None, *, weight_dtype="s8", weight_shape=None,
                epilogue="DEFAULT", dequant_type="f32", dot_type="f32", epilogue_type="f32",
                scale_group_size=None, zero_points=None, group_sizes=None, rhs_contracting_dim=0, out=None,
                scratch="auto", build_only=False, out_dtype="bf16", result_transposed=False, lhs_contracting_dim=1,
                d_scale=None, d_scale_multiplies=False):
    """out = epilogue(lhs . (convert(weights) * scales)).  lhs bf16 [M,K] or [B,M,K].
    scale_group_size: rows of K per scale (0 = per output channel); None leaves the attribute out and
    the handler reads the grouping off the scales' shape.
    weight_dtype "u4": unsigned 4-bit weights, packed like s4; zero_points (uint8, packed u4, one per
    scale) then makes the dequantised weight (w - zero_point) * scale.
    group_sizes (int32 or int64 [G], on the device): ragged dot -- lhs [M,K] with its rows sorted by
    group, weights [G,K,N]; group g multiplies rows [sum(sizes[:g]), +sizes[g]) with weights[g].
    rhs_contracting_dim=1: weights [N,K] or [B,N,K] (4-bit values packed along K), scales [N], [B,N],
    [N,K/g] or [B,N,K/g]; scale_group_size is then required.
    out_dtype "f32": the dot's f32 value is the result.  result_transposed: the result is [..,N,M] (the
    dequantised weights were the lhs of the dot; DEFAULT epilogue only).  lhs_contracting_dim=0: lhs is
    stored [..,K,M].  With d_scale (f32 []) the result is f8e4m3fn codes (uint8):
    convert(clamp(out / d_scale)), or out * d_scale with d_scale_multiplies."""
    _check_cuda(lhs, weights, scales, bias, zero_points, group_sizes, d_scale)
    wdt = {"s4": dtypes.S4, "u4": dtypes.U4}.get(weight_dtype, dtypes.S8)
    wshape = list(weight_shape) if weight_shape is not None else list(weights.shape)
    n = wshape[-2] if rhs_contracting_dim == 1 else wshape[-1]
    m, k = (lhs.shape[-1], lhs.shape[-2]) if lhs_contracting_dim == 0 else (lhs.shape[-2], lhs.shape[-1])
    oshape = list(lhs.shape[:-2]) + ([n, m] if result_transposed else [m, n])
    if out is None:
        odt = torch.uint8 if d_scale is not None else torch.float32 if out_dtype == "f32" else torch.bfloat16
        out = torch.empty(oshape, dtype=odt, device=lhs.device)
    batch = lhs.shape[0] if lhs.dim() == 3 else (wshape[0] if group_sizes is not None else 1)
    args = [(dtypes.BF16, lhs.data_ptr(), lhs.shape), (wdt, weights.data_ptr(), wshape),
            (_FLOAT[scales.dtype], scales.data_ptr(), scales.shape)]
    if zero_points is not None:
        args.append((dtypes.U4, zero_points.data_ptr(), scales.shape))
    if bias is not None:
        args.append((_FLOAT[bias.dtype], bias.data_ptr(), bias.shape))
    if d_scale is not None:
        args.append((dtypes.F32, d_scale.data_ptr(), []))
    if group_sizes is not None:
        args.append((dtypes.S64 if group_sizes.dtype == torch.int64 else dtypes.S32, group_sizes.data_ptr(),
                     group_sizes.shape))
    rets = [(dtypes.F8E4M3FN if d_scale is not None else dtypes.F32 if out.dtype == torch.float32 else dtypes.BF16,
             out.data_ptr(), oshape)]
    if scratch == "auto":
        sizer = (ffi.library().xla_amd_dequant_dot_workspace_bytes_nk if rhs_contracting_dim == 1
                 else ffi.library().xla_amd_dequant_dot_workspace_bytes)
        nbytes = sizer(batch, m, k, n, wdt)
        scratch = _scratch(nbytes, lhs.device)
    if scratch is not None:
        rets.append((dtypes.U8, scratch.data_ptr(), [scratch.numel()]))
    attrs = {"epilogue": ffi.Attr.str(epilogue), "dequant_type": ffi.Attr.i32(_TYPE_ATTR[dequant_type]),
             "dot_type": ffi.Attr.i32(_TYPE_ATTR[dot_type]),
             "epilogue_type": ffi.Attr.i32(_TYPE_ATTR[epilogue_type])}
    if scale_group_size is not None:
        attrs["scale_group_size"] = ffi.Attr.i64(scale_group_size)
    if rhs_contracting_dim != 0:
        attrs["rhs_contracting_dim"] = ffi.Attr.i64(rhs_contracting_dim)
    if lhs_contracting_dim != 1:
        attrs["lhs_contracting_dim"] = ffi.Attr.i64(lhs_contracting_dim)
    if result_transposed:
        attrs["result_transposed"] = ffi.Attr.pred(True)
    if d_scale_multiplies:
        attrs["d_scale_multiplies"] = ffi.Attr.pred(True)
    call = Call("xla_amd.dequant_dot", ffi.Frame(host(), args, rets, attrs), out,
                keep=(lhs, weights, scales, bias, scratch, zero_points, group_sizes, d_scale))
    return call if build_only else call.run()


def fp8_scaled_dot(a, b, a_scale, b_scale, bias=None, *, rhs_contracting_dim=0, epilogue="DEFAULT",
                   dequant_type="f32", dot_type="f32", epilogue_type="f32", out=None, scratch="auto",
                   d_scale=None, d_scale_multiplies=False, amax=False, build_only=False):
    """out = epilogue((a*a_scale) . (b*b_scale)); a f8 [M,K]; b f8 [K,N] or [N,K];
    a_scale f32 [] or [M] (per row of a), b_scale f32 [] or [N] (per output channel); or both uint8
    f8e8m0fnu block scales [M,K/32], [N,K/32] with b = [N,K] (MXFP8).
    With d_scale (f32 []) the result is f8e4m3fn codes (uint8): convert(clamp(out / d_scale)),
    or out * d_scale with d_scale_multiplies; with amax=True the call also returns max |out| (f32 [])
    as a second tensor."""
    _check_cuda(a, b, a_scale, b_scale, bias, d_scale)
    *lead, m, k = a.shape          # one leading batch dimension, or none
    n = b.shape[len(lead) + 1 - rhs_contracting_dim]
    out_f8 = d_scale is not None
    if out is None:
        out = torch.empty((*lead, m, n), dtype=torch.uint8 if out_f8 else torch.bfloat16, device=a.device)
    # uint8 scales are f8e8m0fnu block scales [rows, K/32] (MXFP8); float32 ones per tensor / row / channel
    scale_ty = dtypes.F8E8M0FNU if a_scale.dtype == torch.uint8 else dtypes.F32
    args = [(dtypes.F8E4M3FN, a.data_ptr(), a.shape), (dtypes.F8E4M3FN, b.data_ptr(), b.shape),
            (scale_ty, a_scale.data_ptr(), list(a_scale.shape)),
            (scale_ty, b_scale.data_ptr(), list(b_scale.shape))]
    if bias is not None:
        args.append((_FLOAT[bias.dtype], bias.data_ptr(), bias.shape))
    if out_f8:
        args.append((dtypes.F32, d_scale.data_ptr(), list(d_scale.shape)))
    rets = [(dtypes.F8E4M3FN if out_f8 else dtypes.BF16, out.data_ptr(), [*lead, m, n])]
    amax_t = None
    if amax:
        if not out_f8:
            raise ValueError("amax comes with an f8 result (d_scale)")
        amax_t = torch.empty((), dtype=torch.float32, device=a.device)
        rets.append((dtypes.F32, amax_t.data_ptr(), []))
    if scratch == "auto":
        nbytes = ffi.library().xla_amd_fp8_scaled_dot_workspace_bytes_typed(
            m, k, n, rhs_contracting_dim, dtypes.BF16 if dequant_type == "bf16" else dtypes.F32)
        scratch = _scratch(nbytes, a.device)
    if scratch is not None:
        rets.append((dtypes.U8, scratch.data_ptr(), [scratch.numel()]))
    attrs = {"epilogue": ffi.Attr.str(epilogue), "dequant_type": ffi.Attr.i32(_TYPE_ATTR[dequant_type]),
             "dot_type": ffi.Attr.i32(_TYPE_ATTR[dot_type]),
             "epilogue_type": ffi.Attr.i32(_TYPE_ATTR[epilogue_type]),
             "rhs_contracting_dim": ffi.Attr.i64(rhs_contracting_dim)}
    if out_f8:
        attrs["d_scale_multiplies"] = ffi.Attr.pred(d_scale_multiplies)
    call = Call("xla_amd.fp8_scaled_dot", ffi.Frame(host(), args, rets, attrs),
                (out, amax_t) if amax else out, keep=(a, b, a_scale, b_scale, bias, d_scale, scratch))
    return call if build_only else call.run()


def rowwise_quantize_fp8(x, gamma=None, *, eps=1e-6, q=None, scales=None, build_only=False):
    """(q, scales) = per-row dynamic f8e4m3fn quantisation of x (bf16 [R,C]), after RMSNorm with
    ``gamma`` when given.  q is returned as uint8 codes."""
    _check_cuda(x, gamma)
    r, c = x.shape
    if q is None:
        q = torch.empty((r, c), dtype=torch.uint8, device=x.device)
    if scales is None:
        scales = torch.empty((r,), dtype=torch.float32, device=x.device)
    args = [(dtypes.BF16, x.data_ptr(), [r, c])]
    if gamma is not None:
        args.append((dtypes.BF16, gamma.data_ptr(), gamma.shape))
    rets = [(dtypes.F8E4M3FN, q.data_ptr(), [r, c]), (dtypes.F32, scales.data_ptr(), [r])]
    attrs = {"rmsnorm": ffi.Attr.pred(gamma is not None), "eps": ffi.Attr.f32(eps)}
    call = Call("xla_amd.rowwise_quantize_fp8", ffi.Frame(host(), args, rets, attrs), (q, scales),
                keep=(x, gamma))
    return call if build_only else call.run()
