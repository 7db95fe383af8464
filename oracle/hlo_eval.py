"""Op-by-op evaluation of an (unrewritten) HLO module with the XLA CPU backend's rounding
rules -- test infrastructure, like the rest of ``oracle/``.

Input is the JSON form of a module (``xla_amd.hlo.to_json``).  Every instruction is
evaluated on numpy arrays, one at a time, and its result is re-rounded to the instruction's
element type, which is what FloatNormalization makes of bf16/f8 ops on the CPU
(xla/service/cpu/cpu_compiler.cc:804-840).  Dots accumulate in f32 over increasing k, one
rounding per product and per sum; reduce-add follows TreeReductionRewriter(32).  The scalar
casts, tanh and exp are the ones of ``xla_cpu_oracle.c``.

Values: f32 -> float32 arrays; bf16 -> float32 arrays holding bf16-representable values;
f8e4m3fn -> uint8 codes; s8/s4 -> int8.
"""
import numpy as np

from . import oracle as O


def _round(v, dtype):
    if dtype == "bf16":
        return O.bf16_to_f32(O.f32_to_bf16(np.ascontiguousarray(v, np.float32)))
    if dtype == "f32":
        return np.ascontiguousarray(v, np.float32)
    raise NotImplementedError("result type " + dtype)


def _dims(attr):
    attr = attr.strip("{} ")
    return [int(t) for t in attr.split(",") if t.strip()] if attr else []


def _tree32_sum_last(x):
    """Sum over the last axis: windows of 32 added left to right, recursively."""
    x = np.ascontiguousarray(x, np.float32)
    while x.shape[-1] > 1:
        n = x.shape[-1]
        m = (n + 31) // 32
        pad = m * 32 - n
        if pad:
            x = np.concatenate([x, np.zeros(x.shape[:-1] + (pad,), np.float32)], axis=-1)
        w = x.reshape(x.shape[:-1] + (m, 32))
        acc = np.zeros(w.shape[:-1], np.float32)
        for i in range(32):
            acc = (acc + w[..., i]).astype(np.float32)
        x = acc
    return x[..., 0]


def _dot(a, b, lc, rc, lb, rb):
    """f32 dot, accumulating over increasing k: result [lhs free, rhs free].  Either operand may
    contract its minor or its major non-batch dimension; one leading batch dimension at most."""
    a = np.ascontiguousarray(a, np.float32)
    b = np.ascontiguousarray(b, np.float32)
    if lb:
        assert lb == [0] and rb == [0] and a.ndim == 3 and b.ndim == 3
        return np.stack([_dot(a[i], b[i], [lc[0] - 1], [rc[0] - 1], [], []) for i in range(a.shape[0])])
    assert a.ndim == 2 and b.ndim == 2 and lc in ([0], [1]) and rc in ([0], [1])
    if lc == [0]:
        a = np.ascontiguousarray(a.T)
    if rc == [1]:
        b = np.ascontiguousarray(b.T)
    acc = np.zeros((a.shape[0], b.shape[1]), np.float32)
    for k in range(a.shape[1]):
        p = (a[:, k:k + 1] * b[k:k + 1, :]).astype(np.float32)
        acc = (acc + p).astype(np.float32)
    return acc


def evaluate(module_json, args):
    """args: list of numpy arrays in parameter order (bf16 as uint16 bit patterns, f8 as uint8
    codes, s4 as *unpacked* int8 values).  Returns the root value (tuple -> list); bf16 results
    come back as uint16 bit patterns, f8 as uint8 codes."""
    comps = {c["name"]: c for c in module_json["computations"]}
    entry = next(c for c in module_json["computations"] if c["entry"])
    env = {}

    def reducer_kind(name):
        body = comps[name.lstrip("%")]
        root = next(i for i in body["instructions"] if i["root"])
        return root["opcode"]

    by_name = {i["name"]: i for i in entry["instructions"]}
    uses = {}
    for i in entry["instructions"]:
        for o in i["operands"]:
            uses[o] = uses.get(o, 0) + 1

    def contracted_product(add):
        for k, o in enumerate(add["operands"]):
            m = by_name[o]
            if m["opcode"] == "multiply" and m["shape"].get("dtype") == "f32" and uses[o] == 1 and not m["root"]:
                return k
        return None

    for ins in entry["instructions"]:
        op, sh = ins["opcode"], ins["shape"]
        ty = sh.get("dtype")
        x = [env[o] for o in ins["operands"]]
        if op == "parameter":
            v = args[int(ins["literal"])]
            if ty == "bf16":
                v = O.bf16_to_f32(v)
            elif ty in ("f8e4m3fn", "f8e8m0fnu"):
                v = np.ascontiguousarray(v, np.uint8)
            elif ty in ("s8", "s4", "u4"):
                v = np.ascontiguousarray(v, np.int8)   # unpacked values (u4: 0..15)
            elif ty in ("s32", "s64"):
                v = np.ascontiguousarray(v, np.int64)
            else:
                v = np.ascontiguousarray(v, np.float32)
            v = v.reshape(sh["dims"])
        elif op == "constant":
            v = _round(np.array(float(ins["literal"].strip("{} ")), np.float32), ty)
        elif op == "convert":
            src_ty = next(i for i in entry["instructions"] if i["name"] == ins["operands"][0])["shape"]["dtype"]
            s = x[0]
            if src_ty == "f8e4m3fn":
                s = O.f8e4m3fn_to_f32(s)
            if ty == "f8e4m3fn":
                v = O.f32_to_f8e4m3fn(np.ascontiguousarray(s, np.float32))
            elif ty in ("s8", "s4", "u4"):
                v = np.ascontiguousarray(s, np.int8)
            else:
                v = _round(np.asarray(s).astype(np.float32), ty)
        elif op == "broadcast":
            dims = _dims(ins["attrs"].get("dimensions", ""))
            shape = [1] * len(sh["dims"])
            for i, d in enumerate(dims):
                shape[d] = x[0].shape[i]
            v = np.broadcast_to(np.reshape(x[0], shape), sh["dims"])
        elif op in ("reshape", "bitcast"):
            v = np.reshape(x[0], sh["dims"])
        elif op == "add" and ty == "f32" and contracted_product(ins) is not None:
            # an f32 multiply whose only user is this f32 add: one fused kernel on the CPU backend,
            # whose LLVM may contract the pair (cpu_aot_loader.cc:49-55) -- O.mul_add_f32 decides
            k = contracted_product(ins)
            m = by_name[ins["operands"][k]]
            v = O.mul_add_f32(env[m["operands"][0]], env[m["operands"][1]], x[1 - k])
        elif op in ("multiply", "add", "subtract", "divide", "maximum", "minimum"):
            a, b = np.asarray(x[0], np.float32), np.asarray(x[1], np.float32)
            with np.errstate(all="ignore"):
                r = {"multiply": np.multiply, "add": np.add, "subtract": np.subtract, "divide": np.divide,
                     "maximum": np.maximum, "minimum": np.minimum}[op](a, b)
            v = _round(r, ty)
        elif op == "ragged-dot":
            # lhs [M,K] rows sorted by group, rhs [G,K,N], group sizes [G]: row m of group g is
            # lhs[m] . rhs[g], f32 sums in increasing k; rows no group owns are zero
            # (ragged_dot_rewriter.cc:110-210 masks one dense dot per group)
            a_ = np.asarray(x[0], np.float32)
            b_ = np.asarray(x[1], np.float32)
            sizes = [int(v) for v in np.asarray(x[2]).reshape(-1)]
            assert _dims(ins["attrs"].get("lhs_contracting_dims", "")) == [1]
            rc = _dims(ins["attrs"].get("rhs_contracting_dims", ""))
            assert rc in ([1], [2])          # rhs [G,K,N], or [G,N,K] with the contracting dimension minor
            assert _dims(ins["attrs"].get("lhs_ragged_dims", "")) == [0]
            assert _dims(ins["attrs"].get("rhs_group_dims", "")) == [0]
            r = np.zeros((a_.shape[0], b_.shape[3 - rc[0]]), np.float32)
            start = 0
            for g, n in enumerate(sizes):
                n = max(0, min(n, a_.shape[0] - start))
                if n:
                    r[start:start + n] = _dot(a_[start:start + n], b_[g], [1], [rc[0] - 1], [], [])
                start += n
            v = _round(r, ty)
        elif op == "negate":
            v = _round(-np.asarray(x[0], np.float32), ty)
        elif op == "abs":
            v = _round(np.abs(np.asarray(x[0], np.float32)), ty)
        elif op == "sqrt":
            v = _round(np.sqrt(np.asarray(x[0], np.float32)), ty)
        elif op == "rsqrt":
            # the portable definition (xla/codegen/intrinsic/rsqrt.cc:178-193): 1 / sqrt(x), each op rounded.
            # PARITY UNPINNED against hosts that take the x86 approximation instruction plus Newton steps
            with np.errstate(all="ignore"):
                v = _round(np.float32(1) / np.sqrt(np.asarray(x[0], np.float32)), ty)
        elif op == "exponential":
            v = _round(O.exp_f32(np.asarray(x[0], np.float32)), ty)
        elif op == "tanh":
            v = _round(O.tanh_f32(np.asarray(x[0], np.float32)), ty)
        elif op == "logistic":
            e = O.exp_f32(-np.asarray(x[0], np.float32))
            v = _round(np.float32(1) / (np.float32(1) + e), ty)
        elif op == "clamp":
            lo, val, hi = (np.asarray(t, np.float32) for t in x)
            v = _round(np.minimum(np.maximum(val, lo), hi), ty)
        elif op == "dot":
            a = ins["attrs"]
            r = _dot(x[0], x[1], _dims(a.get("lhs_contracting_dims", "")), _dims(a.get("rhs_contracting_dims", "")),
                     _dims(a.get("lhs_batch_dims", "")), _dims(a.get("rhs_batch_dims", "")))
            v = _round(r, ty)
        elif op == "reduce":
            dims = _dims(ins["attrs"]["dimensions"])
            kind = reducer_kind(ins["attrs"]["to_apply"])
            if kind == "maximum" and sorted(dims) == list(range(np.asarray(x[0]).ndim)):
                # over everything: order-free, NaN passed on (np.max and np.maximum both do)
                v = _round(np.maximum(np.max(np.asarray(x[0], np.float32)), np.asarray(x[1], np.float32)), ty)
                env[ins["name"]] = v
                continue
            assert dims == [np.asarray(x[0]).ndim - 1], "only reductions over the minor dimension"
            if kind == "add":
                v = _round(_tree32_sum_last(x[0]), ty)
            elif kind == "maximum":
                v = _round(np.maximum(np.max(np.asarray(x[0], np.float32), axis=-1), np.asarray(x[1], np.float32)), ty)
            else:
                raise NotImplementedError("reduce with " + kind)
        elif op == "custom-call" and ins["attrs"].get("custom_call_target", "").strip('"') == "__op$block_scaled_dot":
            # what BlockScalingRewriter expands it to (block_scaling_rewriter.cc:194-219, :521-571):
            # convert, multiply by the scale of each block of the minor dimension, contract minor with minor
            a8, b8, sa, sb = x
            blk = a8.shape[-1] // sa.shape[-1]
            ad = _round(O.f8e4m3fn_to_f32(a8) * np.repeat(O.f8e8m0fnu_to_f32(sa), blk, axis=-1), ty)
            bd = _round(O.f8e4m3fn_to_f32(b8) * np.repeat(O.f8e8m0fnu_to_f32(sb), blk, axis=-1), ty)
            lead = list(range(ad.ndim - 2))  # a batch dimension, if present, is the major one (block_scaling_rewriter.h:53)
            v = _round(_dot(ad, bd, [ad.ndim - 1], [bd.ndim - 1], lead, lead), ty)
        elif op == "tuple":
            v = list(x)
        elif op == "get-tuple-element":
            v = x[0][int(ins["attrs"]["index"])]
        else:
            raise NotImplementedError("opcode " + op)
        env[ins["name"]] = v

    root = next(i for i in entry["instructions"] if i["root"])

    def export(v, shape):
        if isinstance(v, list):
            return [export(e, s) for e, s in zip(v, shape["tuple"])]
        if shape["dtype"] == "bf16":
            return O.f32_to_bf16(np.ascontiguousarray(v, np.float32))
        return np.ascontiguousarray(v)

    return export(env[root["name"]], root["shape"])
