"""Runs a rewritten HLO module on the GPU the way XLA's thunk sequence would: walks the entry
computation in order and, for every ``custom-call`` with ``API_VERSION_TYPED_FFI``, looks the
target up in the FFI registry for platform "rocm" and invokes the handler with a call frame
built from the instruction -- flattened tuple results, logical dimensions, attributes parsed
from the MLIR dictionary in ``backend_config`` (xla/service/gpu/thunk_emitter.cc:1235-1369,
xla/backends/gpu/runtime/custom_call_thunk.cc:110-157).

Only what a rewritten quantized-inference module contains is supported besides the custom
calls: parameters, tuples, get-tuple-element, and scalar glue (constants, converts and
divides of rank-0 values, converts of rank-1 scale vectors, a rank-1 broadcast of a scalar), which
run as torch ops.  Anything else raises: this is not an HLO
interpreter, and a module the pass did not fully rewrite does not run here.
"""
import re

import torch

from . import dtypes, ffi, hlo

_TORCH = {"f32": torch.float32, "bf16": torch.bfloat16, "s8": torch.int8, "u8": torch.uint8,
          "f8e4m3fn": torch.uint8, "f8e8m0fnu": torch.uint8, "s4": torch.uint8, "u4": torch.uint8,
          "s32": torch.int32, "s64": torch.int64}
_DT = {"f32": dtypes.F32, "bf16": dtypes.BF16, "s8": dtypes.S8, "u8": dtypes.U8, "s4": dtypes.S4, "u4": dtypes.U4,
       "s32": dtypes.S32, "s64": dtypes.S64, "f8e4m3fn": dtypes.F8E4M3FN, "f8e8m0fnu": dtypes.F8E8M0FNU}


def parse_backend_config(cfg):
    """'"{a = \\"X\\", b = 3 : i32, c = true, d = 1e-06 : f32}"' -> {name: ffi.Attr}."""
    s = cfg.strip()
    if s.startswith('"') and s.endswith('"'):
        s = s[1:-1].replace('\\"', '"')
    s = s.strip()
    if not (s.startswith("{") and s.endswith("}")):
        raise ValueError("backend_config is not an MLIR dictionary: " + cfg)
    out = {}
    for m in re.finditer(r'(\w+)\s*=\s*("(?:[^"\\]|\\.)*"|[^,{}]+)', s[1:-1]):
        key, val = m.group(1), m.group(2).strip()
        if val.startswith('"'):
            out[key] = ffi.Attr.str(val[1:-1])
            continue
        ty = None
        if ":" in val:
            val, ty = (t.strip() for t in val.split(":", 1))
        if val in ("true", "false"):
            out[key] = ffi.Attr.pred(val == "true")
        elif ty == "i32":
            out[key] = ffi.Attr.i32(int(val))
        elif ty in ("i64", None) and re.fullmatch(r"-?\d+", val):
            out[key] = ffi.Attr.i64(int(val))
        elif ty == "f64":
            out[key] = ffi.Attr.f64(float(val))
        else:
            out[key] = ffi.Attr.f32(float(val))
    return out


class Executable:
    """A rewritten module bound to the registry of an FFI host."""

    def __init__(self, text, host=None):
        self.text = text
        self.module = hlo.to_json(text)
        self.host = host or ffi.NativeHost()
        if not getattr(self.host, "_registered", False):
            self.host.register()
            self.host._registered = True
        self.entry = next(c for c in self.module["computations"] if c["entry"])
        for ins in self.entry["instructions"]:
            if ins["opcode"] == "custom-call":
                target = ins["attrs"]["custom_call_target"].strip('"')
                if not self.host.find_handler(target, "rocm"):
                    # XLA fails compilation here too (custom_call_thunk.cc:188-189)
                    raise LookupError("no FFI handler registered for custom call target '%s' on "
                                      "platform rocm" % target)

    def run(self, args):
        """args: device tensors in parameter order (s4 weights as packed uint8).  Returns the
        root value (a list for a tuple)."""
        env, shapes = {}, {}
        self.host.stream = torch.cuda.current_stream().cuda_stream
        for ins in self.entry["instructions"]:
            op, sh = ins["opcode"], ins["shape"]
            x = [env[o] for o in ins["operands"]]
            if op == "parameter":
                v = args[int(ins["literal"])]
            elif op == "custom-call":
                v = self._call(ins, x, [shapes[o] for o in ins["operands"]])
            elif op == "get-tuple-element":
                v = x[0][int(ins["attrs"]["index"])]
            elif op == "tuple":
                v = list(x)
            elif not sh.get("tuple") and (sh["dims"] == [] or (op in ("convert", "broadcast") and len(sh["dims"]) == 1)):
                # scalars, the widening convert of a vector of scales, a vector of one repeated scalar
                v = self._scalar_glue(ins, x)
            else:
                raise NotImplementedError("instruction %s = %s(...) was not rewritten into a custom call; "
                                          "this runner only executes custom calls" % (ins["name"], op))
            env[ins["name"]], shapes[ins["name"]] = v, sh
        root = next(i for i in self.entry["instructions"] if i["root"])
        return env[root["name"]]

    @staticmethod
    def _scalar_glue(ins, x):
        op, ty = ins["opcode"], _TORCH[ins["shape"]["dtype"]]
        if op == "constant":
            return torch.tensor(float(ins["literal"].strip("{} ")), dtype=ty, device="cuda")
        if op == "convert":
            return x[0].to(ty)
        if op == "broadcast" and x[0].dim() == 0:
            return x[0].to(ty).expand(ins["shape"]["dims"]).contiguous()
        if op == "divide":
            return (x[0] / x[1]).to(ty)
        if op == "multiply":
            return (x[0] * x[1]).to(ty)
        raise NotImplementedError("scalar op " + op)

    def _call(self, ins, operands, operand_shapes):
        target = ins["attrs"]["custom_call_target"].strip('"')
        if ins["attrs"].get("api_version") != "API_VERSION_TYPED_FFI":
            raise ValueError("custom call %s does not use the typed FFI" % ins["name"])
        res_shapes = ins["shape"]["tuple"] if "tuple" in ins["shape"] else [ins["shape"]]
        results = [torch.empty(s["dims"], dtype=_TORCH[s["dtype"]], device="cuda") for s in res_shapes]
        args = [(_DT[s["dtype"]], t.data_ptr(), s["dims"]) for t, s in zip(operands, operand_shapes)]
        rets = [(_DT[s["dtype"]], t.data_ptr(), s["dims"]) for t, s in zip(results, res_shapes)]
        attrs = parse_backend_config(ins["attrs"].get("backend_config", '"{}"'))
        frame = ffi.Frame(self.host, args, rets, attrs)
        ffi.invoke(target, frame)
        return results if "tuple" in ins["shape"] else results[0]


def compile_and_run(text, args):
    """rewrite -> bind -> run; returns (result, rewrites, refusals)."""
    new_text, rewrites, refusals = hlo.rewrite(text)
    return Executable(new_text).run(args), rewrites, refusals
