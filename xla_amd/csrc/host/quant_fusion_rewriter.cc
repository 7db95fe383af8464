// QuantFusionRewriter: matches the quantized-inference patterns in an HLO module and replaces
// each with one typed-FFI custom call to this library's kernels, in the place where XLA's
// GemmFusion / GemmRewriter run (xla/service/gpu/gpu_compiler.cc:2113-2129):
//
//   convert(f8e4m3fn) [* or / broadcast(scalar) | * broadcast(per-row / per-channel vector)]
//       -> dot [-> +bias] [-> relu|gelu|silu]
//       => xla_amd.fp8_scaled_dot          (what gemm_rewriter.cc:190-336,1235-1591 turns into
//                                           __cublas$lt$matmul$f8, epilogues :888-1007,1987-2304)
//   (convert(s8|s4|u4) [- zero points]) * broadcast(scale) -> dot | ragged-dot [-> +bias] [-> activation]
//       => xla_amd.dequant_dot             (what gemm_fusion.cc:1629-1702 wraps into __triton_gemm;
//                                           pattern zoo: fusion_emitter_int4_device_test.cc:85-449)
//   custom-call "__op$block_scaled_dot" (f8e4m3fn operands, f8e8m0fnu scales per 32 of K)
//       => xla_amd.fp8_scaled_dot with block scales (block_scaling_rewriter.h:48-69)
//   [RMSNorm ->] reduce-max(abs) -> /448 -> divide -> clamp -> convert(f8e4m3fn)
//       => xla_amd.rowwise_quantize_fp8    (today: several reduction/loop fusions,
//                                           codegen/emitters/reduction.cc:840-991)
//
// Every refusal is recorded with a reason (the reference logs them with VLOG(1),
// gemm_rewriter.cc:295,316,1248).  The kernels produce bf16 (f8 for the quantizer; the dequantize-dot
// also the f32 value itself), so a pattern is only taken when the value leaving it has such a type.
#include "quant_fusion_rewriter.h"

#include <math.h>
#include <stdio.h>
#include <stdlib.h>

#include <algorithm>
#include <functional>
#include <set>

namespace xla_amd {
namespace hlo {
namespace {

bool IsFloatTy(const std::string& t) { return t == "f32" || t == "bf16"; }
int DTypeCode(const std::string& t) { return t == "bf16" ? 16 : 11; }  // XLA PrimitiveType values

std::unique_ptr<Instr> Make(const std::string& name, const std::string& opcode, Shape shape,
                            std::vector<Instr*> operands) {
  auto i = std::make_unique<Instr>();
  i->name = name;
  i->opcode = opcode;
  i->shape = std::move(shape);
  i->operands = std::move(operands);
  return i;
}

// Scalar constant value, looking through broadcast and convert.
bool ConstScalar(const Instr* i, double* v) {
  while (i->Is("broadcast") || i->Is("convert") || i->Is("reshape") || i->Is("bitcast")) i = i->operands[0];
  if (!i->Is("constant") || i->shape.num_elements() != 1) return false;
  std::string lit = i->literal;
  lit.erase(std::remove_if(lit.begin(), lit.end(), [](char c) { return c == '{' || c == '}' || c == ' '; }),
            lit.end());
  if (lit == "inf") { *v = INFINITY; return true; }
  if (lit == "-inf") { *v = -INFINITY; return true; }
  char* end = nullptr;
  *v = strtod(lit.c_str(), &end);
  return end && *end == 0 && !lit.empty();
}

bool IsConst(const Instr* i, double want) {
  double v;
  return ConstScalar(i, &v) && v == want;
}

// A constant close to `want` by the rule of BcastConstScalarNear (gemm_rewriter.cc:472-503):
// |actual - want| < |actual + want| * 128 * epsilon of the constant's own element type.
bool IsConstNear(const Instr* i, double want) {
  double v;
  if (!ConstScalar(i, &v)) return false;
  const Instr* c = i;
  while (!c->Is("constant")) c = c->operands[0];
  double eps;
  if (c->shape.dtype == "f16") eps = 0x1p-10;
  else if (c->shape.dtype == "bf16") eps = 0x1p-7;
  else if (c->shape.dtype == "f32") eps = 0x1p-23;
  else if (c->shape.dtype == "f64") eps = 0x1p-52;
  else return false;
  return fabs(v - want) < fabs(v + want) * 128 * eps;
}

// broadcast of a rank-0 value (dimensions={})
bool ScalarBroadcast(const Instr* i, Instr** scalar) {
  if (!i->Is("broadcast") || i->operands[0]->shape.rank() != 0) return false;
  *scalar = i->operands[0];
  return true;
}

// broadcast(src), dimensions=dims
bool BroadcastAlong(const Instr* i, const std::vector<int64_t>& dims, Instr** src) {
  if (!i->Is("broadcast") || i->DimsAttr("dimensions") != dims) return false;
  *src = i->operands[0];
  return true;
}

bool Binary(const Instr* i, const char* op, Instr** a, Instr** b) {
  if (!i->Is(op) || i->operands.size() != 2) return false;
  *a = i->operands[0];
  *b = i->operands[1];
  return true;
}

// Commutative binary op with one side satisfying `pred`; *other receives the other side.
bool BinaryWith(const Instr* i, const char* op, const std::function<bool(Instr*)>& pred, Instr** other) {
  Instr *a, *b;
  if (!Binary(i, op, &a, &b)) return false;
  if (pred(b)) { *other = a; return true; }
  if (pred(a)) { *other = b; return true; }
  return false;
}

// convert whose operand has element type `from`
bool ConvertFrom(const Instr* i, const std::string& from, Instr** src) {
  if (!i->Is("convert") || i->operands[0]->shape.dtype != from) return false;
  *src = i->operands[0];
  return true;
}

std::string I32(int v) { return std::to_string(v) + " : i32"; }

struct Epilogue {
  Instr* tail = nullptr;     // last instruction absorbed (its value is what the custom call returns)
  Instr* bias = nullptr;     // [N] operand, bf16 or f32 (null if none)
  std::string act = "";      // "", RELU, GELU, SILU
  std::string ops_type;      // element type of the bias add / activation ops
  Instr* d_scale = nullptr;  // f8 result: the scalar the value is divided (or multiplied) by
  bool d_multiplies = false;
  Instr* amax = nullptr;     // f8 result: reduce-maximum of abs(value) over everything, if the module has one
  std::string Name() const {
    std::string a = act.empty() ? "" : act;
    if (bias) return a.empty() ? "BIAS" : "BIAS_" + a;
    return a.empty() ? "DEFAULT" : a;
  }
};

Instr* SoleUser(Instr* i) { return i->users.size() == 1 ? i->users[0] : nullptr; }

// tanh-GELU rooted at `out` = x * cdf, with the op structure of gemm_rewriter.cc:923-973:
//   cdf = 0.5 * (1 + tanh(c1 * (x + c0 * (x*x*x))))
bool MatchGelu(Instr* out, Instr* x) {
  Instr* cdf;
  if (!BinaryWith(out, "multiply", [&](Instr* s) { return s == x; }, &cdf)) return false;
  Instr* onep;
  if (!BinaryWith(cdf, "multiply", [](Instr* s) { return IsConst(s, 0.5); }, &onep)) return false;
  Instr* th;
  if (!BinaryWith(onep, "add", [](Instr* s) { return IsConst(s, 1.0); }, &th)) return false;
  if (!th->Is("tanh")) return false;
  Instr* inner;
  if (!BinaryWith(th->operands[0], "multiply", [](Instr* s) { return IsConstNear(s, 0.7978845608028654); }, &inner))
    return false;
  Instr* cube_term;
  if (!BinaryWith(inner, "add", [&](Instr* s) { return s == x; }, &cube_term)) return false;
  Instr* cube;
  if (!BinaryWith(cube_term, "multiply", [](Instr* s) { return IsConstNear(s, 0.044715); }, &cube)) return false;
  Instr* sq;
  if (!BinaryWith(cube, "multiply", [&](Instr* s) { return s == x; }, &sq)) return false;
  Instr *a, *b;
  return Binary(sq, "multiply", &a, &b) && a == x && b == x;
}

// x * (1 / (1 + exp(-x)))  (gemm_rewriter.cc:995-1002) or x * logistic(x)
bool MatchSilu(Instr* out, Instr* x) {
  Instr* sg;
  if (!BinaryWith(out, "multiply", [&](Instr* s) { return s == x; }, &sg)) return false;
  if (sg->Is("logistic")) return sg->operands[0] == x;
  Instr *one, *den;
  if (!Binary(sg, "divide", &one, &den) || !IsConst(one, 1.0)) return false;
  Instr* ex;
  if (!BinaryWith(den, "add", [](Instr* s) { return IsConst(s, 1.0); }, &ex)) return false;
  return ex->Is("exponential") && ex->operands[0]->Is("negate") && ex->operands[0]->operands[0] == x;
}

// Walks forward from the dot: optional convert, optional + broadcast(bias) along the minor
// dimension, optional activation, optional final convert to bf16.  Returns false when what
// leaves the chain is not bf16.
// allow_f32_result: the kernels behind the call can write the f32 value itself (the dequantize-dot);
// otherwise the value leaving the pattern must be bf16.  allow_amax: the handler can also return the
// amax of an f8 result; without it a value that feeds its own amax is left to the ops after the call.
bool MatchEpilogue(Instr* dot, Epilogue* ep, std::string* why, const Module* f8_result_in = nullptr,
                   bool allow_f32_result = false, bool allow_amax = true) {
  const bool allow_f8_result = f8_result_in != nullptr;
  Instr* cur = dot;
  const int64_t rank = dot->shape.rank();
  ep->ops_type = dot->shape.dtype;
  auto step_convert = [&]() {
    Instr* u = SoleUser(cur);
    if (u && u->Is("convert") && IsFloatTy(u->shape.dtype) && u->shape.dtype != cur->shape.dtype) {
      cur = u;
      return true;
    }
    return false;
  };
  Instr* after_dot = cur;
  if (step_convert()) ep->ops_type = cur->shape.dtype;
  // bias: add(cur, broadcast(bias[N]), dimensions={rank-1})
  if (Instr* u = SoleUser(cur)) {
    Instr* bsrc = nullptr;
    Instr* bb = nullptr;
    if (BinaryWith(u, "add", [&](Instr* s) { return BroadcastAlong(s, {rank - 1}, &bsrc) && s != cur; }, &bb) &&
        bb == cur && bsrc->shape.rank() == 1) {
      Instr* raw = bsrc;
      Instr* inner;
      if (bsrc->Is("convert") && ConvertFrom(bsrc, "bf16", &inner) && bsrc->shape.dtype == "f32") raw = inner;
      if (IsFloatTy(raw->shape.dtype)) {
        ep->bias = raw;
        cur = u;
      }
    }
  }
  // activation on cur
  {
    // the activation's result is the unique multiply/maximum that consumes cur last; find it
    // among cur's (transitive) users by trying each candidate root.
    std::vector<Instr*> frontier = cur->users;
    std::set<Instr*> seen;
    Instr* found = nullptr;
    std::string act;
    while (!frontier.empty() && !found) {
      Instr* c = frontier.back();
      frontier.pop_back();
      if (!seen.insert(c).second) continue;
      Instr* other;
      if (c->Is("maximum") && BinaryWith(c, "maximum", [](Instr* s) { return IsConst(s, 0.0); }, &other) &&
          other == cur) {
        found = c;
        act = "RELU";
      } else if (c->Is("multiply") && MatchGelu(c, cur)) {
        found = c;
        act = "GELU";
      } else if (c->Is("multiply") && MatchSilu(c, cur)) {
        found = c;
        act = "SILU";
      } else if (seen.size() < 24) {
        for (Instr* u : c->users) frontier.push_back(u);
      }
    }
    if (found) {
      // every value between cur and found must stay inside the pattern
      std::set<Instr*> inside;
      std::function<void(Instr*)> collect = [&](Instr* n) {
        if (n == cur || !inside.insert(n).second) return;
        for (Instr* op : n->operands)
          if (!op->Is("constant") && !op->Is("broadcast")) collect(op);
      };
      collect(found);
      bool closed = true;
      for (Instr* n : inside)
        if (n != found)
          for (Instr* u : n->users) closed &= inside.count(u) > 0;
      for (Instr* u : cur->users) closed &= inside.count(u) > 0;
      if (closed) {
        ep->act = act;
        cur = found;
      }
    }
  }
  if (cur != after_dot && cur != dot) ep->ops_type = cur->shape.dtype;
  if (!ep->bias && ep->act.empty()) ep->ops_type = dot->shape.dtype;  // nothing between dot and result
  // f8 result: convert(clamp(-448, cur / broadcast(z) | cur * broadcast(z), 448)) on f32-typed ops
  // (gemm_rewriter_fp8_test.cc:1665-1690, :1730-1748)
  if (allow_f8_result && cur->shape.dtype == "f32" && dot->shape.dtype == "f32" && ep->ops_type == "f32") {
    // the value may also feed its own amax: reduce(abs(cur), -inf) over both dimensions with a
    // maximum (gemm_rewriter_fp8_test.cc:2559-2600)
    Instr* sc = SoleUser(cur);
    Instr* amax = nullptr;
    if (!sc && allow_amax && cur->users.size() == 2) {
      for (int which = 0; which < 2 && !amax; ++which) {
        Instr* ab = cur->users[which];
        Instr* rd = ab->Is("abs") ? SoleUser(ab) : nullptr;
        if (!rd || !rd->Is("reduce") || rd->operands.size() != 2 || rd->operands[0] != ab) continue;
        std::vector<int64_t> all_dims;
        for (int64_t i = 0; i < rank; ++i) all_dims.push_back(i);
        if (rd->DimsAttr("dimensions") != all_dims || !rd->operands[1]->Is("constant") ||
            rd->operands[1]->literal != "-inf")
          continue;
        const std::string* to = rd->Attr("to_apply");
        std::string name = to ? *to : "";
        if (!name.empty() && name[0] == '%') name = name.substr(1);
        const Computation* body = f8_result_in->FindComputation(name);
        if (!body || !body->root() || !body->root()->Is("maximum")) continue;
        amax = rd;
        sc = cur->users[1 - which];
      }
    }
    Instr *val = nullptr, *z = nullptr, *bz = nullptr;
    bool mul = false, ok = false;
    if (sc && Binary(sc, "divide", &val, &bz) && val == cur && ScalarBroadcast(bz, &z)) ok = true;
    else if (sc && BinaryWith(sc, "multiply", [&](Instr* b) { return ScalarBroadcast(b, &z); }, &val) && val == cur)
      ok = mul = true;
    if (ok && z->shape.dtype == "f32") {
      Instr* cl = SoleUser(sc);
      if (cl && cl->Is("clamp") && cl->operands.size() == 3 && cl->operands[1] == sc &&
          IsConst(cl->operands[0], -448.0) && IsConst(cl->operands[2], 448.0)) {
        Instr* cv = SoleUser(cl);
        if (cv && cv->Is("convert") && cv->shape.dtype == "f8e4m3fn") {
          ep->d_scale = z;
          ep->d_multiplies = mul;
          ep->amax = amax;
          ep->tail = cv;
          return true;
        }
      }
    }
  }
  step_convert();
  if (cur->shape.dtype != "bf16" && !(allow_f32_result && cur->shape.dtype == "f32")) {
    *why = "the value leaving the dot pattern is " + cur->shape.dtype + ", the kernels produce bf16";
    return false;
  }
  ep->tail = cur;
  return true;
}

std::string CommonConfig(const Epilogue& ep, const std::string& dequant_ty, const std::string& dot_ty) {
  return "epilogue = \\\"" + ep.Name() + "\\\", dequant_type = " + I32(DTypeCode(dequant_ty)) +
         ", dot_type = " + I32(DTypeCode(dot_ty)) + ", epilogue_type = " + I32(DTypeCode(ep.ops_type));
}

// Emits `(result, scratch) custom-call(...)` + get-tuple-element 0 before `before`, and moves
// the uses of `tail` to it.
Instr* EmitCall(Computation* comp, Instr* tail, const std::string& target, std::vector<Instr*> operands,
                std::vector<Shape> results, const std::string& config) {
  Shape shape = results.size() == 1 ? results[0] : Shape::Tuple(results);
  auto cc = Make(comp->UniqueName(tail->name + ".call"), "custom-call", shape, std::move(operands));
  cc->attrs.emplace_back("custom_call_target", "\"" + target + "\"");
  cc->attrs.emplace_back("api_version", "API_VERSION_TYPED_FFI");
  cc->attrs.emplace_back("backend_config", "\"{" + config + "}\"");
  return comp->Insert(std::move(cc), tail);
}

Instr* EmitGte(Computation* comp, Instr* call, int index, const Instr* before, const std::string& name) {
  auto g = Make(comp->UniqueName(name), "get-tuple-element", call->shape.elements[index], {call});
  g->attrs.emplace_back("index", std::to_string(index));
  return comp->Insert(std::move(g), before);
}

Instr* AsF32Scalar(Computation* comp, Instr* s, const Instr* before) {
  if (s->shape.dtype == "f32") return s;
  return comp->Insert(Make(comp->UniqueName(s->name + ".f32"), "convert", Shape::Array("f32", {}), {s}), before);
}

// ---------------------------------------------------------------- f8 scaled dot
struct F8Operand {
  Instr* value = nullptr;   // the f8e4m3fn tensor
  Instr* scale = nullptr;   // scalar or vector, null = 1
  bool divide = false;
  int64_t scale_dim = -1;   // the operand dimension a rank-1 scale runs along; -1 for a scalar
  std::string type;         // element type of the convert / multiply
};

// broadcast(scalar), or broadcast(vector) along one dimension of a rank-2 operand
bool ScaleBroadcast(const Instr* i, Instr** scale, int64_t* dim) {
  *dim = -1;
  if (ScalarBroadcast(i, scale)) return true;
  if (!i->Is("broadcast") || i->shape.rank() != 2 || i->operands[0]->shape.rank() != 1) return false;
  auto dims = i->DimsAttr("dimensions");
  if (dims.size() != 1 || dims[0] < 0 || dims[0] > 1) return false;
  *scale = i->operands[0];
  *dim = dims[0];
  return true;
}

bool MatchF8Operand(Instr* op, F8Operand* out) {
  Instr* src;
  if (ConvertFrom(op, "f8e4m3fn", &src)) {
    *out = {src, nullptr, false, -1, op->shape.dtype};
    return IsFloatTy(op->shape.dtype);
  }
  Instr *cv = nullptr, *sc = nullptr;
  if (op->Is("multiply")) {
    if (!BinaryWith(op, "multiply", [&](Instr* s) { return ScaleBroadcast(s, &sc, &out->scale_dim); }, &cv))
      return false;
  } else if (op->Is("divide")) {
    Instr* b;
    if (!Binary(op, "divide", &cv, &b) || !ScaleBroadcast(b, &sc, &out->scale_dim)) return false;
    out->divide = true;
  } else {
    return false;
  }
  if (!ConvertFrom(cv, "f8e4m3fn", &src) || cv->shape.dtype != op->shape.dtype || !IsFloatTy(op->shape.dtype))
    return false;
  if (sc->shape.dtype != op->shape.dtype && !(sc->Is("convert") || IsFloatTy(sc->shape.dtype))) return false;
  out->value = src;
  out->scale = sc;
  out->type = op->shape.dtype;
  return true;
}

bool RewriteF8Dot(const Module& mod, Computation* comp, Instr* dot, const RewriteOptions& opt, RewriteLog* log) {
  F8Operand a, b;
  if (!MatchF8Operand(dot->operands[0], &a) || !MatchF8Operand(dot->operands[1], &b)) return false;
  auto refuse = [&](const std::string& why) {
    log->refusals.push_back(dot->name + ": f8 operands found but not rewritten: " + why);
    return false;
  };
  if (a.type != b.type) return refuse("operands are dequantised in different types");
  // [M,K] . [K,N]|[N,K], or the same with one leading batch dimension on both operands
  // (gemm_rewriter_fp8_test.cc:941-957)
  const int64_t rank = dot->shape.rank();
  if ((rank != 2 && rank != 3) || a.value->shape.rank() != rank || b.value->shape.rank() != rank)
    return refuse("only rank-2 dots and rank-3 dots with one batch dimension are supported");
  const int64_t lead = rank - 2;
  const std::vector<int64_t> want_batch = lead ? std::vector<int64_t>{0} : std::vector<int64_t>{};
  if (dot->DimsAttr("lhs_batch_dims") != want_batch || dot->DimsAttr("rhs_batch_dims") != want_batch)
    return refuse(lead ? "the batch dimension must be the leading one of both operands"
                       : "batch dimensions are not supported on rank-2 operands");
  auto lc = dot->DimsAttr("lhs_contracting_dims"), rc = dot->DimsAttr("rhs_contracting_dims");
  if (lc.size() != 1 || rc.size() != 1 || lc[0] != rank - 1 || rc[0] < lead)
    return refuse("lhs must contract its minor dimension");
  rc[0] -= lead;  // from here on: 0 = rhs [K,N], 1 = rhs [N,K]
  if (lead && (a.scale_dim >= 0 || b.scale_dim >= 0)) return refuse("a batched dot takes per-tensor scales");
  if (!IsFloatTy(dot->shape.dtype)) return refuse("dot result type " + dot->shape.dtype);
  Epilogue ep;
  std::string why;
  if (!MatchEpilogue(dot, &ep, &why, /*f8_result_in=*/&mod)) return refuse(why);

  const int64_t M = a.value->shape.dims[lead], K = a.value->shape.dims[lead + 1];
  const int64_t N = b.value->shape.dims[lead + 1 - rc[0]];
  std::vector<int64_t> out_dims = {M, N};
  if (lead) out_dims.insert(out_dims.begin(), a.value->shape.dims[0]);
  // a vector of scales must run along the operand's free dimension (rows of a, output channels
  // of b): along K it does not factor out of the sum
  if (a.scale_dim == 1) return refuse("the lhs scales vary along the contracting dimension");
  if (b.scale_dim == rc[0]) return refuse("the rhs scales vary along the contracting dimension");
  if ((a.scale_dim >= 0 && a.divide) || (b.scale_dim >= 0 && b.divide))
    return refuse("a division by a vector of scales is not taken");
  auto scale_of = [&](const F8Operand& o) -> Instr* {
    Instr* s = o.scale;
    if (!s) {
      auto one = Make(comp->UniqueName("one"), "constant", Shape::Array("f32", {}), {});
      one->literal = "1";
      return comp->Insert(std::move(one), ep.tail);
    }
    if (o.scale_dim >= 0) {
      if (s->shape.dtype == "f32") return s;
      return comp->Insert(Make(comp->UniqueName(s->name + ".f32"), "convert", Shape::Array("f32", s->shape.dims), {s}),
                          ep.tail);
    }
    s = AsF32Scalar(comp, s, ep.tail);
    if (o.divide) {
      auto one = Make(comp->UniqueName("one"), "constant", Shape::Array("f32", {}), {});
      one->literal = "1";
      Instr* o1 = comp->Insert(std::move(one), ep.tail);
      s = comp->Insert(Make(comp->UniqueName(s->name + ".rcp"), "divide", Shape::Array("f32", {}), {o1, s}), ep.tail);
    }
    return s;
  };
  std::vector<Instr*> ops = {a.value, b.value, scale_of(a), scale_of(b)};
  if (ep.bias) ops.push_back(ep.bias);
  if (ep.d_scale) ops.push_back(ep.d_scale);
  std::vector<Shape> results = {Shape::Array(ep.d_scale ? "f8e4m3fn" : "bf16", out_dims)};
  if (ep.amax) results.push_back(Shape::Array("f32", {}));
  size_t ws = opt.fp8_workspace_bytes ? opt.fp8_workspace_bytes(M, K, N, (int32_t)rc[0], DTypeCode(a.type)) : 0;
  if (ws) results.push_back(Shape::Array("s8", {(int64_t)ws}));
  std::string cfg = CommonConfig(ep, a.type, dot->shape.dtype) + ", rhs_contracting_dim = " +
                    std::to_string(rc[0]) + " : i64";
  if (ep.d_scale) cfg += std::string(", d_scale_multiplies = ") + (ep.d_multiplies ? "true" : "false");
  Instr* call = EmitCall(comp, ep.tail, "xla_amd.fp8_scaled_dot", ops, results, cfg);
  Instr* value = results.size() > 1 ? EmitGte(comp, call, 0, ep.tail, ep.tail->name + ".out") : call;
  comp->ReplaceAllUses(ep.tail, value);
  if (ep.amax) comp->ReplaceAllUses(ep.amax, EmitGte(comp, call, 1, ep.tail, ep.amax->name + ".amax"));
  log->rewrites.push_back(dot->name + " -> xla_amd.fp8_scaled_dot [" + ep.Name() + (ep.d_scale ? ", f8 result" : "") +
                          (ep.amax ? ", amax" : "") + "]");
  return true;
}

// ---------------------------------------------------------------- block-scaled (MXFP8) dot
// custom-call(lhs f8e4m3fn [M,K], rhs f8e4m3fn [N,K], lhs_scale f8e8m0fnu [M,K/32], rhs_scale
// [N,K/32]), custom_call_target="__op$block_scaled_dot" -> bf16 [M,N]
// (block_scaling_rewriter.h:48-69) becomes xla_amd.fp8_scaled_dot with the scales as they are:
// the matrix cores multiply them in.  BlockScalingRewriter would expand it into converts,
// multiplies and a dot on anything but cuDNN (block_scaling_rewriter.cc:548-571).
bool RewriteBlockScaledDot(Computation* comp, Instr* cc, const RewriteOptions& opt, RewriteLog* log) {
  const std::string* target = cc->Attr("custom_call_target");
  if (!target || *target != "\"__op$block_scaled_dot\"") return false;
  auto refuse = [&](const std::string& why) {
    log->refusals.push_back(cc->name + ": block-scaled dot found but not rewritten: " + why);
    return false;
  };
  if (cc->operands.size() != 4) return refuse("expected lhs, rhs and a scale for each");
  Instr *a = cc->operands[0], *b = cc->operands[1], *sa = cc->operands[2], *sb = cc->operands[3];
  if (a->shape.dtype != "f8e4m3fn" || b->shape.dtype != "f8e4m3fn" || sa->shape.dtype != "f8e8m0fnu" ||
      sb->shape.dtype != "f8e8m0fnu")
    return refuse("operands must be f8e4m3fn with f8e8m0fnu scales");
  // one leading batch dimension, on all of them or on none (block_scaling_rewriter.h:53: the batch
  // dimension, if present, is the major one)
  const int64_t rank = a->shape.rank();
  if ((rank != 2 && rank != 3) || b->shape.rank() != rank || sa->shape.rank() != rank || sb->shape.rank() != rank ||
      cc->shape.is_tuple || cc->shape.rank() != rank)
    return refuse("operands, scales and result must all be rank 2, or rank 3 with the batch dimension first");
  const int64_t lead = rank - 2;
  const int64_t M = a->shape.dims[lead], K = a->shape.dims[lead + 1], N = b->shape.dims[lead];
  std::vector<int64_t> sa_dims = {M, K / 32}, sb_dims = {N, K / 32}, out_dims = {M, N};
  if (lead) {
    const int64_t B = a->shape.dims[0];
    if (b->shape.dims[0] != B) return refuse("batch dimensions differ");
    for (auto* d : {&sa_dims, &sb_dims, &out_dims}) d->insert(d->begin(), B);
  }
  if (b->shape.dims[lead + 1] != K || K % 32 != 0 || sa->shape.dims != sa_dims || sb->shape.dims != sb_dims)
    return refuse("scales must be one per 32 elements of the contracting (minor) dimension");
  if (cc->Attr("backend_config")) return refuse("a backend_config (explicit block size, global scale) is not taken");
  if (!IsFloatTy(cc->shape.dtype) || cc->shape.dims != out_dims)
    return refuse("the result is " + cc->shape.dtype + ", the kernels produce bf16 [M,N] from a bf16 or f32 dot");
  // what follows the dot (bias, activation, the convert to bf16) goes into the call like behind an
  // ordinary dot; the value that leaves must be bf16
  Epilogue ep;
  std::string why;
  if (!MatchEpilogue(cc, &ep, &why)) return refuse(why);
  std::vector<Instr*> ops = {a, b, sa, sb};
  if (ep.bias) ops.push_back(ep.bias);
  std::string cfg = CommonConfig(ep, "f32", cc->shape.dtype) + ", rhs_contracting_dim = 1 : i64";
  std::vector<Shape> results = {Shape::Array("bf16", out_dims)};
  // scratch: the f32 sums of the K-slices of the kernels that take few rows of lhs, per batch
  size_t ws = opt.fp8_workspace_bytes ? opt.fp8_workspace_bytes(M, K, N, 1, DTypeCode("f32")) : 0;
  if (lead) ws *= (size_t)a->shape.dims[0];
  if (ws) results.push_back(Shape::Array("s8", {(int64_t)ws}));
  Instr* call = EmitCall(comp, ep.tail, "xla_amd.fp8_scaled_dot", ops, results, cfg);
  Instr* value = results.size() > 1 ? EmitGte(comp, call, 0, ep.tail, ep.tail->name + ".out") : call;
  comp->ReplaceAllUses(ep.tail, value);
  log->rewrites.push_back(cc->name + " -> xla_amd.fp8_scaled_dot [" + ep.Name() + ", block scales" +
                          (lead ? ", batched" : "") + "]");
  return true;
}

// ---------------------------------------------------------------- weight-only dequantize dot
struct QWeights {
  Instr* w = nullptr;       // s8, s4 or u4 tensor [B,]K,N -- or [B,]N,K (K minor)
  Instr* scale = nullptr;   // [N] | [G,N] | [B,N] | [B,G,N] -- K minor: [N] | [N,G] | [B,N] | [B,N,G]; bf16 or f32
  std::string type;         // element type of the multiply
  Instr* zero = nullptr;    // u4 zero points, shaped like the scales: (w - zero) * scale
  int64_t groups = 0;       // scales along K, 0 = one per output channel
};

// convert(s4 -> s8) or convert(u4 -> u8): how 4-bit values are often widened before the float convert
bool IsByteWidening(const Instr* s) {
  if (!s->Is("convert")) return false;
  const std::string& from = s->operands[0]->shape.dtype;
  return (s->shape.dtype == "s8" && from == "s4") || (s->shape.dtype == "u8" && from == "u4");
}

// integer tensor behind convert(s4->s8)? -> convert(->float)
bool IntSource(Instr* cv, const std::string& float_ty, Instr** w) {
  if (!cv->Is("convert") || cv->shape.dtype != float_ty) return false;
  Instr* s = cv->operands[0];
  if (IsByteWidening(s)) s = s->operands[0];
  if (s->shape.dtype != "s8" && s->shape.dtype != "s4" && s->shape.dtype != "u4") return false;
  *w = s;
  return true;
}

// v = subtract(x, broadcast(convert(u4 zero points -> ty)) along bdims): peels the subtraction off
bool PeelZeroPoint(Instr* v, const std::vector<int64_t>& bdims, const std::string& ty, Instr** x, Instr** zero) {
  if (!v->Is("subtract") || v->operands.size() != 2 || v->shape.dtype != ty) return false;
  Instr* zs = nullptr;
  if (!BroadcastAlong(v->operands[1], bdims, &zs)) return false;
  if (!zs->Is("convert") || zs->shape.dtype != ty || zs->operands[0]->shape.dtype != "u4") return false;
  *x = v->operands[0];
  *zero = zs->operands[0];
  return true;
}

Instr* LookThroughWidening(Instr* s, const std::string& to) {
  // convert(bf16 -> f32) of a scale is exact: hand the kernel the narrow original
  if (s->Is("convert") && to == "f32" && s->operands[0]->shape.dtype == "bf16") return s->operands[0];
  return s;
}

// k_minor: the weights are [B,]N,K (the dot contracts their minor dimension) instead of [B,]K,N.
bool MatchQWeights(Instr* op, bool k_minor, QWeights* out, std::string* why) {
  const std::string ty = op->shape.dtype;
  if (!IsFloatTy(ty)) return false;
  const int64_t rank = op->shape.rank();
  // grouped: reshape([G,g,N] product) -> [K,N], or with a leading batch / expert dimension
  // reshape([B,G,g,N] product) -> [B,K,N]; K minor: reshape([B,]N,G,g product) -> [B,]N,K
  if (op->Is("reshape") && (rank == 2 || rank == 3) && op->operands[0]->shape.rank() == rank + 1 &&
      op->operands[0]->Is("multiply")) {
    Instr* mul = op->operands[0];
    const int64_t lead = rank - 2;  // 0, or 1 with a batch dimension in front
    std::vector<int64_t> d3(mul->shape.dims.begin() + lead, mul->shape.dims.end());  // G, g, N -- or N, G, g
    if (k_minor) {
      if (d3[0] != op->shape.dims[lead] || d3[1] * d3[2] != op->shape.dims[lead + 1]) return false;
    } else if (d3[0] * d3[1] != op->shape.dims[lead] || d3[2] != op->shape.dims[lead + 1]) {
      return false;
    }
    if (lead && mul->shape.dims[0] != op->shape.dims[0]) return false;
    const std::vector<int64_t> bdims = k_minor ? (lead ? std::vector<int64_t>{0, 1, 2} : std::vector<int64_t>{0, 1})
                                               : (lead ? std::vector<int64_t>{0, 1, 3} : std::vector<int64_t>{0, 2});
    Instr *sc = nullptr, *cv = nullptr;
    if (!BinaryWith(mul, "multiply", [&](Instr* s) { return BroadcastAlong(s, bdims, &sc); }, &cv)) return false;
    Instr* zero = nullptr;
    PeelZeroPoint(cv, bdims, ty, &cv, &zero);
    // the convert may sit before or after the reshape to [G,g,N]
    Instr* w = nullptr;
    if (cv->Is("convert") && cv->operands[0]->Is("reshape")) {
      Instr* rs = cv->operands[0];
      Instr* src = rs->operands[0];
      if (IsByteWidening(src)) src = src->operands[0];
      if ((src->shape.dtype == "s8" || src->shape.dtype == "s4" || src->shape.dtype == "u4") && src->shape.rank() == rank)
        w = src;
    } else if (cv->Is("reshape")) {
      IntSource(cv->operands[0], ty, &w);
    }
    if (!w || w->shape.dims != op->shape.dims) {
      *why = "grouped dequantise: could not find the integer weights behind the reshape";
      return false;
    }
    sc = LookThroughWidening(sc, ty);
    if (sc->shape.rank() != rank || sc->shape.dims[lead] != d3[0] || sc->shape.dims[lead + 1] != d3[k_minor ? 1 : 2])
      return false;
    if (lead && sc->shape.dims[0] != op->shape.dims[0]) return false;
    *out = {w, sc, ty, zero, d3[k_minor ? 1 : 0]};
    return true;
  }
  if (op->Is("convert")) {
    // convert(s4|s8|u4 -> float) straight into the dot: no scale at all (Int4WeightsOnTheRhs / OnTheLhs,
    // fusion_emitter_int4_device_test.cc:495-606); the caller supplies scales of one
    Instr* w;
    if (!IntSource(op, ty, &w) || w->shape.dims != op->shape.dims) return false;
    *out = {w, nullptr, ty, nullptr, 0};
    return true;
  }
  if (!op->Is("multiply")) return false;
  Instr *sc = nullptr, *cv = nullptr;
  const std::vector<int64_t> bdims = k_minor ? (rank == 2 ? std::vector<int64_t>{0} : std::vector<int64_t>{0, 1})
                                             : (rank == 2 ? std::vector<int64_t>{1} : std::vector<int64_t>{0, 2});
  if (!BinaryWith(op, "multiply", [&](Instr* s) { return BroadcastAlong(s, bdims, &sc); }, &cv)) return false;
  Instr* zero = nullptr;
  PeelZeroPoint(cv, bdims, ty, &cv, &zero);
  Instr* w;
  if (!IntSource(cv, ty, &w) || w->shape.dims != op->shape.dims) return false;
  sc = LookThroughWidening(sc, ty);
  *out = {w, sc, ty, zero, 0};
  return true;
}

bool RewriteDequantDot(const Module& mod, Computation* comp, Instr* dot, const RewriteOptions& opt, RewriteLog* log) {
  QWeights q;
  std::string why;
  const int64_t rank = dot->shape.rank();
  auto lb = dot->DimsAttr("lhs_batch_dims"), rb = dot->DimsAttr("rhs_batch_dims");
  auto lc = dot->DimsAttr("lhs_contracting_dims"), rc = dot->DimsAttr("rhs_contracting_dims");
  // The dequantised weights are usually the rhs of the dot; they may be its lhs as well
  // (Int4WeightsOnTheLhs, fusion_emitter_int4_device_test.cc:495-523): the result is then [..,N,M].
  // Either operand may contract its minor or its major (non-batch) dimension: weights [..,K,N] or
  // [..,N,K] (:867-892), activations [..,M,K] or [..,K,M] (the shape table :609-645).
  bool weights_lhs = false;
  bool k_minor = rc == std::vector<int64_t>{rank - 1};
  if (!MatchQWeights(dot->operands[1], k_minor, &q, &why)) {
    std::string why_lhs;
    const bool lhs_k_minor = lc == std::vector<int64_t>{rank - 1};
    if (dot->operands.size() == 2 && MatchQWeights(dot->operands[0], lhs_k_minor, &q, &why_lhs)) {
      weights_lhs = true;
      k_minor = lhs_k_minor;
    } else {
      if (!why.empty()) log->refusals.push_back(dot->name + ": " + why);
      else if (!why_lhs.empty()) log->refusals.push_back(dot->name + ": " + why_lhs);
      return false;
    }
  }
  auto refuse = [&](const std::string& w) {
    log->refusals.push_back(dot->name + ": quantized weights found but not rewritten: " + w);
    return false;
  };
  Instr* lhs = dot->operands[weights_lhs ? 1 : 0];  // the activations
  const auto& ac = weights_lhs ? rc : lc;           // their contracting dimension, and the weights'
  const auto& wc = weights_lhs ? lc : rc;
  Instr* inner;
  if (lhs->Is("convert") && ConvertFrom(lhs, "bf16", &inner) && lhs->shape.dtype == "f32") lhs = inner;
  if (lhs->shape.dtype != "bf16") return refuse("the activation must be bf16 (or its convert to f32)");
  if (rank != 2 && rank != 3) return refuse("rank " + std::to_string(rank));
  if (rank == 3 && (lb != std::vector<int64_t>{0} || rb != std::vector<int64_t>{0}))
    return refuse("the batch dimension must be dimension 0 of both operands");
  if (rank == 2 && !lb.empty()) return refuse("unexpected batch dimensions");
  const bool lhs_k_major = ac == std::vector<int64_t>{rank - 2};
  if ((ac != std::vector<int64_t>{rank - 1} && !lhs_k_major) || (wc != std::vector<int64_t>{rank - 2} && !k_minor))
    return refuse("needs lhs [..,M,K] contracting K and weights [..,K,N] or [..,N,K]; s4 with a "
                  "minor batch dimension is rejected as in gemm_fusion.cc:1572-1590");
  // (4-bit rows of an odd number of values are packed across row ends, xla/packing.cc:142-170: the
  // one-thread-per-output kernel reads them by flat index)
  if (q.zero && q.w->shape.dtype != "u4") return refuse("zero points are taken with u4 weights only");
  if (q.zero && q.zero->shape.dims != q.scale->shape.dims)
    return refuse("zero points must have the shape of the scales (one per scale)");
  if (q.scale && q.type == "bf16" && q.scale->shape.dtype != "bf16") return refuse("bf16 multiply with non-bf16 scales");
  Epilogue ep;
  if (!MatchEpilogue(dot, &ep, &why, /*f8_result_in=*/&mod, /*allow_f32_result=*/true, /*allow_amax=*/false))
    return refuse(why);
  if (weights_lhs && (ep.bias || !ep.act.empty()))
    return refuse("with the weights as the lhs of the dot only the plain dot is taken (a bias would run along the other dimension)");

  const int64_t B = rank == 3 ? lhs->shape.dims[0] : 1;
  const int64_t M = lhs->shape.dims[rank - (lhs_k_major ? 1 : 2)], K = lhs->shape.dims[rank - (lhs_k_major ? 2 : 1)];
  const int64_t N = q.w->shape.dims[rank - (k_minor ? 2 : 1)];
  std::string dequant_ty = q.type;
  if (!q.scale) {
    // no multiply in the module: the integers themselves are the weights.  One scale per channel, all
    // ones, under an f32-typed multiply gives exactly those values (convert(int -> bf16) is exact).
    Instr* one = comp->Insert(Make(comp->UniqueName(dot->name + ".one"), "constant", Shape::Array("f32", {}), {}), dot);
    one->literal = "1";
    auto bc = Make(comp->UniqueName(dot->name + ".unit_scales"), "broadcast", Shape::Array("f32", {N}), {one});
    bc->attrs.emplace_back("dimensions", "{}");
    q.scale = comp->Insert(std::move(bc), dot);
    dequant_ty = "f32";
  }
  std::vector<Instr*> ops = {lhs, q.w, q.scale};
  if (q.zero) ops.push_back(q.zero);
  if (ep.bias) ops.push_back(ep.bias);
  if (ep.d_scale) ops.push_back(ep.d_scale);  // an f8e4m3fn result: its scale goes last
  std::vector<Shape> results = {Shape::Array(ep.tail->shape.dtype, dot->shape.dims)};
  const int32_t wdt = q.w->shape.dtype == "s4" ? 21 : q.w->shape.dtype == "u4" ? 22 : 2;
  auto sizer = k_minor ? opt.dequant_nk_workspace_bytes : opt.dequant_workspace_bytes;
  size_t ws = sizer ? sizer(B, M, K, N, wdt) : 0;
  if (ws) results.push_back(Shape::Array("s8", {(int64_t)ws}));
  // rows of K per scale: 0 = one scale per output channel ([N] or [B,N]); grouped scales are
  // [K/g,N], or [N,K/g] next to weights [N,K]
  const int64_t group_size = q.groups ? K / q.groups : 0;
  Instr* call = EmitCall(comp, ep.tail, "xla_amd.dequant_dot", ops, results,
                         CommonConfig(ep, dequant_ty, dot->shape.dtype) + ", scale_group_size = " +
                             std::to_string(group_size) + " : i64" +
                             (k_minor ? ", rhs_contracting_dim = 1 : i64" : "") +
                             (lhs_k_major ? ", lhs_contracting_dim = 0 : i64" : "") +
                             (weights_lhs ? ", result_transposed = true" : "") +
                             (ep.d_scale ? std::string(", d_scale_multiplies = ") + (ep.d_multiplies ? "true" : "false")
                                         : std::string()));
  Instr* value = results.size() > 1 ? EmitGte(comp, call, 0, ep.tail, ep.tail->name + ".out") : call;
  comp->ReplaceAllUses(ep.tail, value);
  log->rewrites.push_back(dot->name + " -> xla_amd.dequant_dot [" + ep.Name() + ", " + q.w->shape.dtype +
                          (q.zero ? " with zero points" : "") + (k_minor ? ", weights [N,K]" : "") +
                          (weights_lhs ? ", weights as lhs" : "") + (lhs_k_major ? ", activations [K,M]" : "") +
                          (ep.tail->shape.dtype == "f32" ? ", f32 result" : "") + (ep.d_scale ? ", f8 result" : "") + "]");
  return true;
}

// ragged-dot(lhs bf16 [M,K], dequantised weights [G,K,N] or [G,N,K], group_sizes [G]) with the ragged
// dimension on the rows of lhs (what gemm_rewriter.cc:781-863 hands to a grouped matmul): one call
// whose kernels read the group sizes on the device, for any number of rows.
bool RewriteRaggedDequantDot(Computation* comp, Instr* dot, RewriteLog* log) {
  QWeights q;
  std::string why;
  const bool k_minor = dot->DimsAttr("rhs_contracting_dims") == std::vector<int64_t>{2};  // experts stored [G,N,K]
  if (!MatchQWeights(dot->operands[1], k_minor, &q, &why)) {
    if (!why.empty()) log->refusals.push_back(dot->name + ": " + why);
    return false;
  }
  auto refuse = [&](const std::string& w) {
    log->refusals.push_back(dot->name + ": quantized weights found but not rewritten: " + w);
    return false;
  };
  Instr* lhs = dot->operands[0];
  Instr* sizes = dot->operands[2];
  Instr* inner;
  if (lhs->Is("convert") && ConvertFrom(lhs, "bf16", &inner) && lhs->shape.dtype == "f32") lhs = inner;
  if (lhs->shape.dtype != "bf16") return refuse("the activation must be bf16 (or its convert to f32)");
  if (lhs->shape.rank() != 2 || q.w->shape.rank() != 3 || dot->shape.rank() != 2)
    return refuse("a ragged dot is taken with lhs [M,K], weights [groups,K,N] or [groups,N,K] and a result [M,N]");
  if (dot->DimsAttr("lhs_contracting_dims") != std::vector<int64_t>{1} ||
      (dot->DimsAttr("rhs_contracting_dims") != std::vector<int64_t>{1} && !k_minor) ||
      dot->DimsAttr("lhs_ragged_dims") != std::vector<int64_t>{0} ||
      dot->DimsAttr("rhs_group_dims") != std::vector<int64_t>{0} || !dot->DimsAttr("lhs_batch_dims").empty())
    return refuse("a ragged dot is taken with the ragged dimension on the rows of lhs and the group dimension "
                  "leading the weights");
  const int64_t G = q.w->shape.dims[0], K = lhs->shape.dims[1], N = q.w->shape.dims[k_minor ? 1 : 2];  // any number of rows
  if (q.w->shape.dims[k_minor ? 2 : 1] != K) return refuse("contracting dimensions differ");
  if ((sizes->shape.dtype != "s32" && sizes->shape.dtype != "s64") || sizes->shape.dims != std::vector<int64_t>{G})
    return refuse("group sizes must be s32 or s64, one per group of weights");
  const bool four_bit = q.w->shape.dtype == "s4" || q.w->shape.dtype == "u4";
  if (four_bit && q.w->shape.dims[2] % 2 != 0) return refuse("s4 rows must hold an even number of values");
  if (q.zero && q.w->shape.dtype != "u4") return refuse("zero points are taken with u4 weights only");
  if (q.zero && q.zero->shape.dims != q.scale->shape.dims)
    return refuse("zero points must have the shape of the scales (one per scale)");
  // scales [G,N] (one per expert and channel) or [G,K/g,N] (one per g rows of K as well; [G,N,K/g]
  // next to experts stored [G,N,K])
  const bool grouped = q.scale->shape.rank() == 3;
  const int sn = k_minor ? 1 : 2, sg = k_minor ? 2 : 1;  // where N and the groups sit in rank-3 scales
  if (!(q.scale->shape.dims == std::vector<int64_t>{G, N}) &&
      !(grouped && q.scale->shape.dims[0] == G && q.scale->shape.dims[sn] == N && q.scale->shape.dims[sg] > 0 &&
        K % q.scale->shape.dims[sg] == 0))
    return refuse("a ragged dot takes scales [groups,N] or [groups,K/g,N]");
  const int64_t group_size = grouped ? K / q.scale->shape.dims[sg] : 0;
  if (q.type == "bf16" && q.scale->shape.dtype != "bf16") return refuse("bf16 multiply with non-bf16 scales");
  Epilogue ep;
  if (!MatchEpilogue(dot, &ep, &why)) return refuse(why);
  std::vector<Instr*> ops = {lhs, q.w, q.scale};
  if (q.zero) ops.push_back(q.zero);
  if (ep.bias) ops.push_back(ep.bias);
  ops.push_back(sizes);
  Instr* call = EmitCall(comp, ep.tail, "xla_amd.dequant_dot", ops, {Shape::Array("bf16", dot->shape.dims)},
                         CommonConfig(ep, q.type, dot->shape.dtype) + ", scale_group_size = " +
                             std::to_string(group_size) + " : i64" + (k_minor ? ", rhs_contracting_dim = 1 : i64" : ""));
  comp->ReplaceAllUses(ep.tail, call);
  log->rewrites.push_back(dot->name + " -> xla_amd.dequant_dot [" + ep.Name() + ", " + q.w->shape.dtype +
                          (q.zero ? " with zero points" : "") + ", ragged over " + std::to_string(G) + " groups" +
                          (k_minor ? ", weights [G,N,K]" : "") + "]");
  return true;
}

// ---------------------------------------------------------------- row-wise fp8 quantize
bool IsReduceOver(const Instr* r, const Module& m, const char* body_op, int64_t dim, Instr** src, Instr** init) {
  if (!r->Is("reduce") || r->operands.size() != 2 || r->DimsAttr("dimensions") != std::vector<int64_t>{dim}) return false;
  const std::string* to = r->Attr("to_apply");
  if (!to) return false;
  std::string name = *to;
  if (!name.empty() && name[0] == '%') name = name.substr(1);
  const Computation* c = m.FindComputation(name);
  if (!c || !c->root() || !c->root()->Is(body_op)) return false;
  *src = r->operands[0];
  *init = r->operands[1];
  return true;
}

bool RewriteQuantize(const Module& mod, Computation* comp, Instr* q, RewriteLog* log) {
  // q = convert(clamp(-448, yf / broadcast(s), 448)) -> f8e4m3fn [R,C]
  if (!q->Is("convert") || q->shape.dtype != "f8e4m3fn" || q->shape.rank() != 2) return false;
  Instr* cl = q->operands[0];
  if (!cl->Is("clamp") || cl->operands.size() != 3 || !IsConst(cl->operands[0], -448.0) || !IsConst(cl->operands[2], 448.0))
    return false;
  auto refuse = [&](const std::string& w) {
    log->refusals.push_back(q->name + ": clamp/convert to f8e4m3fn found but not rewritten: " + w);
    return false;
  };
  Instr *yf, *sb, *s;
  if (!Binary(cl->operands[1], "divide", &yf, &sb) || !BroadcastAlong(sb, {0}, &s))
    return refuse("the clamped value is not y / broadcast(scale[rows])");
  Instr *amax, *c448;
  if (!Binary(s, "divide", &amax, &c448) || !IsConst(c448, 448.0)) return refuse("scale is not amax / 448");
  Instr *absy, *init;
  if (!IsReduceOver(amax, mod, "maximum", 1, &absy, &init) || !absy->Is("abs") || absy->operands[0] != yf)
    return refuse("amax is not reduce-max(abs(y)) over the columns");
  double iv;
  if (!ConstScalar(init, &iv) || !(iv == 0.0 || iv == -INFINITY)) return refuse("reduce-max init must be 0 or -inf");
  Instr* y;
  if (!ConvertFrom(yf, "bf16", &y) || yf->shape.dtype != "f32") return refuse("y must be a bf16 value converted to f32");
  // users of yf: abs and the divide; of s: its broadcast (and possibly the module result)
  for (Instr* u : yf->users)
    if (u != absy && u != cl->operands[1]) return refuse("f32(y) has other users");

  Instr *x = y, *gamma = nullptr;
  double eps = 1e-6;
  bool rms = false;
  // y = convert((xf * broadcast(rinv)) * broadcast(f32(gamma))) -> bf16
  if (y->Is("convert") && y->operands[0]->shape.dtype == "f32" && y->operands[0]->Is("multiply")) {
    Instr *gsrc = nullptr, *t = nullptr;
    if (BinaryWith(y->operands[0], "multiply", [&](Instr* b) { return BroadcastAlong(b, {1}, &gsrc); }, &t)) {
      Instr *rinv = nullptr, *xf = nullptr, *g = nullptr, *xin = nullptr;
      if (ConvertFrom(gsrc, "bf16", &g) &&
          BinaryWith(t, "multiply", [&](Instr* b) { return BroadcastAlong(b, {0}, &rinv); }, &xf) &&
          ConvertFrom(xf, "bf16", &xin)) {
        // rinv = 1 / sqrt(sum(xf*xf)/C + eps), or the same value spelled rsqrt(...): the CPU backend
        // defines rsqrt as 1 / sqrt(x) wherever it does not use the x86 approximation instruction
        // (xla/codegen/intrinsic/rsqrt.cc:178-193) and refines that approximation towards the same
        // value (rsqrt.cc:195-224); the custom call computes the IEEE 1 / sqrt(x) for both spellings
        Instr *one, *rt;
        const bool as_divide = Binary(rinv, "divide", &one, &rt) && IsConst(one, 1.0) && rt->Is("sqrt");
        if (as_divide || rinv->Is("rsqrt")) {
          Instr* ms = nullptr;
          Instr* me = as_divide ? rt->operands[0] : rinv->operands[0];
          if (BinaryWith(me, "add", [&](Instr* b) { return ConstScalar(b, &eps); }, &ms)) {
            Instr *ssum = nullptr, *cnt = nullptr;
            double cv = 0;
            bool mean_ok = false;
            if (Binary(ms, "divide", &ssum, &cnt) && ConstScalar(cnt, &cv) && cv == (double)q->shape.dims[1]) mean_ok = true;
            Instr *sq, *zero;
            if (mean_ok && IsReduceOver(ssum, mod, "add", 1, &sq, &zero) && IsConst(zero, 0.0)) {
              Instr *a, *b;
              if (Binary(sq, "multiply", &a, &b) && a == xf && b == xf) {
                rms = true;
                x = xin;
                gamma = g;
              }
            }
          }
        }
      }
    }
    if (!rms) return refuse("y is computed from a multiply that is not the RMSNorm form x * (1/sqrt(mean(x^2)+eps)) * gamma (or rsqrt of the same)");
  }
  if (x->shape.dtype != "bf16") return refuse("input must be bf16");

  const int64_t R = q->shape.dims[0], C = q->shape.dims[1];
  std::vector<Instr*> ops = {x};
  if (rms) ops.push_back(gamma);
  char epsbuf[64];
  snprintf(epsbuf, sizeof(epsbuf), "%.9g", eps);
  std::string cfg = std::string("rmsnorm = ") + (rms ? "true" : "false") + ", eps = " + epsbuf + " : f32";
  // place the call where the scale is computed: it precedes every user of q and of s
  Instr* call = EmitCall(comp, s, "xla_amd.rowwise_quantize_fp8", ops,
                         {Shape::Array("f8e4m3fn", {R, C}), Shape::Array("f32", {R})}, cfg);
  Instr* s_new = EmitGte(comp, call, 1, s, s->name + ".scales");
  Instr* q_new = EmitGte(comp, call, 0, s, q->name + ".codes");
  // every user of the scale works on s_new from here on; the pattern's own broadcast too, which
  // may feed a dequantising multiply further down besides the divide that dies with q
  for (auto& i : comp->instrs)
    for (Instr*& op : i->operands)
      if (op == s) op = s_new;
  if (s->is_root) { s->is_root = false; s_new->is_root = true; }
  comp->ReplaceAllUses(q, q_new);
  log->rewrites.push_back(q->name + " -> xla_amd.rowwise_quantize_fp8 [" + (rms ? "rmsnorm" : "plain") + "]");
  return true;
}

}  // namespace

int RunQuantFusionRewriter(Module* mod, const RewriteOptions& opt, RewriteLog* log) {
  int changed = 0;
  for (auto& comp : mod->computations) {
    bool again = true;
    while (again) {
      again = false;
      // what nothing used before this sweep stays: only what a rewrite orphans is removed
      const std::set<const Instr*> unused_before = comp->Unused();
      for (auto& up : comp->instrs) {
        Instr* i = up.get();
        bool did = false;
        if (i->Is("dot") && i->operands.size() == 2) {
          did = RewriteF8Dot(*mod, comp.get(), i, opt, log) || RewriteDequantDot(*mod, comp.get(), i, opt, log);
        } else if (i->Is("ragged-dot") && i->operands.size() == 3) {
          did = RewriteRaggedDequantDot(comp.get(), i, log);
        } else if (i->Is("custom-call")) {
          did = RewriteBlockScaledDot(comp.get(), i, opt, log);
        } else if (i->Is("convert") && i->shape.dtype == "f8e4m3fn") {
          did = RewriteQuantize(*mod, comp.get(), i, log);
        }
        if (did) {
          ++changed;
          comp->RemoveDead(unused_before);
          // a redirected user (of an amax, of the scales) may sit above the new call
          comp->SortDefBeforeUse();
          again = true;
          break;  // the instruction list changed under the loop
        }
      }
    }
  }
  // refusals are re-recorded on every sweep; keep each once
  std::sort(log->refusals.begin(), log->refusals.end());
  log->refusals.erase(std::unique(log->refusals.begin(), log->refusals.end()), log->refusals.end());
  return changed;
}

}  // namespace hlo
}  // namespace xla_amd
