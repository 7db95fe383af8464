/* In-tree form of the quantized-inference rewrite pass (see quant_fusion_rewriter.h).
 *
 * NOT BUILT IN THIS REPOSITORY.  It is the offline matcher
 * (xla_amd/csrc/host/quant_fusion_rewriter.cc) restated on HloInstruction: the same helpers under
 * the same names, the same order of checks, the same refusal reasons word for word (a test compares
 * them).  Where the reference has a matcher for the same thing it is named:
 *   f8 operands and scales      gemm_rewriter.cc:190-336, 1235-1591
 *   bias / relu / gelu / silu   gemm_rewriter.cc:888-1007, 1987-2304 (GELU constants :472-503)
 *   s4 / s8 weights into a dot  gemm_fusion.cc:1572-1702
 *   block-scaled dot            block_scaling_rewriter.h:48-69
 */
#include "xla/backends/gpu/transforms/quant_fusion_rewriter.h"

#include <cmath>
#include <cstdint>
#include <functional>
#include <optional>
#include <string>
#include <utility>
#include <vector>

#include "absl/container/flat_hash_set.h"
#include "absl/log/log.h"
#include "absl/strings/str_cat.h"
#include "absl/strings/str_format.h"
#include "xla/hlo/ir/hlo_casting_utils.h"
#include "xla/hlo/ir/hlo_computation.h"
#include "xla/hlo/ir/hlo_instruction.h"
#include "xla/hlo/ir/hlo_instructions.h"
#include "xla/hlo/ir/hlo_opcode.h"
#include "xla/literal_util.h"
#include "xla/service/pattern_matcher.h"
#include "xla/shape_util.h"
#include "xla/xla_data.pb.h"

extern "C" {
// libxla_amd_quant.so (include/xla_amd_quant.h)
size_t xla_amd_dequant_dot_workspace_bytes(int64_t batch, int64_t M, int64_t K, int64_t N, int32_t weight_dtype);
size_t xla_amd_dequant_dot_workspace_bytes_nk(int64_t batch, int64_t M, int64_t K, int64_t N, int32_t weight_dtype);
size_t xla_amd_fp8_scaled_dot_workspace_bytes_typed(int64_t M, int64_t K, int64_t N, int32_t rhs_contracting_dim,
                                                    int32_t dequant_type);
}

namespace xla {
namespace gpu {
namespace {

namespace m = ::xla::match;
using Instr = HloInstruction;

bool IsFloatTy(PrimitiveType t) { return t == F32 || t == BF16; }
PrimitiveType Ty(const Instr* i) { return i->shape().element_type(); }
int64_t Rank(const Instr* i) { return i->shape().dimensions().size(); }
std::vector<int64_t> Dims(const Instr* i) {
  return std::vector<int64_t>(i->shape().dimensions().begin(), i->shape().dimensions().end());
}
std::string TyName(PrimitiveType t) { return primitive_util::LowercasePrimitiveTypeName(t); }
std::string I32(int v) { return absl::StrCat(v, " : i32"); }

// Scalar constant value, looking through broadcast and convert.
bool ConstScalar(const Instr* i, double* v) {
  while (i->opcode() == HloOpcode::kBroadcast || i->opcode() == HloOpcode::kConvert ||
         i->opcode() == HloOpcode::kReshape || i->opcode() == HloOpcode::kBitcast)
    i = i->operand(0);
  if (i->opcode() != HloOpcode::kConstant || ShapeUtil::ElementsIn(i->shape()) != 1) return false;
  std::optional<double> d = i->literal().GetAsDouble(std::vector<int64_t>(Rank(i), 0));
  if (!d.has_value()) return false;
  *v = *d;
  return true;
}
bool IsConst(const Instr* i, double want) {
  double v;
  return ConstScalar(i, &v) && v == want;
}
// BcastConstScalarNear (gemm_rewriter.cc:472-503): 128 epsilons of the constant's own type
bool IsConstNear(const Instr* i, double want) {
  double v;
  if (!ConstScalar(i, &v)) return false;
  const Instr* c = i;
  while (c->opcode() != HloOpcode::kConstant) c = c->operand(0);
  double eps;
  switch (Ty(c)) {
    case F16: eps = 0x1p-10; break;
    case BF16: eps = 0x1p-7; break;
    case F32: eps = 0x1p-23; break;
    case F64: eps = 0x1p-52; break;
    default: return false;
  }
  return std::fabs(v - want) < std::fabs(v + want) * 128 * eps;
}

// broadcast of a rank-0 value (dimensions={})
bool ScalarBroadcast(Instr* i, Instr** scalar) {
  return Match(i, m::Broadcast(m::Op(scalar).WithShape(m::Shape().IsScalar())));
}
// broadcast(src), dimensions=dims
bool BroadcastAlong(Instr* i, const std::vector<int64_t>& dims, Instr** src) {
  if (i->opcode() != HloOpcode::kBroadcast) return false;
  if (std::vector<int64_t>(i->dimensions().begin(), i->dimensions().end()) != dims) return false;
  *src = i->mutable_operand(0);
  return true;
}
bool Binary(Instr* i, HloOpcode op, Instr** a, Instr** b) {
  if (i->opcode() != op || i->operand_count() != 2) return false;
  *a = i->mutable_operand(0);
  *b = i->mutable_operand(1);
  return true;
}
// Commutative binary op with one side satisfying `pred`; *other receives the other side.
bool BinaryWith(Instr* i, HloOpcode op, const std::function<bool(Instr*)>& pred, Instr** other) {
  Instr *a, *b;
  if (!Binary(i, op, &a, &b)) return false;
  if (pred(b)) { *other = a; return true; }
  if (pred(a)) { *other = b; return true; }
  return false;
}
// convert whose operand has element type `from`
bool ConvertFrom(Instr* i, PrimitiveType from, Instr** src) {
  return Match(i, m::Convert(m::Op(src).WithElementType(from)));
}
Instr* SoleUser(Instr* i) { return i->user_count() == 1 ? i->users()[0] : nullptr; }

struct Epilogue {
  Instr* tail = nullptr;     // last instruction absorbed (its value is what the custom call returns)
  Instr* bias = nullptr;     // [N] operand, bf16 or f32 (null if none)
  std::string act;           // "", RELU, GELU, SILU
  PrimitiveType ops_type = F32;  // element type of the bias add / activation ops
  Instr* d_scale = nullptr;  // f8 result: the scalar the value is divided (or multiplied) by
  bool d_multiplies = false;
  Instr* amax = nullptr;     // f8 result: reduce-maximum of abs(value) over everything
  std::string Name() const {
    if (bias) return act.empty() ? "BIAS" : "BIAS_" + act;
    return act.empty() ? "DEFAULT" : act;
  }
};

// tanh-GELU rooted at `out` = x * cdf (gemm_rewriter.cc:923-973):
//   cdf = 0.5 * (1 + tanh(c1 * (x + c0 * (x*x*x))))
bool MatchGelu(Instr* out, Instr* x) {
  Instr *c1 = nullptr, *c0 = nullptr;
  auto cube = m::MultiplyAnyOrder(m::Op().Is(x), m::Multiply(m::Op().Is(x), m::Op().Is(x)));
  auto inner = m::AddAnyOrder(m::Op().Is(x), m::MultiplyAnyOrder(cube, m::Op(&c0)));
  auto cdf = m::MultiplyAnyOrder(
      m::AddAnyOrder(m::Tanh(m::MultiplyAnyOrder(inner, m::Op(&c1))), m::Op().IsEffectiveConstantScalar(1.0)),
      m::Op().IsEffectiveConstantScalar(0.5));
  return Match(out, m::MultiplyAnyOrder(m::Op().Is(x), cdf)) && IsConstNear(c1, 0.7978845608028654) &&
         IsConstNear(c0, 0.044715);
}
// x * (1 / (1 + exp(-x)))  (gemm_rewriter.cc:995-1002) or x * logistic(x)
bool MatchSilu(Instr* out, Instr* x) {
  auto sigmoid = m::Divide(m::Op().IsEffectiveConstantScalar(1.0),
                           m::AddAnyOrder(m::Exp(m::Negate(m::Op().Is(x))), m::Op().IsEffectiveConstantScalar(1.0)));
  return Match(out, m::MultiplyAnyOrder(m::Op().Is(x), sigmoid)) ||
         Match(out, m::MultiplyAnyOrder(m::Op().Is(x), m::Logistic(m::Op().Is(x))));
}

// Walks forward from the dot: optional convert, optional + broadcast(bias) along the minor
// dimension, optional activation, optional final convert to bf16 -- or, for f32-typed f8 dots, the
// f8 result tail convert(clamp(-448, v / z | v * z, 448)) with its optional amax.
// allow_f32_result: the kernels behind the call can write the f32 value itself (the dequantize-dot);
// otherwise the value leaving the pattern must be bf16.
bool MatchEpilogue(Instr* dot, Epilogue* ep, std::string* why, bool allow_f8_result, bool allow_f32_result = false,
                   bool allow_amax = true) {
  Instr* cur = dot;
  const int64_t rank = Rank(dot);
  ep->ops_type = Ty(dot);
  auto step_convert = [&]() {
    Instr* u = SoleUser(cur);
    if (u && u->opcode() == HloOpcode::kConvert && IsFloatTy(Ty(u)) && Ty(u) != Ty(cur)) {
      cur = u;
      return true;
    }
    return false;
  };
  Instr* after_dot = cur;
  if (step_convert()) ep->ops_type = Ty(cur);
  if (Instr* u = SoleUser(cur)) {  // bias: add(cur, broadcast(bias[N]), dimensions={rank-1})
    Instr *bsrc = nullptr, *bb = nullptr;
    if (BinaryWith(u, HloOpcode::kAdd, [&](Instr* s) { return s != cur && BroadcastAlong(s, {rank - 1}, &bsrc); }, &bb) &&
        bb == cur && Rank(bsrc) == 1) {
      Instr* raw = bsrc;
      Instr* inner;
      if (ConvertFrom(bsrc, BF16, &inner) && Ty(bsrc) == F32) raw = inner;
      if (IsFloatTy(Ty(raw))) {
        ep->bias = raw;
        cur = u;
      }
    }
  }
  {  // activation on cur: the unique maximum / multiply that closes over cur's users
    std::vector<Instr*> frontier(cur->users().begin(), cur->users().end());
    absl::flat_hash_set<Instr*> seen;
    Instr* found = nullptr;
    std::string act;
    while (!frontier.empty() && !found) {
      Instr* c = frontier.back();
      frontier.pop_back();
      if (!seen.insert(c).second) continue;
      Instr* other;
      if (BinaryWith(c, HloOpcode::kMaximum, [](Instr* s) { return IsConst(s, 0.0); }, &other) && other == cur) {
        found = c;
        act = "RELU";
      } else if (c->opcode() == HloOpcode::kMultiply && MatchGelu(c, cur)) {
        found = c;
        act = "GELU";
      } else if (c->opcode() == HloOpcode::kMultiply && MatchSilu(c, cur)) {
        found = c;
        act = "SILU";
      } else if (seen.size() < 24) {
        for (Instr* u : c->users()) frontier.push_back(u);
      }
    }
    if (found) {  // every value between cur and found must stay inside the pattern
      absl::flat_hash_set<Instr*> inside;
      std::function<void(Instr*)> collect = [&](Instr* n) {
        if (n == cur || !inside.insert(n).second) return;
        for (Instr* op : n->operands())
          if (op->opcode() != HloOpcode::kConstant && op->opcode() != HloOpcode::kBroadcast) collect(op);
      };
      collect(found);
      bool closed = true;
      for (Instr* n : inside)
        if (n != found)
          for (Instr* u : n->users()) closed &= inside.contains(u);
      for (Instr* u : cur->users()) closed &= inside.contains(u);
      if (closed) {
        ep->act = act;
        cur = found;
      }
    }
  }
  if (cur != after_dot && cur != dot) ep->ops_type = Ty(cur);
  if (!ep->bias && ep->act.empty()) ep->ops_type = Ty(dot);  // nothing between dot and result
  // f8 result (gemm_rewriter_fp8_test.cc:1665-1690, :1730-1748), amax (:2559-2600)
  if (allow_f8_result && Ty(cur) == F32 && Ty(dot) == F32 && ep->ops_type == F32) {
    Instr* sc = SoleUser(cur);
    Instr* amax = nullptr;
    if (!sc && allow_amax && cur->user_count() == 2) {
      for (int which = 0; which < 2 && !amax; ++which) {
        Instr* ab = cur->users()[which];
        Instr* rd = ab->opcode() == HloOpcode::kAbs ? SoleUser(ab) : nullptr;
        if (!rd || rd->opcode() != HloOpcode::kReduce || rd->operand_count() != 2 || rd->operand(0) != ab) continue;
        std::vector<int64_t> all_dims;
        for (int64_t i = 0; i < rank; ++i) all_dims.push_back(i);
        double init;
        if (std::vector<int64_t>(rd->dimensions().begin(), rd->dimensions().end()) != all_dims ||
            rd->operand(1)->opcode() != HloOpcode::kConstant || !ConstScalar(rd->operand(1), &init) ||
            init != -INFINITY)
          continue;
        if (rd->to_apply()->root_instruction()->opcode() != HloOpcode::kMaximum) continue;
        amax = rd;
        sc = cur->users()[1 - which];
      }
    }
    Instr *val = nullptr, *z = nullptr, *bz = nullptr;
    bool mul = false, ok = false;
    if (sc && Binary(sc, HloOpcode::kDivide, &val, &bz) && val == cur && ScalarBroadcast(bz, &z)) ok = true;
    else if (sc && BinaryWith(sc, HloOpcode::kMultiply, [&](Instr* b) { return ScalarBroadcast(b, &z); }, &val) &&
             val == cur)
      ok = mul = true;
    if (ok && Ty(z) == F32) {
      Instr* cl = SoleUser(sc);
      if (cl && cl->opcode() == HloOpcode::kClamp && cl->operand(1) == sc && IsConst(cl->operand(0), -448.0) &&
          IsConst(cl->operand(2), 448.0)) {
        Instr* cv = SoleUser(cl);
        if (cv && cv->opcode() == HloOpcode::kConvert && Ty(cv) == F8E4M3FN) {
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
  if (Ty(cur) != BF16 && !(allow_f32_result && Ty(cur) == F32)) {
    *why = "the value leaving the dot pattern is " + TyName(Ty(cur)) + ", the kernels produce bf16";
    return false;
  }
  ep->tail = cur;
  return true;
}

std::string CommonConfig(const Epilogue& ep, PrimitiveType dequant_ty, PrimitiveType dot_ty) {
  return "epilogue = \"" + ep.Name() + "\", dequant_type = " + I32(dequant_ty) + ", dot_type = " + I32(dot_ty) +
         ", epilogue_type = " + I32(ep.ops_type);
}

// `(result..., scratch) custom-call(...)`, api_version TYPED_FFI, attributes as an MLIR dictionary
Instr* EmitCall(HloComputation* comp, absl::string_view target, std::vector<Instr*> operands,
                std::vector<Shape> results, const std::string& config) {
  Shape shape = results.size() == 1 ? results[0] : ShapeUtil::MakeTupleShape(results);
  return comp->AddInstruction(HloInstruction::CreateCustomCall(shape, operands, target, "{" + config + "}",
                                                               CustomCallApiVersion::API_VERSION_TYPED_FFI));
}
Instr* EmitGte(HloComputation* comp, Instr* call, int index) {
  return comp->AddInstruction(HloInstruction::CreateGetTupleElement(call->shape().tuple_shapes(index), call, index));
}
Instr* AsF32Scalar(HloComputation* comp, Instr* s) {
  if (Ty(s) == F32) return s;
  return comp->AddInstruction(HloInstruction::CreateConvert(ShapeUtil::MakeShape(F32, {}), s));
}

// ---------------------------------------------------------------- f8 scaled dot
struct F8Operand {
  Instr* value = nullptr;   // the f8e4m3fn tensor
  Instr* scale = nullptr;   // scalar or vector, null = 1
  bool divide = false;
  int64_t scale_dim = -1;   // the operand dimension a rank-1 scale runs along; -1 for a scalar
  PrimitiveType type = F32; // element type of the convert / multiply
};

bool ScaleBroadcast(Instr* i, Instr** scale, int64_t* dim) {
  if (ScalarBroadcast(i, scale)) {
    *dim = -1;
    return true;
  }
  if (i->opcode() != HloOpcode::kBroadcast || Rank(i) != 2 || Rank(i->operand(0)) != 1) return false;
  if (i->dimensions().size() != 1 || i->dimensions(0) < 0 || i->dimensions(0) > 1) return false;
  *scale = i->mutable_operand(0);
  *dim = i->dimensions(0);
  return true;
}

bool MatchF8Operand(Instr* op, F8Operand* out) {
  Instr* src;
  if (ConvertFrom(op, F8E4M3FN, &src)) {
    *out = {src, nullptr, false, -1, Ty(op)};
    return IsFloatTy(Ty(op));
  }
  Instr *cv = nullptr, *sc = nullptr;
  if (op->opcode() == HloOpcode::kMultiply) {
    if (!BinaryWith(op, HloOpcode::kMultiply, [&](Instr* s) { return ScaleBroadcast(s, &sc, &out->scale_dim); }, &cv))
      return false;
  } else if (op->opcode() == HloOpcode::kDivide) {
    Instr* b;
    if (!Binary(op, HloOpcode::kDivide, &cv, &b) || !ScaleBroadcast(b, &sc, &out->scale_dim)) return false;
    out->divide = true;
  } else {
    return false;
  }
  if (!ConvertFrom(cv, F8E4M3FN, &src) || Ty(cv) != Ty(op) || !IsFloatTy(Ty(op))) return false;
  if (Ty(sc) != Ty(op) && !(sc->opcode() == HloOpcode::kConvert || IsFloatTy(Ty(sc)))) return false;
  out->value = src;
  out->scale = sc;
  out->type = Ty(op);
  return true;
}

using Refuse = std::function<bool(const std::string&)>;

bool RewriteF8Dot(HloComputation* comp, Instr* dot, const std::function<void(std::string)>& log) {
  F8Operand a, b;
  if (!MatchF8Operand(dot->mutable_operand(0), &a) || !MatchF8Operand(dot->mutable_operand(1), &b)) return false;
  auto refuse = [&](const std::string& why) {
    log(absl::StrCat(dot->name(), ": f8 operands found but not rewritten: ", why));
    return false;
  };
  if (a.type != b.type) return refuse("operands are dequantised in different types");
  const int64_t rank = Rank(dot);
  if ((rank != 2 && rank != 3) || Rank(a.value) != rank || Rank(b.value) != rank)
    return refuse("only rank-2 dots and rank-3 dots with one batch dimension are supported");
  const int64_t lead = rank - 2;
  const DotDimensionNumbers& dn = dot->dot_dimension_numbers();
  auto is_lead = [&](const auto& dims) { return lead ? dims.size() == 1 && dims[0] == 0 : dims.empty(); };
  if (!is_lead(dn.lhs_batch_dimensions()) || !is_lead(dn.rhs_batch_dimensions()))
    return refuse(lead ? "the batch dimension must be the leading one of both operands"
                       : "batch dimensions are not supported on rank-2 operands");
  if (dn.lhs_contracting_dimensions_size() != 1 || dn.rhs_contracting_dimensions_size() != 1 ||
      dn.lhs_contracting_dimensions(0) != rank - 1 || dn.rhs_contracting_dimensions(0) < lead)
    return refuse("lhs must contract its minor dimension");
  const int64_t rc = dn.rhs_contracting_dimensions(0) - lead;  // 0 = rhs [K,N], 1 = rhs [N,K]
  if (lead && (a.scale_dim >= 0 || b.scale_dim >= 0)) return refuse("a batched dot takes per-tensor scales");
  if (!IsFloatTy(Ty(dot))) return refuse("dot result type " + TyName(Ty(dot)));
  Epilogue ep;
  std::string why;
  if (!MatchEpilogue(dot, &ep, &why, /*allow_f8_result=*/true)) return refuse(why);

  const int64_t M = a.value->shape().dimensions(lead), K = a.value->shape().dimensions(lead + 1);
  const int64_t N = b.value->shape().dimensions(lead + 1 - rc);
  std::vector<int64_t> out_dims = {M, N};
  if (lead) out_dims.insert(out_dims.begin(), a.value->shape().dimensions(0));
  if (a.scale_dim == 1) return refuse("the lhs scales vary along the contracting dimension");
  if (b.scale_dim == rc) return refuse("the rhs scales vary along the contracting dimension");
  if ((a.scale_dim >= 0 && a.divide) || (b.scale_dim >= 0 && b.divide))
    return refuse("a division by a vector of scales is not taken");
  auto scale_of = [&](const F8Operand& o) -> Instr* {
    Instr* s = o.scale;
    if (!s) return comp->AddInstruction(HloInstruction::CreateConstant(LiteralUtil::CreateR0<float>(1.0f)));
    if (o.scale_dim >= 0) {
      if (Ty(s) == F32) return s;
      return comp->AddInstruction(HloInstruction::CreateConvert(ShapeUtil::ChangeElementType(s->shape(), F32), s));
    }
    s = AsF32Scalar(comp, s);
    if (o.divide) {
      Instr* one = comp->AddInstruction(HloInstruction::CreateConstant(LiteralUtil::CreateR0<float>(1.0f)));
      s = comp->AddInstruction(HloInstruction::CreateBinary(ShapeUtil::MakeShape(F32, {}), HloOpcode::kDivide, one, s));
    }
    return s;
  };
  std::vector<Instr*> ops = {a.value, b.value, scale_of(a), scale_of(b)};
  if (ep.bias) ops.push_back(ep.bias);
  if (ep.d_scale) ops.push_back(ep.d_scale);
  std::vector<Shape> results = {ShapeUtil::MakeShape(ep.d_scale ? F8E4M3FN : BF16, out_dims)};
  if (ep.amax) results.push_back(ShapeUtil::MakeShape(F32, {}));
  if (size_t ws = xla_amd_fp8_scaled_dot_workspace_bytes_typed(M, K, N, (int32_t)rc, (int32_t)a.type))
    results.push_back(ShapeUtil::MakeShape(S8, {(int64_t)ws}));
  std::string cfg = CommonConfig(ep, a.type, Ty(dot)) + absl::StrCat(", rhs_contracting_dim = ", rc, " : i64");
  if (ep.d_scale) absl::StrAppend(&cfg, ", d_scale_multiplies = ", ep.d_multiplies ? "true" : "false");
  Instr* call = EmitCall(comp, "xla_amd.fp8_scaled_dot", ops, results, cfg);
  Instr* value = results.size() > 1 ? EmitGte(comp, call, 0) : call;
  CHECK_OK(ep.tail->ReplaceAllUsesWith(value));
  if (ep.amax) CHECK_OK(ep.amax->ReplaceAllUsesWith(EmitGte(comp, call, 1)));
  VLOG(1) << dot->name() << " -> xla_amd.fp8_scaled_dot [" << ep.Name() << (ep.d_scale ? ", f8 result" : "")
          << (ep.amax ? ", amax" : "") << "]";
  return true;
}

// ---------------------------------------------------------------- block-scaled (MXFP8) dot
bool RewriteBlockScaledDot(HloComputation* comp, Instr* cc, const std::function<void(std::string)>& log) {
  if (cc->opcode() != HloOpcode::kCustomCall || cc->custom_call_target() != "__op$block_scaled_dot") return false;
  auto refuse = [&](const std::string& why) {
    log(absl::StrCat(cc->name(), ": block-scaled dot found but not rewritten: ", why));
    return false;
  };
  if (cc->operand_count() != 4) return refuse("expected lhs, rhs and a scale for each");
  Instr *a = cc->mutable_operand(0), *b = cc->mutable_operand(1), *sa = cc->mutable_operand(2),
        *sb = cc->mutable_operand(3);
  if (Ty(a) != F8E4M3FN || Ty(b) != F8E4M3FN || Ty(sa) != F8E8M0FNU || Ty(sb) != F8E8M0FNU)
    return refuse("operands must be f8e4m3fn with f8e8m0fnu scales");
  // one leading batch dimension, on all of them or on none (block_scaling_rewriter.h:53: the batch
  // dimension, if present, is the major one)
  const int64_t rank = Rank(a);
  if ((rank != 2 && rank != 3) || Rank(b) != rank || Rank(sa) != rank || Rank(sb) != rank || cc->shape().IsTuple() ||
      Rank(cc) != rank)
    return refuse("operands, scales and result must all be rank 2, or rank 3 with the batch dimension first");
  const int64_t lead = rank - 2;
  const int64_t M = a->shape().dimensions(lead), K = a->shape().dimensions(lead + 1), N = b->shape().dimensions(lead);
  std::vector<int64_t> sa_dims = {M, K / 32}, sb_dims = {N, K / 32}, out_dims = {M, N};
  if (lead) {
    const int64_t B = a->shape().dimensions(0);
    if (b->shape().dimensions(0) != B) return refuse("batch dimensions differ");
    for (auto* d : {&sa_dims, &sb_dims, &out_dims}) d->insert(d->begin(), B);
  }
  if (b->shape().dimensions(lead + 1) != K || K % 32 != 0 || Dims(sa) != sa_dims || Dims(sb) != sb_dims)
    return refuse("scales must be one per 32 elements of the contracting (minor) dimension");
  if (!cc->raw_backend_config_string().empty())
    return refuse("a backend_config (explicit block size, global scale) is not taken");
  if (!IsFloatTy(Ty(cc)) || Dims(cc) != out_dims)
    return refuse("the result is " + TyName(Ty(cc)) + ", the kernels produce bf16 [M,N] from a bf16 or f32 dot");
  // what follows the dot (bias, activation, the convert to bf16) goes into the call like behind an
  // ordinary dot; the value that leaves must be bf16
  Epilogue ep;
  std::string why;
  if (!MatchEpilogue(cc, &ep, &why, /*allow_f8_result=*/false)) return refuse(why);
  std::vector<Instr*> ops = {a, b, sa, sb};
  if (ep.bias) ops.push_back(ep.bias);
  std::string cfg = CommonConfig(ep, F32, Ty(cc)) + ", rhs_contracting_dim = 1 : i64";
  std::vector<Shape> results = {ShapeUtil::MakeShape(BF16, out_dims)};
  // scratch: the f32 sums of the K-slices of the kernels that take few rows of lhs, per batch
  size_t ws = xla_amd_fp8_scaled_dot_workspace_bytes_typed(M, K, N, 1, (int32_t)F32);
  if (lead) ws *= (size_t)a->shape().dimensions(0);
  if (ws) results.push_back(ShapeUtil::MakeShape(S8, {(int64_t)ws}));
  Instr* call = EmitCall(comp, "xla_amd.fp8_scaled_dot", ops, results, cfg);
  Instr* value = results.size() > 1 ? EmitGte(comp, call, 0) : call;
  CHECK_OK(ep.tail->ReplaceAllUsesWith(value));
  VLOG(1) << cc->name() << " -> xla_amd.fp8_scaled_dot [" << ep.Name() << ", block scales" << (lead ? ", batched" : "")
          << "]";
  return true;
}

// ---------------------------------------------------------------- weight-only dequantize dot
struct QWeights {
  Instr* w = nullptr;       // s8, s4 or u4 tensor [B,]K,N -- or [B,]N,K (K minor)
  Instr* scale = nullptr;   // [N] | [G,N] | [B,N] | [B,G,N] -- K minor: [N] | [N,G] | [B,N] | [B,N,G]; bf16 or f32
  PrimitiveType type = F32; // element type of the multiply
  Instr* zero = nullptr;    // u4 zero points, shaped like the scales: (w - zero) * scale
  int64_t groups = 0;       // scales along K, 0 = one per output channel
};

bool IsQuantTy(PrimitiveType t) { return t == S8 || t == S4 || t == U4; }
// convert(s4 -> s8) or convert(u4 -> u8): how 4-bit values are often widened before the float convert
bool IsByteWidening(const Instr* s) {
  if (s->opcode() != HloOpcode::kConvert) return false;
  const PrimitiveType from = Ty(s->operand(0));
  return (Ty(s) == S8 && from == S4) || (Ty(s) == U8 && from == U4);
}
// integer tensor behind convert(s4->s8)? -> convert(->float)
bool IntSource(Instr* cv, PrimitiveType float_ty, Instr** w) {
  if (cv->opcode() != HloOpcode::kConvert || Ty(cv) != float_ty) return false;
  Instr* s = cv->mutable_operand(0);
  if (IsByteWidening(s)) s = s->mutable_operand(0);
  if (!IsQuantTy(Ty(s))) return false;
  *w = s;
  return true;
}
// v = subtract(x, broadcast(convert(u4 zero points -> ty)) along bdims): peels the subtraction off
bool PeelZeroPoint(Instr* v, const std::vector<int64_t>& bdims, PrimitiveType ty, Instr** x, Instr** zero) {
  if (v->opcode() != HloOpcode::kSubtract || Ty(v) != ty) return false;
  Instr* zs = nullptr;
  if (!BroadcastAlong(v->mutable_operand(1), bdims, &zs)) return false;
  if (zs->opcode() != HloOpcode::kConvert || Ty(zs) != ty || Ty(zs->operand(0)) != U4) return false;
  *x = v->mutable_operand(0);
  *zero = zs->mutable_operand(0);
  return true;
}
Instr* LookThroughWidening(Instr* s, PrimitiveType to) {
  // convert(bf16 -> f32) of a scale is exact: hand the kernel the narrow original
  if (s->opcode() == HloOpcode::kConvert && to == F32 && Ty(s->operand(0)) == BF16) return s->mutable_operand(0);
  return s;
}

// k_minor: the weights are [B,]N,K (the dot contracts their minor dimension) instead of [B,]K,N.
bool MatchQWeights(Instr* op, bool k_minor, QWeights* out, std::string* why) {
  const PrimitiveType ty = Ty(op);
  if (!IsFloatTy(ty)) return false;
  const int64_t rank = Rank(op);
  // grouped: reshape([G,g,N] product) -> [K,N], or with a leading batch / expert dimension
  // reshape([B,G,g,N] product) -> [B,K,N]; K minor: reshape([B,]N,G,g product) -> [B,]N,K
  if (op->opcode() == HloOpcode::kReshape && (rank == 2 || rank == 3) && Rank(op->operand(0)) == rank + 1 &&
      op->operand(0)->opcode() == HloOpcode::kMultiply) {
    Instr* mul = op->mutable_operand(0);
    const int64_t lead = rank - 2;  // 0, or 1 with a batch dimension in front
    const std::vector<int64_t> dm = Dims(mul);
    const std::vector<int64_t> d3(dm.begin() + lead, dm.end());  // G, g, N -- or N, G, g
    if (k_minor) {
      if (d3[0] != op->shape().dimensions(lead) || d3[1] * d3[2] != op->shape().dimensions(lead + 1)) return false;
    } else if (d3[0] * d3[1] != op->shape().dimensions(lead) || d3[2] != op->shape().dimensions(lead + 1)) {
      return false;
    }
    if (lead && dm[0] != op->shape().dimensions(0)) return false;
    const std::vector<int64_t> gdims = k_minor ? (lead ? std::vector<int64_t>{0, 1, 2} : std::vector<int64_t>{0, 1})
                                               : (lead ? std::vector<int64_t>{0, 1, 3} : std::vector<int64_t>{0, 2});
    Instr *sc = nullptr, *cv = nullptr;
    if (!BinaryWith(mul, HloOpcode::kMultiply, [&](Instr* s) { return BroadcastAlong(s, gdims, &sc); }, &cv))
      return false;
    Instr* zero = nullptr;
    PeelZeroPoint(cv, gdims, ty, &cv, &zero);
    Instr* w = nullptr;  // the convert may sit before or after the reshape to [G,g,N]
    if (cv->opcode() == HloOpcode::kConvert && cv->operand(0)->opcode() == HloOpcode::kReshape) {
      Instr* src = cv->mutable_operand(0)->mutable_operand(0);
      if (IsByteWidening(src)) src = src->mutable_operand(0);
      if (IsQuantTy(Ty(src)) && Rank(src) == rank) w = src;
    } else if (cv->opcode() == HloOpcode::kReshape) {
      IntSource(cv->mutable_operand(0), ty, &w);
    }
    if (!w || Dims(w) != Dims(op)) {
      *why = "grouped dequantise: could not find the integer weights behind the reshape";
      return false;
    }
    sc = LookThroughWidening(sc, ty);
    if (Rank(sc) != rank || sc->shape().dimensions(lead) != d3[0] ||
        sc->shape().dimensions(lead + 1) != d3[k_minor ? 1 : 2])
      return false;
    if (lead && sc->shape().dimensions(0) != op->shape().dimensions(0)) return false;
    *out = {w, sc, ty, zero, d3[k_minor ? 1 : 0]};
    return true;
  }
  if (op->opcode() == HloOpcode::kConvert) {
    // convert(s4|s8|u4 -> float) straight into the dot: no scale at all (Int4WeightsOnTheRhs / OnTheLhs,
    // fusion_emitter_int4_device_test.cc:495-606); the caller supplies scales of one
    Instr* w;
    if (!IntSource(op, ty, &w) || Dims(w) != Dims(op)) return false;
    *out = {w, nullptr, ty, nullptr, 0};
    return true;
  }
  if (op->opcode() != HloOpcode::kMultiply) return false;
  Instr *sc = nullptr, *cv = nullptr;
  const std::vector<int64_t> bdims = k_minor ? (rank == 2 ? std::vector<int64_t>{0} : std::vector<int64_t>{0, 1})
                                             : (rank == 2 ? std::vector<int64_t>{1} : std::vector<int64_t>{0, 2});
  if (!BinaryWith(op, HloOpcode::kMultiply, [&](Instr* s) { return BroadcastAlong(s, bdims, &sc); }, &cv)) return false;
  Instr* zero = nullptr;
  PeelZeroPoint(cv, bdims, ty, &cv, &zero);
  Instr* w;
  if (!IntSource(cv, ty, &w) || Dims(w) != Dims(op)) return false;
  sc = LookThroughWidening(sc, ty);
  *out = {w, sc, ty, zero, 0};
  return true;
}

bool RewriteDequantDot(HloComputation* comp, Instr* dot, const std::function<void(std::string)>& log) {
  QWeights q;
  std::string why;
  const int64_t rank = Rank(dot);
  const DotDimensionNumbers& dn = dot->dot_dimension_numbers();
  auto contracts = [](const auto& dims, int64_t d) { return dims.size() == 1 && dims[0] == d; };
  // The dequantised weights are usually the rhs of the dot; they may be its lhs as well
  // (Int4WeightsOnTheLhs, fusion_emitter_int4_device_test.cc:495-523): the result is then [..,N,M].
  // Either operand may contract its minor or its major (non-batch) dimension: weights [..,K,N] or
  // [..,N,K] (:867-892), activations [..,M,K] or [..,K,M] (the shape table :609-645).
  bool weights_lhs = false;
  bool k_minor = contracts(dn.rhs_contracting_dimensions(), rank - 1);
  if (!MatchQWeights(dot->mutable_operand(1), k_minor, &q, &why)) {
    std::string why_lhs;
    const bool lhs_k_minor = contracts(dn.lhs_contracting_dimensions(), rank - 1);
    if (dot->operand_count() == 2 && MatchQWeights(dot->mutable_operand(0), lhs_k_minor, &q, &why_lhs)) {
      weights_lhs = true;
      k_minor = lhs_k_minor;
    } else {
      if (!why.empty()) log(absl::StrCat(dot->name(), ": ", why));
      else if (!why_lhs.empty()) log(absl::StrCat(dot->name(), ": ", why_lhs));
      return false;
    }
  }
  auto refuse = [&](const std::string& w) {
    log(absl::StrCat(dot->name(), ": quantized weights found but not rewritten: ", w));
    return false;
  };
  Instr* lhs = dot->mutable_operand(weights_lhs ? 1 : 0);  // the activations
  const auto& ac = weights_lhs ? dn.rhs_contracting_dimensions() : dn.lhs_contracting_dimensions();
  const auto& wc = weights_lhs ? dn.lhs_contracting_dimensions() : dn.rhs_contracting_dimensions();
  Instr* inner;
  if (ConvertFrom(lhs, BF16, &inner) && Ty(lhs) == F32) lhs = inner;
  if (Ty(lhs) != BF16) return refuse("the activation must be bf16 (or its convert to f32)");
  if (rank != 2 && rank != 3) return refuse("rank " + std::to_string(rank));
  auto is0 = [](const auto& d) { return d.size() == 1 && d[0] == 0; };
  if (rank == 3 && (!is0(dn.lhs_batch_dimensions()) || !is0(dn.rhs_batch_dimensions())))
    return refuse("the batch dimension must be dimension 0 of both operands");
  if (rank == 2 && dn.lhs_batch_dimensions_size() != 0) return refuse("unexpected batch dimensions");
  const bool lhs_k_major = contracts(ac, rank - 2);
  if ((!contracts(ac, rank - 1) && !lhs_k_major) || (!contracts(wc, rank - 2) && !k_minor))
    return refuse("needs lhs [..,M,K] contracting K and weights [..,K,N] or [..,N,K]; s4 with a "
                  "minor batch dimension is rejected as in gemm_fusion.cc:1572-1590");
  // (4-bit rows of an odd number of values are packed across row ends, xla/packing.cc:142-170: the
  // one-thread-per-output kernel reads them by flat index)
  if (q.zero && Ty(q.w) != U4) return refuse("zero points are taken with u4 weights only");
  if (q.zero && Dims(q.zero) != Dims(q.scale))
    return refuse("zero points must have the shape of the scales (one per scale)");
  if (q.scale && q.type == BF16 && Ty(q.scale) != BF16) return refuse("bf16 multiply with non-bf16 scales");
  Epilogue ep;
  if (!MatchEpilogue(dot, &ep, &why, /*allow_f8_result=*/true, /*allow_f32_result=*/true, /*allow_amax=*/false))
    return refuse(why);
  if (weights_lhs && (ep.bias || !ep.act.empty()))
    return refuse("with the weights as the lhs of the dot only the plain dot is taken (a bias would run along the other dimension)");

  const int64_t B = rank == 3 ? lhs->shape().dimensions(0) : 1;
  const int64_t M = lhs->shape().dimensions(rank - (lhs_k_major ? 1 : 2)), K = lhs->shape().dimensions(rank - (lhs_k_major ? 2 : 1));
  const int64_t N = q.w->shape().dimensions(rank - (k_minor ? 2 : 1));
  PrimitiveType dequant_ty = q.type;
  if (!q.scale) {
    // no multiply in the module: the integers themselves are the weights.  One scale per channel, all
    // ones, under an f32-typed multiply gives exactly those values (convert(int -> bf16) is exact).
    Instr* one = comp->AddInstruction(HloInstruction::CreateConstant(LiteralUtil::CreateR0<float>(1.0f)));
    q.scale = comp->AddInstruction(HloInstruction::CreateBroadcast(ShapeUtil::MakeShape(F32, {N}), one, {}));
    dequant_ty = F32;
  }
  std::vector<Instr*> ops = {lhs, q.w, q.scale};
  if (q.zero) ops.push_back(q.zero);
  if (ep.bias) ops.push_back(ep.bias);
  if (ep.d_scale) ops.push_back(ep.d_scale);  // an f8e4m3fn result: its scale goes last
  std::vector<Shape> results = {ShapeUtil::MakeShape(Ty(ep.tail), Dims(dot))};
  if (size_t ws = k_minor ? xla_amd_dequant_dot_workspace_bytes_nk(B, M, K, N, (int32_t)Ty(q.w))
                          : xla_amd_dequant_dot_workspace_bytes(B, M, K, N, (int32_t)Ty(q.w)))
    results.push_back(ShapeUtil::MakeShape(S8, {(int64_t)ws}));
  // rows of K per scale: 0 = one scale per output channel ([N] or [B,N]); grouped scales are
  // [K/g,N], or [N,K/g] next to weights [N,K]
  const int64_t group_size = q.groups ? K / q.groups : 0;
  Instr* call = EmitCall(comp, "xla_amd.dequant_dot", ops, results,
                         CommonConfig(ep, dequant_ty, Ty(dot)) + absl::StrCat(", scale_group_size = ", group_size, " : i64") +
                             (k_minor ? ", rhs_contracting_dim = 1 : i64" : "") +
                             (lhs_k_major ? ", lhs_contracting_dim = 0 : i64" : "") +
                             (weights_lhs ? ", result_transposed = true" : "") +
                             (ep.d_scale ? absl::StrCat(", d_scale_multiplies = ", ep.d_multiplies ? "true" : "false")
                                         : std::string()));
  Instr* value = results.size() > 1 ? EmitGte(comp, call, 0) : call;
  CHECK_OK(ep.tail->ReplaceAllUsesWith(value));
  VLOG(1) << dot->name() << " -> xla_amd.dequant_dot [" << ep.Name() << ", " << TyName(Ty(q.w))
          << (q.zero ? " with zero points" : "") << (k_minor ? ", weights [N,K]" : "")
          << (weights_lhs ? ", weights as lhs" : "") << (lhs_k_major ? ", activations [K,M]" : "")
          << (Ty(ep.tail) == F32 ? ", f32 result" : "") << (ep.d_scale ? ", f8 result" : "") << "]";
  return true;
}

// ragged-dot(lhs bf16 [M,K], dequantised weights [G,K,N], group_sizes [G]) with the ragged dimension
// on the rows of lhs (what gemm_rewriter.cc:781-863 hands to a grouped matmul): one call whose
// kernels read the group sizes on the device, for any number of rows.
bool RewriteRaggedDequantDot(HloComputation* comp, Instr* dot, const std::function<void(std::string)>& log) {
  QWeights q;
  std::string why;
  const RaggedDotDimensionNumbers& rd = Cast<HloRaggedDotInstruction>(dot)->ragged_dot_dimension_numbers();
  const DotDimensionNumbers& dn = rd.dot_dimension_numbers();
  auto is = [](const auto& d, int64_t v) { return d.size() == 1 && d[0] == v; };
  const bool k_minor = is(dn.rhs_contracting_dimensions(), 2);  // experts stored [G,N,K]
  if (!MatchQWeights(dot->mutable_operand(1), k_minor, &q, &why)) {
    if (!why.empty()) log(absl::StrCat(dot->name(), ": ", why));
    return false;
  }
  auto refuse = [&](const std::string& w) {
    log(absl::StrCat(dot->name(), ": quantized weights found but not rewritten: ", w));
    return false;
  };
  Instr* lhs = dot->mutable_operand(0);
  Instr* sizes = dot->mutable_operand(2);
  Instr* inner;
  if (ConvertFrom(lhs, BF16, &inner) && Ty(lhs) == F32) lhs = inner;
  if (Ty(lhs) != BF16) return refuse("the activation must be bf16 (or its convert to f32)");
  if (Rank(lhs) != 2 || Rank(q.w) != 3 || Rank(dot) != 2)
    return refuse("a ragged dot is taken with lhs [M,K], weights [groups,K,N] or [groups,N,K] and a result [M,N]");
  if (!is(dn.lhs_contracting_dimensions(), 1) || (!is(dn.rhs_contracting_dimensions(), 1) && !k_minor) ||
      !is(rd.lhs_ragged_dimensions(), 0) || !is(rd.rhs_group_dimensions(), 0) || dn.lhs_batch_dimensions_size() != 0)
    return refuse("a ragged dot is taken with the ragged dimension on the rows of lhs and the group dimension "
                  "leading the weights");
  const int64_t G = q.w->shape().dimensions(0), K = lhs->shape().dimensions(1),  // any number of rows
                N = q.w->shape().dimensions(k_minor ? 1 : 2);
  if (q.w->shape().dimensions(k_minor ? 2 : 1) != K) return refuse("contracting dimensions differ");
  if ((Ty(sizes) != S32 && Ty(sizes) != S64) || Dims(sizes) != std::vector<int64_t>{G})
    return refuse("group sizes must be s32 or s64, one per group of weights");
  const bool four_bit = Ty(q.w) == S4 || Ty(q.w) == U4;
  if (four_bit && q.w->shape().dimensions(2) % 2 != 0) return refuse("s4 rows must hold an even number of values");
  if (q.zero && Ty(q.w) != U4) return refuse("zero points are taken with u4 weights only");
  if (q.zero && Dims(q.zero) != Dims(q.scale))
    return refuse("zero points must have the shape of the scales (one per scale)");
  // scales [G,N] (one per expert and channel) or [G,K/g,N] (one per g rows of K as well; [G,N,K/g]
  // next to experts stored [G,N,K])
  const bool grouped = Rank(q.scale) == 3;
  const int sn = k_minor ? 1 : 2, sg = k_minor ? 2 : 1;  // where N and the groups sit in rank-3 scales
  if (!(Dims(q.scale) == std::vector<int64_t>{G, N}) &&
      !(grouped && q.scale->shape().dimensions(0) == G && q.scale->shape().dimensions(sn) == N &&
        q.scale->shape().dimensions(sg) > 0 && K % q.scale->shape().dimensions(sg) == 0))
    return refuse("a ragged dot takes scales [groups,N] or [groups,K/g,N]");
  const int64_t group_size = grouped ? K / q.scale->shape().dimensions(sg) : 0;
  if (q.type == BF16 && Ty(q.scale) != BF16) return refuse("bf16 multiply with non-bf16 scales");
  Epilogue ep;
  if (!MatchEpilogue(dot, &ep, &why, /*allow_f8_result=*/false)) return refuse(why);
  std::vector<Instr*> ops = {lhs, q.w, q.scale};
  if (q.zero) ops.push_back(q.zero);
  if (ep.bias) ops.push_back(ep.bias);
  ops.push_back(sizes);
  Instr* call = EmitCall(comp, "xla_amd.dequant_dot", ops, {ShapeUtil::MakeShape(BF16, Dims(dot))},
                         CommonConfig(ep, q.type, Ty(dot)) + absl::StrCat(", scale_group_size = ", group_size, " : i64") +
                             (k_minor ? ", rhs_contracting_dim = 1 : i64" : ""));
  CHECK_OK(ep.tail->ReplaceAllUsesWith(call));
  VLOG(1) << dot->name() << " -> xla_amd.dequant_dot [" << ep.Name() << ", " << TyName(Ty(q.w))
          << (q.zero ? " with zero points" : "") << ", ragged over " << G << " groups"
          << (k_minor ? ", weights [G,N,K]" : "") << "]";
  return true;
}

// ---------------------------------------------------------------- row-wise fp8 quantize
bool IsReduceOver(Instr* r, HloOpcode body_op, int64_t dim, Instr** src, Instr** init) {
  if (r->opcode() != HloOpcode::kReduce || r->operand_count() != 2 || r->dimensions().size() != 1 ||
      r->dimensions(0) != dim)
    return false;
  if (r->to_apply()->root_instruction()->opcode() != body_op) return false;
  *src = r->mutable_operand(0);
  *init = r->mutable_operand(1);
  return true;
}

bool RewriteQuantize(HloComputation* comp, Instr* q, const std::function<void(std::string)>& log) {
  // q = convert(clamp(-448, yf / broadcast(s), 448)) -> f8e4m3fn [R,C]
  if (q->opcode() != HloOpcode::kConvert || Ty(q) != F8E4M3FN || Rank(q) != 2) return false;
  Instr* cl = q->mutable_operand(0);
  if (cl->opcode() != HloOpcode::kClamp || !IsConst(cl->operand(0), -448.0) || !IsConst(cl->operand(2), 448.0))
    return false;
  auto refuse = [&](const std::string& why) {
    log(absl::StrCat(q->name(), ": clamp/convert to f8e4m3fn found but not rewritten: ", why));
    return false;
  };
  Instr *yf, *sb, *s;
  if (!Binary(cl->mutable_operand(1), HloOpcode::kDivide, &yf, &sb) || !BroadcastAlong(sb, {0}, &s))
    return refuse("the clamped value is not y / broadcast(scale[rows])");
  Instr *amax, *c448;
  if (!Binary(s, HloOpcode::kDivide, &amax, &c448) || !IsConst(c448, 448.0)) return refuse("scale is not amax / 448");
  Instr *absy, *init;
  if (!IsReduceOver(amax, HloOpcode::kMaximum, 1, &absy, &init) || absy->opcode() != HloOpcode::kAbs ||
      absy->operand(0) != yf)
    return refuse("amax is not reduce-max(abs(y)) over the columns");
  double iv;
  if (!ConstScalar(init, &iv) || !(iv == 0.0 || iv == -INFINITY)) return refuse("reduce-max init must be 0 or -inf");
  Instr* y;
  if (!ConvertFrom(yf, BF16, &y) || Ty(yf) != F32) return refuse("y must be a bf16 value converted to f32");
  for (Instr* u : yf->users())
    if (u != absy && u != cl->operand(1)) return refuse("f32(y) has other users");

  Instr *x = y, *gamma = nullptr;
  double eps = 1e-6;
  bool rms = false;
  // y = convert((xf * broadcast(rinv)) * broadcast(f32(gamma))) -> bf16
  if (y->opcode() == HloOpcode::kConvert && Ty(y->operand(0)) == F32 && y->operand(0)->opcode() == HloOpcode::kMultiply) {
    Instr *gsrc = nullptr, *t = nullptr;
    if (BinaryWith(y->mutable_operand(0), HloOpcode::kMultiply, [&](Instr* b) { return BroadcastAlong(b, {1}, &gsrc); }, &t)) {
      Instr *rinv = nullptr, *xf = nullptr, *g = nullptr, *xin = nullptr;
      if (ConvertFrom(gsrc, BF16, &g) &&
          BinaryWith(t, HloOpcode::kMultiply, [&](Instr* b) { return BroadcastAlong(b, {0}, &rinv); }, &xf) &&
          ConvertFrom(xf, BF16, &xin)) {
        // rinv = 1 / sqrt(sum(xf*xf)/C + eps), or rsqrt of the same (rsqrt.cc:178-193: 1 / sqrt(x))
        Instr *one, *rt;
        const bool as_divide = Binary(rinv, HloOpcode::kDivide, &one, &rt) && IsConst(one, 1.0) &&
                               rt->opcode() == HloOpcode::kSqrt;
        if (as_divide || rinv->opcode() == HloOpcode::kRsqrt) {
          Instr* ms = nullptr;
          Instr* me = as_divide ? rt->mutable_operand(0) : rinv->mutable_operand(0);
          if (BinaryWith(me, HloOpcode::kAdd, [&](Instr* b) { return ConstScalar(b, &eps); }, &ms)) {
            Instr *ssum = nullptr, *cnt = nullptr;
            double cv = 0;
            const bool mean_ok = Binary(ms, HloOpcode::kDivide, &ssum, &cnt) && ConstScalar(cnt, &cv) &&
                                 cv == (double)q->shape().dimensions(1);
            Instr *sq, *zero;
            if (mean_ok && IsReduceOver(ssum, HloOpcode::kAdd, 1, &sq, &zero) && IsConst(zero, 0.0)) {
              Instr *a, *b;
              if (Binary(sq, HloOpcode::kMultiply, &a, &b) && a == xf && b == xf) {
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
  if (Ty(x) != BF16) return refuse("input must be bf16");

  const int64_t R = q->shape().dimensions(0), C = q->shape().dimensions(1);
  std::vector<Instr*> ops = {x};
  if (rms) ops.push_back(gamma);
  std::string cfg = absl::StrCat("rmsnorm = ", rms ? "true" : "false", ", eps = ", absl::StrFormat("%.9g", eps), " : f32");
  Instr* call = EmitCall(comp, "xla_amd.rowwise_quantize_fp8", ops,
                         {ShapeUtil::MakeShape(F8E4M3FN, {R, C}), ShapeUtil::MakeShape(F32, {R})}, cfg);
  // every user of the scale (its broadcast may feed a dequantising multiply further down) and of q
  CHECK_OK(s->ReplaceAllUsesWith(EmitGte(comp, call, 1)));
  CHECK_OK(q->ReplaceAllUsesWith(EmitGte(comp, call, 0)));
  VLOG(1) << q->name() << " -> xla_amd.rowwise_quantize_fp8 [" << (rms ? "rmsnorm" : "plain") << "]";
  return true;
}

}  // namespace

absl::StatusOr<bool> QuantFusionRewriter::RunImpl(HloModule* module,
                                                  const absl::flat_hash_set<absl::string_view>& execution_threads) {
  bool changed = false;
  auto log = [&](std::string line) {
    VLOG(1) << "quant-fusion-rewriter refused: " << line;
    if (refusals_) refusals_->push_back(std::move(line));
  };
  for (HloComputation* comp : module->MakeNonfusionComputations(execution_threads)) {
    // post order: a quantizer feeding a dot is rewritten before the dot looks at its operands
    for (Instr* i : comp->MakeInstructionPostOrder()) {
      bool did = false;
      if (i->opcode() == HloOpcode::kDot && i->operand_count() == 2) {
        did = RewriteF8Dot(comp, i, log) || RewriteDequantDot(comp, i, log);
      } else if (i->opcode() == HloOpcode::kRaggedDot && i->operand_count() == 3) {
        did = RewriteRaggedDequantDot(comp, i, log);
      } else if (i->opcode() == HloOpcode::kCustomCall) {
        did = RewriteBlockScaledDot(comp, i, log);
      } else if (i->opcode() == HloOpcode::kConvert && Ty(i) == F8E4M3FN) {
        did = RewriteQuantize(comp, i, log);
      }
      changed |= did;
    }
  }
  // what the rewrites orphaned is left to the HloDCE that follows in the pipeline
  return changed;
}

}  // namespace gpu
}  // namespace xla
