// XLA typed-FFI handlers (include/xla_amd_quant.h, "Layer 1").
//
// Each handler does what the reference's generated `Handler::Call` does
// (xla/ffi/api/api.h:2296-2565), by hand and in the same order: check the
// call-frame struct size, answer the metadata query, check the stage, check
// operand counts, decode buffers and attributes, fetch the stream, launch.
// Messages keep the reference's wording so its tests' substring checks
// (xla/ffi/api/ffi_test.cc:869-932) apply unchanged.
#include <stdint.h>
#include <stdio.h>
#include <string.h>

#include <string>

#include "launch.h"
#include "xla_amd_quant.h"
#include "xla_ffi_record_abi.h"

namespace xla_amd {
namespace {

const char* StageName(XLA_FFI_ExecutionStage s) {
  switch (s) {
    case XLA_FFI_ExecutionStage_INSTANTIATE: return "instantiate";
    case XLA_FFI_ExecutionStage_PREPARE: return "prepare";
    case XLA_FFI_ExecutionStage_INITIALIZE: return "initialize";
    case XLA_FFI_ExecutionStage_EXECUTE: return "execute";
    case XLA_FFI_ExecutionStage_RECORD: return "record";
  }
  return "unknown";
}

const char* DTypeName(int d) {
  switch (d) {
    case XLA_FFI_DataType_PRED: return "PRED";
    case XLA_FFI_DataType_S4: return "S4";
    case XLA_FFI_DataType_S8: return "S8";
    case XLA_FFI_DataType_S16: return "S16";
    case XLA_FFI_DataType_S32: return "S32";
    case XLA_FFI_DataType_S64: return "S64";
    case XLA_FFI_DataType_U4: return "U4";
    case XLA_FFI_DataType_U8: return "U8";
    case XLA_FFI_DataType_U16: return "U16";
    case XLA_FFI_DataType_U32: return "U32";
    case XLA_FFI_DataType_U64: return "U64";
    case XLA_FFI_DataType_F16: return "F16";
    case XLA_FFI_DataType_F32: return "F32";
    case XLA_FFI_DataType_F64: return "F64";
    case XLA_FFI_DataType_BF16: return "BF16";
    case XLA_FFI_DataType_F8E5M2: return "F8E5M2";
    case XLA_FFI_DataType_F8E4M3FN: return "F8E4M3FN";
    case XLA_FFI_DataType_F8E4M3: return "F8E4M3";
    case XLA_FFI_DataType_F8E4M3FNUZ: return "F8E4M3FNUZ";
    case XLA_FFI_DataType_F8E5M2FNUZ: return "F8E5M2FNUZ";
    case XLA_FFI_DataType_F8E4M3B11FNUZ: return "F8E4M3B11FNUZ";
    case XLA_FFI_DataType_F8E8M0FNU: return "F8E8M0FNU";
    default: return "INVALID";
  }
}

const char* AttrTypeName(XLA_FFI_AttrType t) {
  switch (t) {
    case XLA_FFI_AttrType_ARRAY: return "array";
    case XLA_FFI_AttrType_DICTIONARY: return "dictionary";
    case XLA_FFI_AttrType_SCALAR: return "scalar";
    case XLA_FFI_AttrType_STRING: return "string";
  }
  return "unknown";
}

XLA_FFI_Error* MakeError(const XLA_FFI_Api* api, XLA_FFI_Error_Code code, const std::string& msg) {
  XLA_FFI_Error_Create_Args args;
  args.struct_size = XLA_FFI_Error_Create_Args_STRUCT_SIZE;
  args.extension_start = nullptr;
  args.message = msg.c_str();
  args.errc = code;
  return api->XLA_FFI_Error_Create(&args);
}

XLA_FFI_Error* InvalidArgument(const XLA_FFI_Api* api, const std::string& msg) {
  return MakeError(api, XLA_FFI_Error_Code_INVALID_ARGUMENT, msg);
}

// Collects per-operand diagnostics the way DiagnosticEngine does, and remembers which
// operand positions failed (args first, then rets, then attributes, then context).
struct Decoder {
  XLA_FFI_CallFrame* frame;
  std::string diagnostics;
  std::string bad;
  int position = 0;

  void Failed(const std::string& why) {
    if (!bad.empty()) bad += ", ";
    bad += std::to_string(position);
    diagnostics += why;
    diagnostics += "\n";
  }
  bool ok() const { return bad.empty(); }

  XLA_FFI_Error* Error() const {
    std::string msg = std::string("[") + StageName(frame->stage) +
                      "] Failed to decode all FFI handler operands (bad operands at: " + bad + ")";
    if (!diagnostics.empty()) msg += "\nDiagnostics:\n" + diagnostics;
    return InvalidArgument(frame->api, msg);
  }

  // dtype_mask: bit set of accepted XLA_FFI_DataType values (all < 64); rank < 0: any.
  XLA_FFI_Buffer* Buffer(void* raw, uint64_t dtype_mask, int rank_lo, int rank_hi, const char* what) {
    XLA_FFI_Buffer* b = static_cast<XLA_FFI_Buffer*>(raw);
    bool good = true;
    if (!((dtype_mask >> (int)b->dtype) & 1u) || (int)b->dtype >= 64) {
      std::string want;
      for (int d = 0; d < 64; ++d)
        if ((dtype_mask >> d) & 1u) want += (want.empty() ? "" : "|") + std::string(DTypeName(d));
      Failed(std::string("Wrong buffer dtype: expected ") + want + " but got " + DTypeName(b->dtype) +
             " (" + what + ")");
      good = false;
    } else if (b->rank < rank_lo || b->rank > rank_hi) {
      Failed(std::string("Wrong buffer rank: expected ") +
             (rank_lo == rank_hi ? std::to_string(rank_lo)
                                 : std::to_string(rank_lo) + ".." + std::to_string(rank_hi)) +
             " but got " + std::to_string(b->rank) + " (" + what + ")");
      good = false;
    }
    ++position;
    return good ? b : nullptr;
  }
  XLA_FFI_Buffer* Arg(int i, uint64_t mask, int lo, int hi, const char* what) {
    if (frame->args.types[i] != XLA_FFI_ArgType_BUFFER) {
      Failed(std::string("Wrong argument type: expected buffer (") + what + ")");
      ++position;
      return nullptr;
    }
    return Buffer(frame->args.args[i], mask, lo, hi, what);
  }
  XLA_FFI_Buffer* Ret(int i, uint64_t mask, int lo, int hi, const char* what) {
    if (frame->rets.types[i] != XLA_FFI_RetType_BUFFER) {
      Failed(std::string("Wrong result type: expected buffer (") + what + ")");
      ++position;
      return nullptr;
    }
    return Buffer(frame->rets.rets[i], mask, lo, hi, what);
  }

  // Attributes are a dictionary looked up by name (names arrive sorted, api.h:2076-2100);
  // every one has a default, so absence is not an error, a wrong type is.
  int Find(const char* name) const {
    const size_t len = strlen(name);
    for (int64_t i = 0; i < frame->attrs.size; ++i) {
      const XLA_FFI_ByteSpan* n = frame->attrs.names[i];
      if (n->len == len && memcmp(n->ptr, name, len) == 0) return (int)i;
    }
    return -1;
  }
  bool Scalar(const char* name, int dtype, void* out, size_t bytes) {
    ++position;
    const int i = Find(name);
    if (i < 0) return false;
    if (frame->attrs.types[i] != XLA_FFI_AttrType_SCALAR) {
      --position;
      Failed(std::string("Wrong attribute type: expected scalar but got ") +
             AttrTypeName(frame->attrs.types[i]) + " (" + name + ")");
      ++position;
      return false;
    }
    const XLA_FFI_Scalar* s = static_cast<const XLA_FFI_Scalar*>(frame->attrs.attrs[i]);
    if ((int)s->dtype != dtype) {
      --position;
      Failed(std::string("Wrong scalar data type: expected ") + DTypeName(dtype) + " but got " +
             DTypeName(s->dtype) + " (" + name + ")");
      ++position;
      return false;
    }
    memcpy(out, s->value, bytes);
    return true;
  }
  // integer attribute of any signed width (MLIR i32/i64 both appear in backend_config)
  bool Int(const char* name, int64_t* out) {
    const int i = Find(name);
    if (i >= 0 && frame->attrs.types[i] == XLA_FFI_AttrType_SCALAR) {
      const XLA_FFI_Scalar* s = static_cast<const XLA_FFI_Scalar*>(frame->attrs.attrs[i]);
      if (s->dtype == XLA_FFI_DataType_S32) {
        int32_t v;
        memcpy(&v, s->value, 4);
        *out = v;
        ++position;
        return true;
      }
    }
    return Scalar(name, XLA_FFI_DataType_S64, out, 8);
  }
  bool String(const char* name, std::string* out) {
    ++position;
    const int i = Find(name);
    if (i < 0) return false;
    if (frame->attrs.types[i] != XLA_FFI_AttrType_STRING) {
      --position;
      Failed(std::string("Wrong attribute type: expected string but got ") +
             AttrTypeName(frame->attrs.types[i]) + " (" + name + ")");
      ++position;
      return false;
    }
    const XLA_FFI_ByteSpan* s = static_cast<const XLA_FFI_ByteSpan*>(frame->attrs.attrs[i]);
    out->assign(s->ptr, s->len);
    return true;
  }
};

constexpr uint64_t Bit(int d) { return 1ull << d; }
constexpr uint64_t kFloatMask = Bit(XLA_FFI_DataType_F32) | Bit(XLA_FFI_DataType_BF16);
constexpr uint64_t kBytesMask = Bit(XLA_FFI_DataType_S8) | Bit(XLA_FFI_DataType_U8);

// The RECORD stage (xla/backends/gpu/runtime/custom_call_thunk.cc:577-684): XLA is building a
// command buffer and asks the handler to add its commands through the record extension.  These
// handlers launch prebuilt kernels on a stream, so they ask for the alternative the record API
// offers -- request_stream_capture (record_c_api.h:189-191) -- and XLA then traces the EXECUTE
// stage into the command buffer, which is what it does for a handler without a record stage.
// Nothing is launched here.
XLA_FFI_Error* AnswerRecord(XLA_FFI_CallFrame* f) {
  const XLA_FFI_Api* api = f->api;
  const size_t need = offsetof(XLA_FFI_Api, XLA_FFI_InvokeContext_FindExtension) + sizeof(void*);
  if (api->struct_size < need || api->XLA_FFI_InvokeContext_FindExtension == nullptr)
    return InvalidArgument(api, "[record] this XLA_FFI_Api has no XLA_FFI_InvokeContext_FindExtension");
  XLA_FFI_InvokeContext_FindExtension_Args a;
  memset(&a, 0, sizeof(a));
  a.struct_size = XLA_FFI_STRUCT_SIZE(XLA_FFI_InvokeContext_FindExtension_Args, extension);
  a.ctx = f->ctx;
  a.extension_type = XLA_FFI_Extension_Record;
  if (XLA_FFI_Error* e = api->XLA_FFI_InvokeContext_FindExtension(&a)) return e;
  const XLA_FFI_Record_Extension* ext = reinterpret_cast<const XLA_FFI_Record_Extension*>(a.extension);
  if (ext == nullptr || ext->extension_base.struct_size < XLA_FFI_Record_Extension_STRUCT_SIZE ||
      ext->extension_base.id.extension_type != XLA_FFI_Extension_Record ||
      ext->extension_base.id.major_version != XLA_FFI_Extension_Record_MajorVersion ||
      ext->record_frame == nullptr || ext->record_frame->api == nullptr ||
      ext->record_frame->api->request_stream_capture == nullptr)
    return InvalidArgument(api, "[record] the call carries no usable record extension (type 128, version 0.x)");
  return ext->record_frame->api->request_stream_capture(ext->record_frame->record_ctx);
}

// Steps shared by all handlers up to operand decoding (api.h:2296-2424).  Returns true when
// the caller should return *err (which may be null for the metadata query).
bool Preamble(XLA_FFI_CallFrame* f, int min_args, int max_args, int min_rets, int max_rets,
              XLA_FFI_Error** err) {
  *err = nullptr;
  if (f->struct_size != XLA_FFI_CallFrame_STRUCT_SIZE) {
    *err = InvalidArgument(f->api, "Unexpected XLA_FFI_CallFrame size: expected " +
                                       std::to_string((size_t)XLA_FFI_CallFrame_STRUCT_SIZE) + " got " +
                                       std::to_string(f->struct_size) +
                                       ". Check installed software versions.");
    return true;
  }
  if (f->extension_start != nullptr && f->extension_start->type == XLA_FFI_Extension_Metadata) {
    auto* ext = reinterpret_cast<XLA_FFI_Metadata_Extension*>(f->extension_start);
    if (ext->extension_base.struct_size < XLA_FFI_Metadata_Extension_STRUCT_SIZE ||
        ext->metadata->struct_size < XLA_FFI_Metadata_STRUCT_SIZE) {
      *err = InvalidArgument(f->api,
                             "Unexpected XLA_FFI_Metadata size. Check installed software versions.");
      return true;
    }
    ext->metadata->api_version.struct_size = XLA_FFI_Api_Version_STRUCT_SIZE;
    ext->metadata->api_version.extension_start = nullptr;
    ext->metadata->api_version.major_version = XLA_FFI_API_MAJOR;
    ext->metadata->api_version.minor_version = XLA_FFI_API_MINOR;
    ext->metadata->traits = XLA_FFI_HANDLER_TRAITS_COMMAND_BUFFER_COMPATIBLE;
    ext->metadata->state_type_id.type_id = 0;  // stateless
    return true;
  }
  if (f->stage == XLA_FFI_ExecutionStage_RECORD) {
    *err = AnswerRecord(f);
    return true;
  }
  if (f->stage != XLA_FFI_ExecutionStage_EXECUTE) {
    *err = InvalidArgument(f->api, std::string("Wrong execution stage: expected `execute` but got `") +
                                       StageName(f->stage) + "`");
    return true;
  }
  const std::string tag = std::string("[") + StageName(f->stage) + "] ";
  if (f->args.size < min_args || f->args.size > max_args) {
    *err = InvalidArgument(
        f->api, tag + "Wrong number of arguments: expected " +
                    (min_args == max_args ? std::to_string(min_args)
                                          : "at least " + std::to_string(min_args)) +
                    " but got " + std::to_string(f->args.size));
    return true;
  }
  if (f->rets.size < min_rets || f->rets.size > max_rets) {
    *err = InvalidArgument(
        f->api, tag + "Wrong number of results: expected " +
                    (min_rets == max_rets ? std::to_string(min_rets)
                                          : "at least " + std::to_string(min_rets)) +
                    " but got " + std::to_string(f->rets.size));
    return true;
  }
  return false;
}

XLA_FFI_Error* GetStream(XLA_FFI_CallFrame* f, void** stream) {
  XLA_FFI_Stream_Get_Args args;
  args.struct_size = XLA_FFI_Stream_Get_Args_STRUCT_SIZE;
  args.extension_start = nullptr;
  args.ctx = f->ctx;
  args.stream = nullptr;
  if (XLA_FFI_Error* e = f->api->XLA_FFI_Stream_Get(&args)) return e;
  *stream = args.stream;
  return nullptr;
}

bool ParseEpilogue(const std::string& s, int* out) {
  static const char* names[] = {"DEFAULT", "BIAS", "RELU", "BIAS_RELU",
                                "GELU", "BIAS_GELU", "SILU", "BIAS_SILU"};
  for (int i = 0; i < 8; ++i)
    if (s == names[i]) {
      *out = i;
      return true;
    }
  return false;
}

XLA_FFI_Error* LaunchStatus(XLA_FFI_CallFrame* f, int rc) {
  if (rc == 0) return nullptr;
  return MakeError(f->api, (XLA_FFI_Error_Code)rc, xla_amd_last_error());
}

int64_t Elements(const XLA_FFI_Buffer* b) {
  int64_t n = 1;
  for (int64_t i = 0; i < b->rank; ++i) n *= b->dims[i];
  return n;
}

struct CommonAttrs {
  int epilogue = XLA_AMD_EPI_DEFAULT;
  int32_t dequant_type = XLA_FFI_DataType_F32;
  int32_t dot_type = XLA_FFI_DataType_F32;
  int32_t epilogue_type = XLA_FFI_DataType_F32;
};

void DecodeCommonAttrs(Decoder& d, CommonAttrs* a) {
  std::string epi;
  if (d.String("epilogue", &epi) && !ParseEpilogue(epi, &a->epilogue)) {
    --d.position;
    d.Failed("Unknown epilogue `" + epi + "`");
    ++d.position;
  }
  int64_t v;
  if (d.Int("dequant_type", &v)) a->dequant_type = (int32_t)v;
  if (d.Int("dot_type", &v)) a->dot_type = (int32_t)v;
  if (d.Int("epilogue_type", &v)) a->epilogue_type = (int32_t)v;
}

}  // namespace
}  // namespace xla_amd

using namespace xla_amd;

extern "C" {

XLA_FFI_Error* xla_amd_dequant_dot(XLA_FFI_CallFrame* f) {
  XLA_FFI_Error* err;
  if (Preamble(f, 3, 7, 1, 2, &err)) return err;
  Decoder d{f};
  // a ragged dot brings its group sizes (S32 or S64 [groups]) as the last operand
  int64_t nargs = f->args.size;
  XLA_FFI_Buffer* gs = nullptr;
  // an F8E4M3FN result brings its scale (one F32) as the last operand
  const bool out_f8 = f->rets.types[0] == XLA_FFI_RetType_BUFFER &&
                      static_cast<XLA_FFI_Buffer*>(f->rets.rets[0])->dtype == XLA_FFI_DataType_F8E4M3FN;
  XLA_FFI_Buffer* sd = nullptr;
  if (out_f8) {
    if (nargs < 4)
      return InvalidArgument(f->api, "xla_amd.dequant_dot: an F8E4M3FN result takes d_scale as the last operand");
    sd = d.Arg((int)nargs - 1, Bit(XLA_FFI_DataType_F32), 0, 0, "d_scale");
    --nargs;
  }
  if (nargs > 3 && f->args.types[nargs - 1] == XLA_FFI_ArgType_BUFFER) {
    XLA_FFI_Buffer* last = static_cast<XLA_FFI_Buffer*>(f->args.args[nargs - 1]);
    if (last->dtype == XLA_FFI_DataType_S32 || last->dtype == XLA_FFI_DataType_S64) {
      gs = d.Arg((int)nargs - 1, Bit(XLA_FFI_DataType_S32) | Bit(XLA_FFI_DataType_S64), 1, 1, "group_sizes");
      --nargs;
    }
  }
  XLA_FFI_Buffer* lhs = d.Arg(0, Bit(XLA_FFI_DataType_BF16), 2, 3, "lhs");
  XLA_FFI_Buffer* w = d.Arg(1, Bit(XLA_FFI_DataType_S8) | Bit(XLA_FFI_DataType_S4) | Bit(XLA_FFI_DataType_U4), 2, 3,
                            "weights");
  XLA_FFI_Buffer* sc = d.Arg(2, kFloatMask, 1, 3, "scales");
  // operands: lhs, weights, scales[, zero_points][, bias] -- a U4 operand after the scales is the
  // zero points (one per scale), a float one the bias
  const bool has_zp = nargs > 3 && f->args.types[3] == XLA_FFI_ArgType_BUFFER &&
                      static_cast<XLA_FFI_Buffer*>(f->args.args[3])->dtype == XLA_FFI_DataType_U4;
  XLA_FFI_Buffer* zp = has_zp ? d.Arg(3, Bit(XLA_FFI_DataType_U4), 1, 3, "zero_points") : nullptr;
  const int bias_at = has_zp ? 4 : 3;
  XLA_FFI_Buffer* bias = nargs > bias_at ? d.Arg(bias_at, kFloatMask, 1, 1, "bias") : nullptr;
  if (((!has_zp && nargs > 4) || nargs > 5) && d.ok())
    return InvalidArgument(f->api, "xla_amd.dequant_dot: five operands are lhs, weights, scales, zero_points (U4), bias");
  XLA_FFI_Buffer* out = d.Ret(0, Bit(XLA_FFI_DataType_BF16) | Bit(XLA_FFI_DataType_F32) | Bit(XLA_FFI_DataType_F8E4M3FN),
                              2, 3, "out");
  XLA_FFI_Buffer* ws = f->rets.size > 1 ? d.Ret(1, kBytesMask, 1, 1, "scratch") : nullptr;
  CommonAttrs a;
  DecodeCommonAttrs(d, &a);
  bool d_mul = false;
  d.Scalar("d_scale_multiplies", XLA_FFI_DataType_PRED, &d_mul, 1);
  int64_t group_size = 0;
  const bool has_group_size = d.Int("scale_group_size", &group_size);
  int64_t rcd = 0;  // 1: weights [..,N,K], scales [N] | [B,N] | [N,K/g] | [B,N,K/g]
  d.Int("rhs_contracting_dim", &rcd);
  int64_t lcd = -1;  // which of lhs's last two dimensions the dot contracts: 1 (default) = the minor one, lhs [..,M,K]
  const bool has_lcd = d.Int("lhs_contracting_dim", &lcd);
  uint8_t transposed_attr = 0;  // the dequantised weights were the dot's lhs: out is [..,N,M]
  d.Scalar("result_transposed", XLA_FFI_DataType_PRED, &transposed_attr, 1);
  const bool transposed = transposed_attr != 0;
  if (!d.ok()) return d.Error();
  const bool nk = rcd == 1;
  const bool lhs_k_major = has_lcd && lcd == 0;

  // ragged: lhs [M,K] (rows sorted by group), weights [groups,K,N], out [M,N]; the groups take the
  // place of the batch for weights and scales
  const bool ragged = gs != nullptr;
  const bool batched = lhs->rank == 3 || ragged;
  XlaAmdDequantDot p{};
  p.batch = ragged ? (w->rank == 3 ? w->dims[0] : 0) : batched ? lhs->dims[0] : 1;
  p.M = lhs->dims[lhs->rank - (lhs_k_major ? 1 : 2)];
  p.K = lhs->dims[lhs->rank - (lhs_k_major ? 2 : 1)];
  p.N = w->dims[w->rank - (nk ? 2 : 1)];
  p.rhs_contracting_dim = (int32_t)rcd;
  std::string why;
  if (rcd != 0 && rcd != 1) why = "rhs_contracting_dim must be 0 or 1";
  else if (has_lcd && lcd != 0 && lcd != 1) why = "lhs_contracting_dim must be 0 (lhs [..,K,M]) or 1 (lhs [..,M,K])";
  else if (ragged && (transposed || lhs_k_major || out->dtype != XLA_FFI_DataType_BF16))
    why = "a ragged dot writes bf16 [M,N] from lhs [M,K]";
  else if (transposed && a.epilogue != 0) why = "a transposed result takes the DEFAULT epilogue only";
  else if (nk && !has_group_size) why = "weights [N,K] come with scale_group_size";
  else if (ragged && (lhs->rank != 2 || w->rank != 3)) why = "a ragged dot takes lhs [M,K] and weights [groups,K,N]";
  else if (ragged && gs->dims[0] != p.batch) why = "group_sizes must have one entry per group of weights";
  else if (!ragged && w->rank != lhs->rank) why = "lhs and weights must have the same rank";
  else if (w->dims[w->rank - (nk ? 1 : 2)] != p.K) why = "contracting dimensions differ";
  else if (!ragged && batched && w->dims[0] != p.batch) why = "batch dimensions differ";
  else if (out->rank != lhs->rank || out->dims[out->rank - (transposed ? 2 : 1)] != p.N ||
           out->dims[out->rank - (transposed ? 1 : 2)] != p.M || (!ragged && batched && out->dims[0] != p.batch))
    why = transposed ? "result shape must be [batch,]N,M" : "result shape must be [batch,]M,N";
  else if (!(nk && group_size > 0) && sc->dims[sc->rank - 1] != p.N) why = "scales must have N as their last dimension";
  else if (bias && bias->dims[0] != p.N) why = "bias must have N elements";
  else if (zp && w->dtype != XLA_FFI_DataType_U4) why = "zero points go with U4 weights";
  else if (zp && (zp->rank != sc->rank || memcmp(zp->dims, sc->dims, sizeof(int64_t) * sc->rank) != 0))
    why = "zero points must have the shape of the scales (one per scale)";
  else if (((a.epilogue & 1) != 0) != (bias != nullptr)) why = "a bias operand goes with a BIAS* epilogue, and only with one";
  if (why.empty()) {
    // scales: [N] | [G,N] | [B,N] | [B,G,N].  scale_group_size says which: 0 = one scale per output
    // channel (then a rank-2 [x,N] is per batch), g > 0 = one per g rows of K (then a rank-2 [x,N]
    // is [K/g,N], shared by the batch).  Without the attribute a rank-2 [x,N] on a batched call is
    // taken per batch when x == batch and per group otherwise, and refused when both readings fit.
    int64_t groups = 1;
    p.scale_batch = 1;
    if (has_group_size) {
      if (group_size < 0 || (group_size > 0 && p.K % group_size != 0)) why = "scale_group_size must divide K";
      else if (nk && group_size > 0) {
        groups = p.K == 0 ? 1 : p.K / group_size;
        if (sc->rank == 3) p.scale_batch = sc->dims[0];
        if (sc->rank < 2 || sc->dims[sc->rank - 1] != groups || sc->dims[sc->rank - 2] != p.N)
          why = "scales of weights [N,K] must be [batch,]N,K/scale_group_size";
      } else {
        groups = group_size == 0 || p.K == 0 ? 1 : p.K / group_size;
        const bool per_channel = group_size == 0;
        if (sc->rank == 3) {
          p.scale_batch = sc->dims[0];
          if (sc->dims[1] != groups) why = "scales must be [batch,K/scale_group_size,N]";
        } else if (sc->rank == 2) {
          if (per_channel) p.scale_batch = sc->dims[0];
          else if (sc->dims[0] != groups) why = "scales must be [K/scale_group_size,N]";
        } else if (groups != 1) {
          why = "rank-1 scales go with scale_group_size = 0";
        }
      }
    } else if (sc->rank == 3) {
      p.scale_batch = sc->dims[0];
      groups = sc->dims[1];
    } else if (sc->rank == 2) {
      const int64_t x = sc->dims[0];
      if (batched && x == p.batch && p.batch > 1 && x < p.K && p.K % x == 0)
        why = "rank-2 scales [" + std::to_string(x) + ",N] can be read per batch or per group of " +
              std::to_string(p.K / x) + " rows: set scale_group_size, or pass rank-3 scales";
      else if (batched && x == p.batch) p.scale_batch = p.batch;
      else groups = x;
    }
    if (!why.empty()) {
    } else if (groups <= 0 || (p.K > 0 && p.K % groups != 0)) why = "the number of scale groups must divide K";
    else if (p.scale_batch != 1 && p.scale_batch != p.batch) why = "scales batch dimension differs";
    else p.group = p.K > 0 ? p.K / groups : 1;
  }
  if (!why.empty()) return InvalidArgument(f->api, "xla_amd.dequant_dot: " + why);

  p.lhs = lhs->data; p.weights = w->data; p.scales = sc->data;
  p.bias = bias ? bias->data : nullptr;
  p.zero_points = zp ? zp->data : nullptr;
  p.group_sizes = gs ? gs->data : nullptr;
  p.group_sizes_dtype = gs ? gs->dtype : 0;
  p.out = out->data;
  p.workspace = ws ? ws->data : nullptr;
  p.workspace_bytes = ws ? (size_t)Elements(ws) : 0;
  p.weight_dtype = w->dtype; p.scale_dtype = sc->dtype;
  p.bias_dtype = bias ? bias->dtype : XLA_FFI_DataType_F32;
  p.dequant_type = a.dequant_type; p.dot_type = a.dot_type; p.epilogue_type = a.epilogue_type;
  p.epilogue = a.epilogue;
  p.out_dtype = out->dtype;
  p.d_scale = sd ? (const float*)sd->data : nullptr;
  p.d_scale_multiplies = d_mul;
  p.out_transposed = transposed ? 1 : 0;
  p.lhs_k_major = lhs_k_major ? 1 : 0;
  void* stream;
  if (XLA_FFI_Error* e = GetStream(f, &stream)) return e;
  return LaunchStatus(f, xla_amd_launch_dequant_dot(&p, stream));
}

XLA_FFI_Error* xla_amd_fp8_scaled_dot(XLA_FFI_CallFrame* f) {
  XLA_FFI_Error* err;
  if (Preamble(f, 4, 6, 1, 3, &err)) return err;
  Decoder d{f};
  const uint64_t f8 = Bit(XLA_FFI_DataType_F8E4M3FN);
  XLA_FFI_Buffer* a = d.Arg(0, f8, 2, 3, "a");
  XLA_FFI_Buffer* b = d.Arg(1, f8, 2, 3, "b");
  // per-tensor / per-row / per-channel f32 scales, or f8e8m0fnu block scales [rows, K/32] on both
  const bool mx = f->args.size > 3 && f->args.types[2] == XLA_FFI_ArgType_BUFFER &&
                  static_cast<XLA_FFI_Buffer*>(f->args.args[2])->dtype == XLA_FFI_DataType_F8E8M0FNU;
  XLA_FFI_Buffer* sa = mx ? d.Arg(2, Bit(XLA_FFI_DataType_F8E8M0FNU), 2, 3, "a_scale")
                          : d.Arg(2, Bit(XLA_FFI_DataType_F32), 0, 1, "a_scale");
  XLA_FFI_Buffer* sb = mx ? d.Arg(3, Bit(XLA_FFI_DataType_F8E8M0FNU), 2, 3, "b_scale")
                          : d.Arg(3, Bit(XLA_FFI_DataType_F32), 0, 1, "b_scale");
  // an F8E4M3FN result brings its scale as the last operand; a bias, if any, sits before it
  const bool out_f8 = f->rets.types[0] == XLA_FFI_RetType_BUFFER &&
                      static_cast<XLA_FFI_Buffer*>(f->rets.rets[0])->dtype == XLA_FFI_DataType_F8E4M3FN;
  const int64_t n_bias = f->args.size - 4 - (out_f8 ? 1 : 0);
  if (n_bias < 0 || n_bias > 1)
    return InvalidArgument(f->api, out_f8 ? "xla_amd.fp8_scaled_dot: an F8E4M3FN result takes a, b, a_scale, b_scale, "
                                            "[bias,] d_scale"
                                          : "xla_amd.fp8_scaled_dot: a BF16 result takes a, b, a_scale, b_scale[, bias]");
  XLA_FFI_Buffer* bias = n_bias ? d.Arg(4, kFloatMask, 1, 1, "bias") : nullptr;
  XLA_FFI_Buffer* sd = out_f8 ? d.Arg(4 + (int)n_bias, Bit(XLA_FFI_DataType_F32), 0, 0, "d_scale") : nullptr;
  XLA_FFI_Buffer* out = d.Ret(0, Bit(XLA_FFI_DataType_BF16) | Bit(XLA_FFI_DataType_F8E4M3FN), 2, 3, "out");
  // after out: an f32 scalar is the amax of an f8 result, a byte vector is scratch
  XLA_FFI_Buffer* amax = nullptr;
  XLA_FFI_Buffer* ws = nullptr;
  for (int64_t i = 1; i < f->rets.size; ++i) {
    const bool scalar_f32 = f->rets.types[i] == XLA_FFI_RetType_BUFFER &&
                            static_cast<XLA_FFI_Buffer*>(f->rets.rets[i])->dtype == XLA_FFI_DataType_F32;
    if (scalar_f32 && out_f8 && !amax && !ws) amax = d.Ret((int)i, Bit(XLA_FFI_DataType_F32), 0, 0, "amax");
    else if (!ws) ws = d.Ret((int)i, kBytesMask, 1, 1, "scratch");
    else return InvalidArgument(f->api, "xla_amd.fp8_scaled_dot: results are out[, amax][, scratch]");
  }
  CommonAttrs at;
  DecodeCommonAttrs(d, &at);
  int64_t rcd = 0;
  d.Int("rhs_contracting_dim", &rcd);
  bool d_mul = false;
  d.Scalar("d_scale_multiplies", XLA_FFI_DataType_PRED, &d_mul, 1);
  if (!d.ok()) return d.Error();

  XlaAmdFp8ScaledDot p{};
  const int lead = a->rank == 3 ? 1 : 0;  // one leading batch dimension, on all three or on none
  p.M = a->dims[lead];
  p.K = a->dims[lead + 1];
  p.batch = lead ? (a->dims[0] > 0 ? a->dims[0] : -1) : 1;  // -1: an empty batch, nothing to do
  std::string why;
  if (rcd != 0 && rcd != 1) why = "rhs_contracting_dim must be 0 or 1";
  else if (mx && rcd != 1) why = "block scales go with a [M,K] and b [N,K]";
  else if (mx && (sa->rank != a->rank || sb->rank != a->rank)) why = "block scales have the rank of their operand";
  else if (b->rank != a->rank || out->rank != a->rank) why = "a, b and out must have the same rank";
  else if (lead && (b->dims[0] != p.batch || out->dims[0] != p.batch)) why = "batch dimensions differ";
  else if (lead && !mx && (sa->rank != 0 || sb->rank != 0)) why = "a batched dot takes per-tensor scales";
  else if (lead && mx && (sa->dims[0] != p.batch || sb->dims[0] != p.batch)) why = "batch dimensions differ";
  else {
    p.N = b->dims[lead + 1 - rcd];
    if (b->dims[lead + rcd] != p.K) why = "contracting dimensions differ";
    else if (out->dims[lead] != p.M || out->dims[lead + 1] != p.N) why = "result shape must be M,N";
    else if (bias && bias->dims[0] != p.N) why = "bias must have N elements";

    else if (((at.epilogue & 1) != 0) != (bias != nullptr)) why = "a bias operand goes with a BIAS* epilogue, and only with one";
    else if (mx && (p.K % 32 != 0 || sa->dims[lead] != p.M || sb->dims[lead] != p.N || sa->dims[lead + 1] != p.K / 32 ||
                    sb->dims[lead + 1] != p.K / 32))
      why = "block scales must be [M,K/32] and [N,K/32]";
    else if (!mx && sa->rank == 1 && sa->dims[0] != p.M) why = "a rank-1 a_scale must have M elements";
    else if (!mx && sb->rank == 1 && sb->dims[0] != p.N) why = "a rank-1 b_scale must have N elements";
  }
  if (!why.empty()) return InvalidArgument(f->api, "xla_amd.fp8_scaled_dot: " + why);
  p.a = a->data; p.b = b->data;
  if (mx) {
    p.a_block_scales = sa->data; p.b_block_scales = sb->data;
    p.block = 32;
  } else {
    p.a_scale = (const float*)sa->data; p.b_scale = (const float*)sb->data;
    p.a_scale_per_row = sa->rank == 1;
    p.b_scale_per_channel = sb->rank == 1;
  }
  p.out_dtype = out->dtype;
  p.d_scale = sd ? (const float*)sd->data : nullptr;
  p.d_scale_multiplies = d_mul;
  p.amax = amax ? (float*)amax->data : nullptr;
  p.bias = bias ? bias->data : nullptr;
  p.out = out->data;
  p.workspace = ws ? ws->data : nullptr;
  p.workspace_bytes = ws ? (size_t)Elements(ws) : 0;
  p.rhs_contracting_dim = (int32_t)rcd;
  p.bias_dtype = bias ? bias->dtype : XLA_FFI_DataType_F32;
  p.dequant_type = at.dequant_type; p.dot_type = at.dot_type; p.epilogue_type = at.epilogue_type;
  p.epilogue = at.epilogue;
  void* stream;
  if (XLA_FFI_Error* e = GetStream(f, &stream)) return e;
  return LaunchStatus(f, xla_amd_launch_fp8_scaled_dot(&p, stream));
}

XLA_FFI_Error* xla_amd_rowwise_quantize_fp8(XLA_FFI_CallFrame* f) {
  XLA_FFI_Error* err;
  if (Preamble(f, 1, 2, 2, 2, &err)) return err;
  Decoder d{f};
  XLA_FFI_Buffer* x = d.Arg(0, Bit(XLA_FFI_DataType_BF16), 2, 2, "x");
  XLA_FFI_Buffer* g = f->args.size > 1 ? d.Arg(1, Bit(XLA_FFI_DataType_BF16), 1, 1, "gamma") : nullptr;
  XLA_FFI_Buffer* q = d.Ret(0, Bit(XLA_FFI_DataType_F8E4M3FN), 2, 2, "q");
  XLA_FFI_Buffer* s = d.Ret(1, Bit(XLA_FFI_DataType_F32), 1, 1, "scales");
  bool rms = true;
  float eps = 1e-6f;
  d.Scalar("rmsnorm", XLA_FFI_DataType_PRED, &rms, 1);
  d.Scalar("eps", XLA_FFI_DataType_F32, &eps, 4);
  if (!d.ok()) return d.Error();
  std::string why;
  if (q->dims[0] != x->dims[0] || q->dims[1] != x->dims[1]) why = "q must have the shape of x";
  else if (s->dims[0] != x->dims[0]) why = "scales must have one entry per row";
  else if (rms && !g) why = "rmsnorm needs the gamma operand";
  else if (!rms && g) why = "gamma operand given but rmsnorm is false";
  else if (g && g->dims[0] != x->dims[1]) why = "gamma must have one entry per column";
  if (!why.empty()) return InvalidArgument(f->api, "xla_amd.rowwise_quantize_fp8: " + why);
  XlaAmdRowwiseQuantize p{};
  p.x = x->data; p.gamma = g ? g->data : nullptr; p.q = q->data; p.scales = (float*)s->data;
  p.rows = x->dims[0]; p.cols = x->dims[1]; p.eps = eps; p.rmsnorm = rms ? 1 : 0;
  void* stream;
  if (XLA_FFI_Error* e = GetStream(f, &stream)) return e;
  return LaunchStatus(f, xla_amd_launch_rowwise_quantize_fp8(&p, stream));
}

XLA_FFI_Error* xla_amd_register_handlers(const XLA_FFI_Api* api) {
  struct Entry { const char* name; XLA_FFI_Handler* fn; };
  const Entry entries[] = {{XLA_AMD_TARGET_DEQUANT_DOT, xla_amd_dequant_dot},
                           {XLA_AMD_TARGET_FP8_SCALED_DOT, xla_amd_fp8_scaled_dot},
                           {XLA_AMD_TARGET_QUANTIZE_FP8, xla_amd_rowwise_quantize_fp8}};
  for (const Entry& e : entries) {
    XLA_FFI_Handler_Register_Args args;
    memset(&args, 0, sizeof(args));
    args.struct_size = XLA_FFI_Handler_Register_Args_STRUCT_SIZE;
    args.name = XLA_FFI_ByteSpan{e.name, strlen(e.name)};
    args.platform = XLA_FFI_ByteSpan{"ROCM", 4};
    args.bundle.execute = e.fn;
    args.bundle.record = e.fn;  // the RECORD stage asks for stream capture of the execute stage
    args.traits = XLA_FFI_HANDLER_TRAITS_COMMAND_BUFFER_COMPATIBLE;
    if (XLA_FFI_Error* err = api->XLA_FFI_Handler_Register(&args)) return err;
  }
  return nullptr;
}

}  // extern "C"
