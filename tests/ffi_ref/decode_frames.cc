// Compiled by tests/test_ffi_reference_headers.py against the reference's own FFI headers
// (-I<reference root>).  One handler per custom call of this library, written the way an XLA user
// writes one -- Ffi::Bind().Arg<AnyBuffer>()...Attr<T>("name") (xla/ffi/api/api.h:283-312,
// xla/ffi/api/ffi.h) -- so that the reference's decoder (Handler::Call, api.h:2296-2430) is what
// reads the call frames this package's frame builder produces.  Each handler writes down what it
// decoded; the test compares that with what went in.
#include <cstdint>
#include <sstream>
#include <string>
#include <string_view>

#include "xla/ffi/api/ffi.h"

namespace ffi = xla::ffi;

static std::string g_log;

static void Describe(std::ostringstream& os, const char* what, ffi::AnyBuffer b) {
  os << what << " dtype=" << static_cast<int>(b.element_type()) << " dims=[";
  for (size_t i = 0; i < b.dimensions().size(); ++i) os << (i ? "," : "") << b.dimensions()[i];
  os << "] ptr=" << reinterpret_cast<uintptr_t>(b.untyped_data()) << ";";
}

static void DescribeRest(std::ostringstream& os, ffi::RemainingArgs args, ffi::RemainingRets rets) {
  for (size_t i = 0; i < args.size(); ++i) {
    auto b = args.get<ffi::AnyBuffer>(i);
    if (b.has_value()) Describe(os, "arg", *b); else os << "arg ERROR;";
  }
  for (size_t i = 0; i < rets.size(); ++i) {
    auto b = rets.get<ffi::AnyBuffer>(i);
    if (b.has_value()) Describe(os, "ret", **b); else os << "ret ERROR;";
  }
}

static ffi::Error DequantDot(ffi::AnyBuffer lhs, ffi::AnyBuffer weights, ffi::AnyBuffer scales, ffi::RemainingArgs rest,
                             ffi::Result<ffi::AnyBuffer> out, ffi::RemainingRets rest_rets, int32_t dequant_type,
                             int32_t dot_type, std::string_view epilogue, int32_t epilogue_type) {
  std::ostringstream os;
  Describe(os, "arg", lhs); Describe(os, "arg", weights); Describe(os, "arg", scales); Describe(os, "ret", *out);
  DescribeRest(os, rest, rest_rets);
  os << "dequant_type=" << dequant_type << ";dot_type=" << dot_type << ";epilogue=" << epilogue
     << ";epilogue_type=" << epilogue_type << ";";
  g_log = os.str();
  return ffi::Error::Success();
}

static ffi::Error DequantDotGrouped(ffi::AnyBuffer lhs, ffi::AnyBuffer weights, ffi::AnyBuffer scales,
                                    ffi::RemainingArgs rest, ffi::Result<ffi::AnyBuffer> out, ffi::RemainingRets rest_rets,
                                    int32_t dequant_type, int32_t dot_type, std::string_view epilogue,
                                    int32_t epilogue_type, int64_t scale_group_size) {
  ffi::Error e = DequantDot(lhs, weights, scales, rest, out, rest_rets, dequant_type, dot_type, epilogue, epilogue_type);
  g_log += "scale_group_size=" + std::to_string(scale_group_size) + ";";
  return e;
}

static ffi::Error Fp8ScaledDot(ffi::AnyBuffer a, ffi::AnyBuffer b, ffi::AnyBuffer a_scale, ffi::AnyBuffer b_scale,
                               ffi::RemainingArgs rest, ffi::Result<ffi::AnyBuffer> out, ffi::RemainingRets rest_rets,
                               int32_t dequant_type, int32_t dot_type, std::string_view epilogue, int32_t epilogue_type,
                               int64_t rhs_contracting_dim) {
  std::ostringstream os;
  Describe(os, "arg", a); Describe(os, "arg", b); Describe(os, "arg", a_scale); Describe(os, "arg", b_scale);
  Describe(os, "ret", *out);
  DescribeRest(os, rest, rest_rets);
  os << "dequant_type=" << dequant_type << ";dot_type=" << dot_type << ";epilogue=" << epilogue
     << ";epilogue_type=" << epilogue_type << ";rhs_contracting_dim=" << rhs_contracting_dim << ";";
  g_log = os.str();
  return ffi::Error::Success();
}

static ffi::Error Fp8ScaledDotF8Result(ffi::AnyBuffer a, ffi::AnyBuffer b, ffi::AnyBuffer a_scale, ffi::AnyBuffer b_scale,
                                       ffi::RemainingArgs rest, ffi::Result<ffi::AnyBuffer> out,
                                       ffi::RemainingRets rest_rets, bool d_scale_multiplies, int32_t dequant_type,
                                       int32_t dot_type, std::string_view epilogue, int32_t epilogue_type,
                                       int64_t rhs_contracting_dim) {
  ffi::Error e = Fp8ScaledDot(a, b, a_scale, b_scale, rest, out, rest_rets, dequant_type, dot_type, epilogue,
                              epilogue_type, rhs_contracting_dim);
  g_log += std::string("d_scale_multiplies=") + (d_scale_multiplies ? "1" : "0") + ";";
  return e;
}

static ffi::Error RowwiseQuantize(ffi::AnyBuffer x, ffi::RemainingArgs rest, ffi::Result<ffi::AnyBuffer> q,
                                  ffi::Result<ffi::AnyBuffer> scales, float eps, bool rmsnorm) {
  std::ostringstream os;
  Describe(os, "arg", x); Describe(os, "ret", *q); Describe(os, "ret", *scales);
  for (size_t i = 0; i < rest.size(); ++i) {
    auto b = rest.get<ffi::AnyBuffer>(i);
    if (b.has_value()) Describe(os, "arg", *b); else os << "arg ERROR;";
  }
  os << "eps=" << eps << ";rmsnorm=" << (rmsnorm ? 1 : 0) << ";";
  g_log = os.str();
  return ffi::Error::Success();
}

#define DOT_ARGS .Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>()
#define TYPE_ATTRS \
  .Attr<int32_t>("dequant_type").Attr<int32_t>("dot_type").Attr<std::string_view>("epilogue").Attr<int32_t>("epilogue_type")

XLA_FFI_DEFINE_HANDLER_SYMBOL(ref_decode_dequant_dot, DequantDot,
                              ffi::Ffi::Bind() DOT_ARGS.RemainingArgs().Ret<ffi::AnyBuffer>().RemainingRets() TYPE_ATTRS);
XLA_FFI_DEFINE_HANDLER_SYMBOL(ref_decode_dequant_dot_grouped, DequantDotGrouped,
                              ffi::Ffi::Bind() DOT_ARGS.RemainingArgs().Ret<ffi::AnyBuffer>().RemainingRets() TYPE_ATTRS
                                  .Attr<int64_t>("scale_group_size"));
XLA_FFI_DEFINE_HANDLER_SYMBOL(ref_decode_fp8_scaled_dot, Fp8ScaledDot,
                              ffi::Ffi::Bind() DOT_ARGS.Arg<ffi::AnyBuffer>().RemainingArgs().Ret<ffi::AnyBuffer>()
                                  .RemainingRets() TYPE_ATTRS.Attr<int64_t>("rhs_contracting_dim"));
XLA_FFI_DEFINE_HANDLER_SYMBOL(ref_decode_fp8_scaled_dot_f8_result, Fp8ScaledDotF8Result,
                              ffi::Ffi::Bind() DOT_ARGS.Arg<ffi::AnyBuffer>().RemainingArgs().Ret<ffi::AnyBuffer>()
                                  .RemainingRets().Attr<bool>("d_scale_multiplies") TYPE_ATTRS
                                  .Attr<int64_t>("rhs_contracting_dim"));
XLA_FFI_DEFINE_HANDLER_SYMBOL(ref_decode_rowwise_quantize_fp8, RowwiseQuantize,
                              ffi::Ffi::Bind().Arg<ffi::AnyBuffer>().RemainingArgs().Ret<ffi::AnyBuffer>()
                                  .Ret<ffi::AnyBuffer>().Attr<float>("eps").Attr<bool>("rmsnorm"));

extern "C" const char* ref_decode_log() { return g_log.c_str(); }
extern "C" void ref_decode_reset() { g_log.clear(); }
