// Compiled by tests/test_ffi_reference_headers.py against the reference's own FFI headers
// (-I<reference root>): the three handlers of libxla_amd_quant.so registered with the real
// XLA_FFI_REGISTER_HANDLER macro (xla/ffi/api/api.h:2881-2891), exactly as the translation unit a
// maintainer adds to an XLA build would, against the XLA_FFI_Api table of libxla_amd_host.so.
// The registration runs from static initialisers when this object is loaded.
#include "xla/ffi/api/api.h"
#include "xla/ffi/api/c_api.h"

extern "C" {
XLA_FFI_Error* xla_amd_dequant_dot(XLA_FFI_CallFrame*);
XLA_FFI_Error* xla_amd_fp8_scaled_dot(XLA_FFI_CallFrame*);
XLA_FFI_Error* xla_amd_rowwise_quantize_fp8(XLA_FFI_CallFrame*);
void* xla_amd_host_create(void);
const XLA_FFI_Api* xla_amd_host_api(void* host);
}

static const XLA_FFI_Api* HostApi() {
  static void* host = xla_amd_host_create();
  return xla_amd_host_api(host);
}

// execute and record stages are the same symbol: at RECORD the handler asks for stream capture
#define XLA_AMD_BUNDLE(fn) (XLA_FFI_Handler_Bundle{nullptr, nullptr, nullptr, fn, fn})

XLA_FFI_REGISTER_HANDLER(HostApi(), "xla_amd.dequant_dot", "ROCM", XLA_AMD_BUNDLE(xla_amd_dequant_dot),
                         XLA_FFI_HANDLER_TRAITS_COMMAND_BUFFER_COMPATIBLE);
XLA_FFI_REGISTER_HANDLER(HostApi(), "xla_amd.fp8_scaled_dot", "ROCM", XLA_AMD_BUNDLE(xla_amd_fp8_scaled_dot),
                         XLA_FFI_HANDLER_TRAITS_COMMAND_BUFFER_COMPATIBLE);
XLA_FFI_REGISTER_HANDLER(HostApi(), "xla_amd.rowwise_quantize_fp8", "ROCM",
                         XLA_AMD_BUNDLE(xla_amd_rowwise_quantize_fp8), XLA_FFI_HANDLER_TRAITS_COMMAND_BUFFER_COMPATIBLE);

// A second registration of the same handler under the same name is accepted (the library linked
// twice); the same name with another handler is refused.  Returns the two error codes.
extern "C" int register_again(int* same_handler_code, int* other_handler_code) {
  const XLA_FFI_Api* api = HostApi();
  auto code_of = [&](XLA_FFI_Error* e) {
    if (!e) return 0;
    XLA_FFI_Error_GetDetails_Args d;
    d.struct_size = XLA_FFI_Error_GetDetails_Args_STRUCT_SIZE;
    d.extension_start = nullptr;
    d.error = e;
    api->XLA_FFI_Error_GetDetails(&d);
    const int code = (int)d.errc;
    XLA_FFI_Error_Destroy_Args x;
    x.struct_size = XLA_FFI_Error_Destroy_Args_STRUCT_SIZE;
    x.extension_start = nullptr;
    x.error = e;
    api->XLA_FFI_Error_Destroy(&x);
    return code;
  };
  *same_handler_code = code_of(xla::ffi::Ffi::RegisterStaticHandler(
      api, "xla_amd.dequant_dot", "rocm", XLA_AMD_BUNDLE(xla_amd_dequant_dot),
      XLA_FFI_HANDLER_TRAITS_COMMAND_BUFFER_COMPATIBLE));
  *other_handler_code = code_of(xla::ffi::Ffi::RegisterStaticHandler(
      api, "xla_amd.dequant_dot", "ROCM", XLA_AMD_BUNDLE(xla_amd_fp8_scaled_dot),
      XLA_FFI_HANDLER_TRAITS_COMMAND_BUFFER_COMPATIBLE));
  return 0;
}
