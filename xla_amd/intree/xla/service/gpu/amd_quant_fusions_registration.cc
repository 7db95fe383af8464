/* Registers the handlers of libxla_amd_quant.so with XLA's FFI registry at load time.  Add to the
 * ROCm build of XLA and link the library.  The same three lines are compiled and run against the
 * reference's real api.h by tests/test_ffi_reference_headers.py (tests/ffi_ref/register_static.cc). */
#include "xla/ffi/api/api.h"
#include "xla/ffi/api/c_api.h"
#include "xla/ffi/ffi_api.h"

extern "C" {
XLA_FFI_Error* xla_amd_dequant_dot(XLA_FFI_CallFrame*);
XLA_FFI_Error* xla_amd_fp8_scaled_dot(XLA_FFI_CallFrame*);
XLA_FFI_Error* xla_amd_rowwise_quantize_fp8(XLA_FFI_CallFrame*);
}

// execute and record stage are the same symbol: at RECORD the handler asks for stream capture
#define XLA_AMD_BUNDLE(fn) (XLA_FFI_Handler_Bundle{nullptr, nullptr, nullptr, fn, fn})

XLA_FFI_REGISTER_HANDLER(xla::ffi::GetXlaFfiApi(), "xla_amd.dequant_dot", "ROCM", XLA_AMD_BUNDLE(xla_amd_dequant_dot),
                         XLA_FFI_HANDLER_TRAITS_COMMAND_BUFFER_COMPATIBLE);
XLA_FFI_REGISTER_HANDLER(xla::ffi::GetXlaFfiApi(), "xla_amd.fp8_scaled_dot", "ROCM",
                         XLA_AMD_BUNDLE(xla_amd_fp8_scaled_dot), XLA_FFI_HANDLER_TRAITS_COMMAND_BUFFER_COMPATIBLE);
XLA_FFI_REGISTER_HANDLER(xla::ffi::GetXlaFfiApi(), "xla_amd.rowwise_quantize_fp8", "ROCM",
                         XLA_AMD_BUNDLE(xla_amd_rowwise_quantize_fp8), XLA_FFI_HANDLER_TRAITS_COMMAND_BUFFER_COMPATIBLE);
