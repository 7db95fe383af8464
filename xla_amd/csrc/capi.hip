// C ABI of the launcher layer (include/xla_amd_quant.h, "Layer 2") and the
// per-thread state behind xla_amd_last_error / xla_amd_last_kernel.
#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>

#include "launch.h"

namespace xla_amd {
namespace {
thread_local char g_error[512] = "";
thread_local char g_kernel[128] = "";

// Kernel-selection overrides of the calling thread (a launcher runs on the thread that calls it):
// one thread's tuning sweep does not steer another thread's calls.
struct Option {
  const char* key;
  int value;
};
thread_local Option g_options[] = {{"dequant_dot_kernel", 0}, {"dequant_dot_vec", 0},
                      {"dequant_dot_slices", 0}, {"dequant_dot_waves", 0}, {"dequant_dot_skew", 0}, {"dequant_dot_x", 0}, {"dequant_dot_nk_ct", 0}, {"dequant_dot_pair", 0}, {"dequant_dot_share", 0}, {"dequant_dot_depth", 0}, {"dequant_dot_steps", 0}, {"dequant_dot_strip", 0}, {"handover_test", 0}, {"dequant_dot_ragged_tile", 0},
                      {"fp8_dot_kernel", 0}, {"fp8_decode_slices", 0}, {"fp8_decode_cols", 0}, {"fp8_scales_on_sum", 0},
                      {"quantize_variant", 0}, {"fp8_dot_layout", 0}, {"tiled_epilogue", 0}, {"tiled_tail", 0}};
}  // namespace

int Fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
  return code;
}

void SetLastKernel(const char* name) {
  strncpy(g_kernel, name, sizeof(g_kernel) - 1);
  g_kernel[sizeof(g_kernel) - 1] = 0;
}

int CheckLaunch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e == hipSuccess) return 0;
  return Fail(XLA_FFI_Error_Code_INTERNAL, "%s: kernel launch failed: %s", what, hipGetErrorString(e));
}

int GetOption(const char* key) {
  for (auto& o : g_options)
    if (strcmp(o.key, key) == 0) return o.value;
  return 0;
}

size_t DequantDotDecodeWorkspaceBytes(int64_t batch, int64_t M, int64_t K, int64_t N, bool s4);
size_t DequantDotNkWorkspaceBytes(int64_t batch, int64_t M, int64_t K, int64_t N, bool four_bit);
size_t Fp8ScaledDotWorkspaceBytes(int64_t M, int64_t K, int64_t N, int rhs_contracting_dim, int dequant_type);
size_t TiledTailWorkspaceBytes(int64_t batch, int64_t M, int64_t K, int64_t N);

}  // namespace xla_amd

extern "C" {

int xla_amd_launch_dequant_dot(const XlaAmdDequantDot* p, void* stream) {
  if (!p) return xla_amd::Fail(XLA_FFI_Error_Code_INVALID_ARGUMENT, "dequant_dot: null params");
  return xla_amd::LaunchDequantDot(*p, (hipStream_t)stream);
}

int xla_amd_launch_dequant_dot_static_scratch(const XlaAmdDequantDot* p, void* stream) {
  if (!p) return xla_amd::Fail(XLA_FFI_Error_Code_INVALID_ARGUMENT, "dequant_dot_static_scratch: null params");
  return xla_amd::LaunchDequantDotStaticScratch(*p, (hipStream_t)stream);
}

int xla_amd_launch_fp8_scaled_dot(const XlaAmdFp8ScaledDot* p, void* stream) {
  if (!p) return xla_amd::Fail(XLA_FFI_Error_Code_INVALID_ARGUMENT, "fp8_scaled_dot: null params");
  return xla_amd::LaunchFp8ScaledDot(*p, (hipStream_t)stream);
}

int xla_amd_launch_rowwise_quantize_fp8(const XlaAmdRowwiseQuantize* p, void* stream) {
  if (!p) return xla_amd::Fail(XLA_FFI_Error_Code_INVALID_ARGUMENT, "rowwise_quantize_fp8: null params");
  return xla_amd::LaunchRowwiseQuantize(*p, (hipStream_t)stream, xla_amd::GetOption("quantize_variant"));
}

size_t xla_amd_dequant_dot_workspace_bytes(int64_t batch, int64_t M, int64_t K, int64_t N,
                                           int32_t weight_dtype) {
  const size_t decode = xla_amd::DequantDotDecodeWorkspaceBytes(
      batch, M, K, N, weight_dtype == XLA_FFI_DataType_S4 || weight_dtype == XLA_FFI_DataType_U4);
  // more than 64 tokens may run on the tiled kernel, which splits the tiles of a short last round
  const size_t tail = xla_amd::TiledTailWorkspaceBytes(batch, M, K, N);
  return decode > tail ? decode : tail;
}

size_t xla_amd_dequant_dot_workspace_bytes_nk(int64_t batch, int64_t M, int64_t K, int64_t N,
                                              int32_t weight_dtype) {
  return xla_amd::DequantDotNkWorkspaceBytes(
      batch, M, K, N, weight_dtype == XLA_FFI_DataType_S4 || weight_dtype == XLA_FFI_DataType_U4);
}

size_t xla_amd_fp8_scaled_dot_workspace_bytes(int64_t M, int64_t K, int64_t N,
                                              int32_t rhs_contracting_dim) {
  return xla_amd::Fp8ScaledDotWorkspaceBytes(M, K, N, rhs_contracting_dim, XLA_FFI_DataType_F32);
}

size_t xla_amd_fp8_scaled_dot_workspace_bytes_typed(int64_t M, int64_t K, int64_t N, int32_t rhs_contracting_dim,
                                                    int32_t dequant_type) {
  return xla_amd::Fp8ScaledDotWorkspaceBytes(M, K, N, rhs_contracting_dim, dequant_type);
}

const char* xla_amd_last_error(void) { return xla_amd::g_error; }
const char* xla_amd_last_kernel(void) { return xla_amd::g_kernel; }

int xla_amd_debug_set_option(const char* key, int value) {
  for (auto& o : xla_amd::g_options)
    if (strcmp(o.key, key) == 0) {
      o.value = value;
      return 0;
    }
  return -1;
}

}  // extern "C"
