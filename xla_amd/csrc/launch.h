// Host-side plumbing shared by the launchers: per-thread error text, the name
// of the kernel variant last selected, and the internal launch entry points
// the C ABI in include/xla_amd_quant.h forwards to.
#ifndef XLA_AMD_CSRC_LAUNCH_H_
#define XLA_AMD_CSRC_LAUNCH_H_

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "xla_amd_quant.h"

namespace xla_amd {

// Records `msg` as this thread's last error and returns `code`.
int Fail(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));
void SetLastKernel(const char* name);
// hipGetLastError() after a launch -> 0 or XLA_FFI_Error_Code_INTERNAL with the HIP message.
int CheckLaunch(const char* what);

// Tuning knobs set through xla_amd_debug_set_option (0 = default choice).
int GetOption(const char* key);

int LaunchRowwiseQuantize(const XlaAmdRowwiseQuantize& p, hipStream_t stream, int variant);
int LaunchDequantDot(const XlaAmdDequantDot& p, hipStream_t stream);
// Same, with the split-K partial sums in the library's static device array (allocates nothing).
int LaunchDequantDotStaticScratch(const XlaAmdDequantDot& p, hipStream_t stream);
int LaunchFp8ScaledDot(const XlaAmdFp8ScaledDot& p, hipStream_t stream);
// Up to 64 rows of a per launch (48 with the rhs [N,K]), per-tensor / per-row / per-channel scales under
// f32-typed multiplies: the rhs streamed once (fp8_dot_decode.hip); more rows in passes where that is
// cheaper than tiles.  Returns -1 when the shape is not covered (or tiles are cheaper), else the launch
// status; p comes validated and an amax result already zeroed.  The scratch is the f32 sums of its
// K-slices (0: one slice).
// bf16_multiply: the caller takes care of a bf16-typed dequantise multiply whose per-tensor scales are no
// powers of two (the kernels here then return at once); without it such calls are not covered.
// *any_scale (if given): the launches also cover scales that are no powers of two (rhs [K,N]).
int LaunchFp8DotDecode(const XlaAmdFp8ScaledDot& p, hipStream_t stream, bool bf16_multiply = false,
                       bool* any_scale = nullptr);
size_t Fp8DotDecodeWorkspaceBytes(int64_t batch, int64_t M, int64_t K, int64_t N, int rhs_contracting_dim);

inline bool IsF32OrBf16(int32_t t) {
  return t == XLA_FFI_DataType_F32 || t == XLA_FFI_DataType_BF16;
}

}  // namespace xla_amd
#endif  // XLA_AMD_CSRC_LAUNCH_H_
