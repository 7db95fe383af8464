/* In-tree form of the quantized-inference rewrite pass: drop into xla/backends/gpu/transforms/.
 *
 * NOT BUILT IN THIS REPOSITORY: it needs an XLA checkout and bazel.  The rules, their order and
 * every refusal reason are kept in step with the offline matcher
 * (xla_amd/csrc/host/quant_fusion_rewriter.cc, which runs on HLO text and is what the tests here
 * exercise); tests/test_intree_pass_in_step.py compares the two files' refusal reasons and runs the
 * lit tests' modules through the offline matcher.
 *
 * Shape of the class: xla/backends/gpu/transforms/gemm_fusion.h:34-50. */
#ifndef XLA_BACKENDS_GPU_TRANSFORMS_QUANT_FUSION_REWRITER_H_
#define XLA_BACKENDS_GPU_TRANSFORMS_QUANT_FUSION_REWRITER_H_

#include <string>
#include <vector>

#include "absl/container/flat_hash_set.h"
#include "absl/status/statusor.h"
#include "absl/strings/string_view.h"
#include "xla/hlo/ir/hlo_module.h"
#include "xla/hlo/pass/hlo_pass_interface.h"

namespace xla {
namespace gpu {

// Replaces, on ROCm,
//   convert(f8e4m3fn) [* | / scale] -> dot [-> + bias] [-> relu | gelu | silu] [-> f8 result, amax]
//   (convert(s8 | s4 | u4) [- zero points]) * scale -> dot [-> + bias] [-> activation]
//   "__op$block_scaled_dot" on f8e4m3fn operands with f8e8m0fnu scales
//   [RMSNorm ->] amax -> / 448 -> divide -> clamp -> convert(f8e4m3fn)
// by typed-FFI custom calls "xla_amd.fp8_scaled_dot", "xla_amd.dequant_dot" and
// "xla_amd.rowwise_quantize_fp8" (handlers: libxla_amd_quant.so, registered by
// xla/service/gpu/amd_quant_fusions_registration.cc).  Must run before GemmFusion and the gemm
// rewriter passes, and before TreeReductionRewriter splits the quantizer's reductions.  What it does
// not match it leaves untouched and says why with VLOG(1).
class QuantFusionRewriter : public HloModulePass {
 public:
  // `refusals`, if given, receives "<instruction>: <reason>" for every pattern that was recognised
  // but not taken (tests read it; production passes nullptr).
  explicit QuantFusionRewriter(std::vector<std::string>* refusals = nullptr) : refusals_(refusals) {}
  absl::string_view name() const override { return "quant-fusion-rewriter"; }

 protected:
  absl::StatusOr<bool> RunImpl(HloModule* module,
                               const absl::flat_hash_set<absl::string_view>& execution_threads) override;

 private:
  std::vector<std::string>* refusals_;
};

}  // namespace gpu
}  // namespace xla

#endif  // XLA_BACKENDS_GPU_TRANSFORMS_QUANT_FUSION_REWRITER_H_
