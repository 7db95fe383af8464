// Interface of the HLO rewrite pass that replaces quantized-inference patterns with this
// library's custom calls (see quant_fusion_rewriter.cc for the patterns).
#ifndef XLA_AMD_CSRC_HOST_QUANT_FUSION_REWRITER_H_
#define XLA_AMD_CSRC_HOST_QUANT_FUSION_REWRITER_H_

#include <stddef.h>
#include <stdint.h>

#include <string>
#include <vector>

#include "hlo_ir.h"

namespace xla_amd {
namespace hlo {

// Scratch sizes come from the kernel library (xla_amd_*_workspace_bytes); a null pointer means
// "emit no scratch result".
struct RewriteOptions {
  size_t (*dequant_workspace_bytes)(int64_t batch, int64_t M, int64_t K, int64_t N, int32_t weight_dtype) = nullptr;
  // the same for weights [N,K] (xla_amd_dequant_dot_workspace_bytes_nk)
  size_t (*dequant_nk_workspace_bytes)(int64_t batch, int64_t M, int64_t K, int64_t N, int32_t weight_dtype) = nullptr;
  size_t (*fp8_workspace_bytes)(int64_t M, int64_t K, int64_t N, int32_t rhs_contracting_dim,
                                int32_t dequant_type) = nullptr;
};

struct RewriteLog {
  std::vector<std::string> rewrites;  // "dot.1 -> xla_amd.dequant_dot [BIAS_SILU, s4]"
  std::vector<std::string> refusals;  // why a near-match was left alone
};

// Rewrites in place; returns the number of patterns replaced.
int RunQuantFusionRewriter(Module* mod, const RewriteOptions& opt, RewriteLog* log);

}  // namespace hlo
}  // namespace xla_amd
#endif  // XLA_AMD_CSRC_HOST_QUANT_FUSION_REWRITER_H_
