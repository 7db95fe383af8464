/*
 * libxla_amd_quant.so -- hand-written CDNA4 (gfx950) kernels for XLA's GPU
 * quantized-inference fusions, exposed as XLA typed-FFI custom calls.
 *
 * Two layers, both plain C ABI:
 *   1. XLA FFI handlers: `XLA_FFI_Error* fn(XLA_FFI_CallFrame*)`
 *      (XLA_FFI_Handler, xla/ffi/api/c_api.h:517).  These are what
 *      XLA_FFI_REGISTER_HANDLER(GetXlaFfiApi(), "<target>", "ROCM", fn)
 *      (xla/ffi/api/api.h:2881-2891) binds and what CustomCallThunk invokes
 *      (xla/backends/gpu/runtime/custom_call_thunk.cc:394-422,546-575).
 *   2. Launchers taking raw device pointers, sizes and a hipStream_t, for
 *      callers that have no call frame.  The handlers are thin decoders over
 *      these.
 *
 * Every entry point only enqueues work on the given stream and returns; none
 * synchronises, allocates device memory or reads device data on the host, so
 * all handlers advertise XLA_FFI_HANDLER_TRAITS_COMMAND_BUFFER_COMPATIBLE.
 */
#ifndef XLA_AMD_QUANT_H_
#define XLA_AMD_QUANT_H_

#include <stddef.h>
#include <stdint.h>

#include "xla_ffi_abi.h"

#ifdef __cplusplus
extern "C" {
#endif

#define XLA_AMD_EXPORT __attribute__((visibility("default")))

/* custom_call_target strings the rewrite pass emits */
#define XLA_AMD_TARGET_DEQUANT_DOT "xla_amd.dequant_dot"
#define XLA_AMD_TARGET_FP8_SCALED_DOT "xla_amd.fp8_scaled_dot"
#define XLA_AMD_TARGET_QUANTIZE_FP8 "xla_amd.rowwise_quantize_fp8"

/* ------------------------------------------------------------------------
 * Layer 1: XLA FFI handlers (stage EXECUTE; they also answer the metadata
 * query of xla/ffi/api/api.h:2305-2313 with api version 0.4).
 * ------------------------------------------------------------------------ */

/*
 * Weight-only dequantize-dot.  Replaces the `__triton_gemm` fusion that
 * GemmFusion builds for convert(s4|s8) -> [multiply by broadcast scale] -> dot
 * (xla/backends/gpu/transforms/gemm_fusion.cc:1629-1702) together with the
 * bias/activation epilogue that GemmRewriter folds into a library matmul
 * (xla/backends/gpu/transforms/gemm_rewriter.cc:888-1007,1987-2304).
 *   args, in this order (optional ones are told apart by their element type):
 *         lhs         BF16 [M,K] or [B,M,K]     ([..,K,M] with lhs_contracting_dim = 0)
 *         weights     S8, S4 or U4 [K,N] or [B,K,N]; [N,K] or [B,N,K] with rhs_contracting_dim = 1
 *                     (4-bit: two per byte, low nibble first over the row-major index,
 *                     ir_array.cc:588-603; U4 is unsigned, 0..15)
 *         scales      F32 or BF16 [N] | [K/g,N] | [B,N] | [B,K/g,N]; next to weights [..,N,K]:
 *                     [N] | [B,N] | [N,K/g] | [B,N,K/g]
 *         zero_points U4, shaped like the scales (optional; U4 weights only): the dequantised
 *                     weight is (w - zero_point) * scale
 *         bias        BF16 or F32 [N]            (optional; exactly with a BIAS* epilogue)
 *         d_scale     F32 []                     (exactly with an F8E4M3FN out, after the bias): out is
 *                     convert(clamp(-448, v / d_scale, 448)) of the f32 value v after the epilogue, the D
 *                     scaling of gemm_rewriter_fp8_test.cc:1665-1690 (v * d_scale with d_scale_multiplies,
 *                     :1730-1748) -- the next fp8 dot's activations made in this dot's store
 *         group_sizes S32 or S64 [G], last       (optional): a ragged dot -- lhs [M,K] with its rows
 *                     sorted by group, weights [G,K,N] (or [G,N,K]), out [M,N]; group g multiplies rows
 *                     [sum of the sizes before it, + its size), rows past the last group are epilogue(0)
 *                     (xla ragged-dot, ragged_dot_rewriter.cc:110-210; gemm_rewriter.cc:781-863)
 *   rets: out     BF16, F32 or F8E4M3FN [M,N] or [B,M,N] (F32: the value before the final convert, the
 *                 root of fusion_emitter_int4_device_test.cc:101,205,320,508; F8E4M3FN: with d_scale);
 *                 [..,N,M] with result_transposed
 *         scratch S8 or U8 [bytes]             (optional second result: what
 *                 xla_amd_dequant_dot_workspace_bytes[_nk] reports for the shape; without it the
 *                 kernels that need none run)
 *   attrs (all optional, looked up by name):
 *     epilogue      string: DEFAULT|BIAS|RELU|BIAS_RELU|GELU|BIAS_GELU|SILU|BIAS_SILU
 *                   (GemmBackendConfig.Epilogue, xla/service/gpu/backend_configs.proto:105-119)
 *     dequant_type  i32 XLA dtype of the multiply that applies the scale: 11 (F32, default)
 *                   or 16 (BF16: each dequantised weight is rounded to bf16, as in
 *                   fusion_emitter_int4_device_test.cc:93-104)
 *     dot_type      i32: 11 (default) or 16 -- element type of the dot instruction
 *     epilogue_type i32: 11 (default) or 16 -- element type of the bias add / activation ops
 *     scale_group_size i64: rows of K that share one scale; 0 = all of them (one scale per output
 *                   channel: scales [N] or [B,N]), g > 0: scales [K/g,N] or [B,K/g,N].  The rewrite
 *                   pass always sets it.  Without it the grouping is read off the scales' shape,
 *                   and a batched call whose rank-2 scales fit both readings is refused.
 *     rhs_contracting_dim i64: 0 (default) weights [..,K,N]; 1 weights [..,N,K], 4-bit values packed
 *                   along K (fusion_emitter_int4_device_test.cc:867-892); needs scale_group_size
 *     lhs_contracting_dim i64: 1 (default) lhs [..,M,K]; 0 lhs [..,K,M] (the dot contracts the
 *                   activations' major dimension, shape table :609-645)
 *     result_transposed pred (default false): the dequantised weights were the lhs of the dot
 *                   (Int4WeightsOnTheLhs, :495-523), so out is [..,N,M]; DEFAULT epilogue only
 *     d_scale_multiplies pred (default false): an F8E4M3FN out is v * d_scale, not v / d_scale
 */
XLA_AMD_EXPORT XLA_FFI_Error* xla_amd_dequant_dot(XLA_FFI_CallFrame* call_frame);

/*
 * f8e4m3fn scaled dot.  Replaces `__cublas$lt$matmul$f8`
 * (xla/backends/gpu/transforms/gemm_rewriter.cc:1235-1591, executed by
 * CublasLtMatmulThunk -> hipBLASLt, xla/stream_executor/rocm/hip_blas_lt.cc:468-484).
 *   args: a F8E4M3FN [M,K]; b F8E4M3FN [K,N] (rhs_contracting_dim=0) or [N,K] (=1); or both
 *         with one leading batch dimension ([B,M,K], [B,K,N]|[B,N,K], out [B,M,N]: the batched
 *         dot of gemm_rewriter_fp8_test.cc:941-957), then with per-tensor or block scales only;
 *         a_scale, b_scale F8E8M0FNU [M,K/32], [N,K/32] with b = [N,K]: block-scaled (MXFP8)
 *         operands, "__op$block_scaled_dot" of block_scaling_rewriter.h:48-69 (a leading batch
 *         dimension goes on the scales as well: [B,M,K/32], [B,N,K/32]); otherwise
 *         a_scale F32 [] or [M] (one per row of a, as a row-wise quantizer produces them);
 *         b_scale F32 [] or [N] (one per output channel); bias BF16|F32 [N] (only with BIAS*)
 *         d_scale F32 [] (last; only when out is F8E4M3FN)
 *   rets: out BF16 [M,N], or F8E4M3FN [M,N] = convert(clamp(-448, v / d_scale, 448)) for the
 *         f32 value v after the epilogue (the D scaling of gemm_rewriter_fp8_test.cc:1665-1690,
 *         which GemmRewriter leaves unfused on ROCm, :1710)
 *         then optionally amax F32 [] = max |v| (reduce-maximum of abs, NaN passed on:
 *         gemm_rewriter_fp8_test.cc:2559-2600), only next to an F8E4M3FN out
 *   attrs: epilogue, dequant_type, dot_type, epilogue_type as above;
 *          rhs_contracting_dim i64 (default 0);
 *          d_scale_multiplies pred (default false): v * d_scale instead (:1730-1748)
 * One handler for every size: up to 64 rows of a take kernels that stream the rhs once (HBM-bound), as do
 * a few hundred rows of a matrix with few 256 x 256 tiles (in passes of up to 64 rows); more rows the
 * tiled kernel (MFMA-bound).
 */
XLA_AMD_EXPORT XLA_FFI_Error* xla_amd_fp8_scaled_dot(XLA_FFI_CallFrame* call_frame);

/*
 * Row-wise dynamic quantisation to f8e4m3fn, optionally preceded by RMSNorm.
 * Replaces the chain of reduction + elementwise fusions that PriorityFusion and
 * the row-reduction emitter produce (xla/backends/gpu/codegen/emitters/reduction.cc:840-991).
 *   args: x BF16 [R,C]; gamma BF16 [C] (only when rmsnorm is true)
 *   rets: q F8E4M3FN [R,C]; scales F32 [R]
 *   attrs: rmsnorm bool (default true); eps f32 (default 1e-6)
 */
XLA_AMD_EXPORT XLA_FFI_Error* xla_amd_rowwise_quantize_fp8(XLA_FFI_CallFrame* call_frame);

/*
 * Registers the three handlers above for platform "ROCM" through the table's
 * XLA_FFI_Handler_Register (xla/ffi/ffi_api.cc:280-315) -- the dynamic
 * counterpart of XLA_FFI_REGISTER_HANDLER.  Returns NULL or the first error.
 */
XLA_AMD_EXPORT XLA_FFI_Error* xla_amd_register_handlers(const XLA_FFI_Api* api);

/* ------------------------------------------------------------------------
 * Layer 2: launchers.  Return 0 on success, else an XLA_FFI_Error_Code; the
 * message is available from xla_amd_last_error() on the calling thread.
 * `stream` is a hipStream_t.  dtype / type fields hold XLA_FFI_DataType values.
 * ------------------------------------------------------------------------ */

enum {
  XLA_AMD_EPI_DEFAULT = 0,
  XLA_AMD_EPI_BIAS = 1,
  XLA_AMD_EPI_RELU = 2,
  XLA_AMD_EPI_BIAS_RELU = 3,
  XLA_AMD_EPI_GELU = 4,
  XLA_AMD_EPI_BIAS_GELU = 5,
  XLA_AMD_EPI_SILU = 6,
  XLA_AMD_EPI_BIAS_SILU = 7
};

typedef struct XlaAmdDequantDot {
  const void* lhs;     /* bf16 [batch,M,K] */
  const void* weights; /* s8 [batch,K,N] or packed s4 / u4 */
  const void* scales;  /* [batch or 1, K/group, N] */
  const void* bias;    /* [N] or NULL */
  void* out;           /* bf16 [batch,M,N] */
  void* workspace;     /* optional scratch, see xla_amd_dequant_dot_workspace_bytes */
  size_t workspace_bytes;
  int64_t batch, M, K, N;
  int64_t group;           /* K for per-channel scales */
  int64_t scale_batch;     /* 1 if the scales are shared by all batches, else batch */
  int32_t weight_dtype;    /* S8, S4 or U4 */
  int32_t scale_dtype;     /* F32 or BF16 */
  int32_t bias_dtype;      /* F32 or BF16 */
  int32_t dequant_type, dot_type, epilogue_type; /* F32 or BF16 */
  int32_t epilogue;        /* XLA_AMD_EPI_* */
  /* U4 weights only, or NULL: one u4 zero point per scale, [scale_batch, K/group, N] packed two per
   * byte like the weights; the dequantised weight is (w - zero_point) * scale */
  const void* zero_points;
  /* Ragged dot (xla ragged-dot with the ragged dimension on the rows of lhs): NULL for an ordinary
   * dot.  Otherwise `batch` row counts in device memory, S32 or S64 (group_sizes_dtype): lhs is
   * [M,K] with its rows sorted by group, weights [batch,K,N] hold one matrix per group, out is
   * [M,N]; group g takes rows [sum of the sizes before it, + its size), rows past the last group
   * are a dot of nothing (epilogue(0)).  Never read on the host.  A ragged dot over zero groups
   * (batch = 0, where the pointer of the empty array may be NULL) is told by group_sizes_dtype
   * being S32 or S64: every row of out is then epilogue(0). */
  const void* group_sizes;
  int32_t group_sizes_dtype; /* S32 or S64; 0 for an ordinary dot */
  /* 0: weights [batch,K,N] as above.  1: weights [batch,N,K], the contracting dimension minor
   * (dot ... rhs_contracting_dims={1}, fusion_emitter_int4_device_test.cc:867-892): 4-bit values are
   * packed two per byte along K, scales and zero points are [batch or 1, N, K/group].  With
   * group_sizes the experts are [groups,N,K]. */
  int32_t rhs_contracting_dim;
  /* Element type of out: BF16 (also 0), F32 -- a dot whose f32 value is the result
   * (fusion_emitter_int4_device_test.cc:101,205,320,508) -- or F8E4M3FN with d_scale below. */
  int32_t out_dtype;
  /* 1: out is [batch,N,M]: the dequantised weights were the lhs of the dot
   * (Int4WeightsOnTheLhs, fusion_emitter_int4_device_test.cc:495-523); the epilogue must be DEFAULT. */
  int32_t out_transposed;
  /* 1: lhs (the activations) is stored [batch,K,M]: the dot contracts their major dimension
   * (the "128,16" x "128,256" cases of fusion_emitter_int4_device_test.cc:609-645). */
  int32_t lhs_k_major;
  /* out_dtype F8E4M3FN: out holds convert(clamp(-448, v / d_scale, 448)) of the f32 value v after the
   * epilogue (v * d_scale with d_scale_multiplies), as for xla_amd_fp8_scaled_dot: d_scale is one f32
   * in device memory.  Such calls run on the general kernels (bf16 [M,N] results have the tuned ones). */
  const float* d_scale;
  int32_t d_scale_multiplies;
} XlaAmdDequantDot;

XLA_AMD_EXPORT int xla_amd_launch_dequant_dot(const XlaAmdDequantDot* p, void* stream);

/* Scratch bytes with which the kernels may split K across workgroups (0 = never needed for this
 * shape): the decode kernels' K-slices up to 64 tokens, and above that the tiled kernel's last round
 * of tiles when it is at most half full (256 KiB of f32 sums per tile of that round).  The rewrite pass sizes the custom call's second result with it,
 * the way `__cublas$lt$matmul` carries its workspace (gemm_rewriter_fp8_test.cc:1167).
 * A call without (enough) scratch still works; it just cannot split K. */
XLA_AMD_EXPORT size_t xla_amd_dequant_dot_workspace_bytes(int64_t batch, int64_t M, int64_t K,
                                                          int64_t N, int32_t weight_dtype);

/* The same for weights [batch,N,K] (rhs_contracting_dim = 1): the f32 partial sums of the K-slices
 * a call with few output channels is cut into. */
XLA_AMD_EXPORT size_t xla_amd_dequant_dot_workspace_bytes_nk(int64_t batch, int64_t M, int64_t K,
                                                             int64_t N, int32_t weight_dtype);

/*
 * xla_amd_launch_dequant_dot for callers that cannot allocate device memory (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.
 * p->workspace and p->workspace_bytes are ignored: where the decode kernels split K across
 * workgroups, the f32 partial sums go into a fixed 8 MiB array in device memory that is part of
 * the library's code object (every GPU the library runs on holds its own copy until the process
 * ends); its address is looked up once per device on the first call there.  A shape whose partial
 * sums need more (xla_amd_dequant_dot_workspace_bytes > 8 MiB) is refused with
 * XLA_FFI_Error_Code_RESOURCE_EXHAUSTED.  The call itself allocates nothing and results are
 * bit-identical to xla_amd_launch_dequant_dot with a sufficient workspace.  All calls on one GPU
 * share the array: calls that may overlap on one GPU (different streams) race on it.
 */
XLA_AMD_EXPORT int xla_amd_launch_dequant_dot_static_scratch(const XlaAmdDequantDot* p, void* stream);

typedef struct XlaAmdFp8ScaledDot {
  const void* a;       /* f8e4m3fn [M,K] */
  const void* b;       /* f8e4m3fn [K,N] or [N,K] */
  const float* a_scale; /* device: one value, or M values when a_scale_per_row */
  const float* b_scale; /* device: one value, or N values when b_scale_per_channel */
  const void* bias;
  void* out;           /* bf16 [M,N] */
  void* workspace;     /* optional scratch, see xla_amd_fp8_scaled_dot_workspace_bytes */
  size_t workspace_bytes;
  int64_t M, K, N;
  int32_t rhs_contracting_dim; /* 0: b is [K,N]; 1: b is [N,K] */
  int32_t bias_dtype;
  int32_t dequant_type, dot_type, epilogue_type;
  int32_t epilogue;
  int32_t a_scale_per_row;     /* a_scale is f32[M]: row m of a is scaled by a_scale[m] */
  int32_t b_scale_per_channel; /* b_scale is f32[N]: output channel n of b by b_scale[n] */
  int32_t out_dtype;           /* 0 or XLA_FFI_DataType_BF16: bf16 out; XLA_FFI_DataType_F8E4M3FN:
                                  out = convert(clamp(-448, v / *d_scale, 448)), one byte each */
  int32_t d_scale_multiplies;  /* the f8 result is v * *d_scale instead of v / *d_scale */
  const float* d_scale;        /* device scalar, only with an F8E4M3FN result */
  float* amax;                 /* optional device scalar result with an F8E4M3FN result:
                                  max |v| over all outputs, NaN if any v is NaN */
  const void* a_block_scales;  /* MXFP8: f8e8m0fnu [batch, M, K/32], one per 32 elements of K of a;  */
  const void* b_block_scales;  /* f8e8m0fnu [batch, N, K/32] for b = [N,K]; both or neither; a_scale and */
  int32_t block;               /* b_scale are unused then; block must be 32                          */
  int32_t reserved0;
  int64_t batch;               /* 0 or 1: a [M,K], b [K,N]|[N,K]; B > 1: a [B,M,K], b [B,K,N]|[B,N,K],
                                  out [B,M,N], scales per tensor only; negative: empty batch */
} XlaAmdFp8ScaledDot;

XLA_AMD_EXPORT int xla_amd_launch_fp8_scaled_dot(const XlaAmdFp8ScaledDot* p, void* stream);

/* Scratch the call can use (0 = none).  A [K,N] rhs whose N is a multiple of 16 goes in as it is;
 * any other [K,N] rhs is re-laid out with K minor first (the transpose GemmRewriter inserts at
 * gemm_rewriter.cc:1235-1591), which takes K*N bytes -- without them such a rhs runs on the slow
 * exact kernel.  Up to 64 rows of a (48 with an [N,K] rhs, 32 with block scales; K and N multiples
 * of 8, resp. 16 and 8, K of 128 with block scales) stream the rhs once instead and, where the channels alone leave CUs idle, split K over workgroups:
 * slices * M * N * 4 bytes of f32 sums, per batch -- without them one slice.  More rows that go through
 * those kernels in passes (no batch, no block scales) need the sums of one pass. */
XLA_AMD_EXPORT size_t xla_amd_fp8_scaled_dot_workspace_bytes(int64_t M, int64_t K, int64_t N,
                                                             int32_t rhs_contracting_dim);

/* The same for a call whose dequantise multiply has the given type (XLA_FFI_DataType): under a BF16
 * multiply every a * a_scale and b * b_scale is rounded to bf16, and unless both scales turn out to
 * be powers of two the call runs on the bf16 matrix cores from operands a pre-pass writes into the
 * scratch ((M + N) * K * 2 bytes more); without that scratch it runs on the slow exact kernel. */
XLA_AMD_EXPORT size_t xla_amd_fp8_scaled_dot_workspace_bytes_typed(int64_t M, int64_t K, int64_t N,
                                                                   int32_t rhs_contracting_dim,
                                                                   int32_t dequant_type);

typedef struct XlaAmdRowwiseQuantize {
  const void* x;     /* bf16 [rows, cols] */
  const void* gamma; /* bf16 [cols] or NULL when rmsnorm == 0 */
  void* q;           /* f8e4m3fn [rows, cols] */
  float* scales;     /* f32 [rows] */
  int64_t rows, cols;
  float eps;
  int32_t rmsnorm;
} XlaAmdRowwiseQuantize;

XLA_AMD_EXPORT int xla_amd_launch_rowwise_quantize_fp8(const XlaAmdRowwiseQuantize* p, void* stream);

/* Message of the last failed launcher call on this thread ("" if none). */
XLA_AMD_EXPORT const char* xla_amd_last_error(void);

/* Name of the kernel variant the last successful launcher call on this thread selected
 * (e.g. "dequant_dot_decode_s4_m16"); for profiling scripts and tests. */
XLA_AMD_EXPORT const char* xla_amd_last_kernel(void);

/* Tuning hook for benchmarks and tests: overrides a kernel-selection heuristic for calls made by the
 * calling thread (value 0 restores the default); other threads are not affected.  Keys:
 * "dequant_dot_kernel" (1 generic, 2 decode, also in passes of 64 tokens, 3 tiled whenever it covers
 * the shape), "dequant_dot_vec", "dequant_dot_slices", "dequant_dot_waves", "dequant_dot_skew" (shares
 * of K of a SIMD's waves, oldest first, as decimal digits), "dequant_dot_x" (1: s4 / s8 weights stay
 * off the matrix-instruction-dequantising and the single-launch kernels), "dequant_dot_pair" (1: two
 * workgroups per 256-channel strip wherever the shape allows, 2: never), "dequant_dot_share" (the
 * first workgroup's sixteenths of K), "dequant_dot_depth" (ring depth 2 or 4), "dequant_dot_steps"
 * (steps per wave of the single-launch s8 kernel: 1, 2, 4), "dequant_dot_strip" (channels per strip of
 * that kernel: 64 or 128), "handover_test" (1: workgroups that hand partial sums over never raise their
 * flags and the waiting side gives up after 16 polls, so that its own fallback computes the result --
 * for tests of that fallback only), "dequant_dot_ragged_tile" (rows per chunk of a ragged dot's groups on the
 * decode kernels: 16, 32, 48 or 64, at most what the launcher would take), "fp8_dot_kernel" (1 exact, 2 tiled, 3 streaming), "fp8_decode_slices" (K-slices of the streaming kernels),
 * "fp8_scales_on_sum" (1: a bf16-typed dequantise multiply of xla_amd.fp8_scaled_dot is computed as the
 * reference's GPU pipeline computes that HLO -- scales on the f32 sum, gemm_rewriter.cc:1235-1591 -- not
 * op by op: no rounding of a * a_scale and b * b_scale to bf16, so scales that are no powers of two keep
 * the fp8 kernels; differs from the op-by-op value by up to the bf16 rounding of the operands),
 * "quantize_variant", "fp8_dot_layout" (1: transpose a [K,N] rhs in a pre-pass), "tiled_epilogue" (1:
 * the tiled kernels compute f32-typed GELU / SiLU from x * sigmoid(.) with the hardware exponential
 * instead of op by op as the HLO does; faster, but the far negative tail no longer matches the
 * reference's cancellation to 2 bf16 ulp), "tiled_tail" (1: the tiled dequantize-dot kernel never
 * splits the tiles of its last round along K).  Returns 0, or -1 for an unknown key. */
XLA_AMD_EXPORT int xla_amd_debug_set_option(const char* key, int value);

#ifdef __cplusplus
}
#endif
#endif /* XLA_AMD_QUANT_H_ */
