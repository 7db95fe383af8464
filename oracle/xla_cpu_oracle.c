/*
 * TEST INFRASTRUCTURE ONLY.  CPU restatement of what the XLA CPU backend
 * computes for the quantized-inference patterns (weight-only s8/s4
 * dequantize-dot, f8e4m3fn scaled dot, RMSNorm + per-row dynamic fp8
 * quantize).  Nothing in the shipped library links, loads or calls this file;
 * it exists so that the HIP kernels can be checked against an independent
 * scalar implementation, and so that a CPU figure can be timed beside them.
 *
 * Semantics restated (paths relative to the XLA source tree):
 *   - every bf16-typed op is evaluated in f32 and re-rounded to bf16 after the
 *     op (FloatNormalization): xla/service/cpu/cpu_compiler.cc:804-840,
 *     xla/service/float_support.cc:30-140
 *   - f32 -> bf16: xla/codegen/intrinsic/fptrunc.cc:64-114
 *   - f32 -> f8e4m3fn: xla/codegen/intrinsic/fptrunc.cc:275-511 and
 *     xla/service/llvm_ir/llvm_util.cc:1034-1130
 *   - f8e4m3fn -> f16 (-> f32): xla/codegen/intrinsic/fptrunc.cc:131-230
 *   - s4 storage: xla/service/llvm_ir/ir_array.cc:588-603, xla/packing.cc
 *   - tanh: xla/codegen/intrinsic/tanh.cc:33-108
 *   - exp: xla/backends/cpu/codegen/polynomial_approximations.cc:173-296
 *   - logistic(x) = 1/(1+exp(-x)): xla/hlo/transforms/expanders/logistic_expander.cc:33-46
 *   - row reductions as windows of 32, applied recursively:
 *     xla/hlo/transforms/simplifiers/tree_reduction_rewriter.cc:50-121 with
 *     window 32 from xla/service/cpu/cpu_compiler.cc:529-535
 *   - dot: f32 accumulation over k, xla/backends/cpu/runtime/dot_thunk.cc:75-229
 *     and the textbook loop xla/hlo/evaluator/hlo_evaluator_typed_visitor.h:967-1067
 *
 * Pinned by the reference's own vectors (tests/test_oracle_golden.py):
 * s4 pack/unpack, f32->bf16, f32/f16->f8e4m3fn, f8e4m3fn->f16/f32.
 * PARITY UNPINNED at bit level (only a run of the real CPU backend could pin
 * them; they live in Eigen / LLVM code generation, outside the XLA tree):
 *   - xo_dequant_dot / xo_fp8_scaled_dot: the order of the f32 additions over
 *     k (this file adds in increasing k, one rounding per multiply and per add)
 *   - xo_rmsnorm_quantize_fp8: the order of additions inside one 32-wide
 *     window of the sum of squares (this file adds left to right)
 *   - xo_tanh_f32 / xo_exp_f32 and the f32-typed GELU: which multiply-add pairs
 *     the host's LLVM contracts into fma (fusion is allowed there; this file
 *     fuses exactly the pairs written as mul_add when xo_set_fp_contract(1),
 *     none when 0; it must be compiled with -ffp-contract=off and without
 *     -ffast-math so that nothing else fuses or reorders)
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#if defined(_OPENMP)
#include <omp.h>
#endif

#define XO_API __attribute__((visibility("default")))

static inline uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

/* ------------------------------------------------------------------ casts */

/* fptrunc.cc:88-110: bias 0x7fff + lsb, NaN -> quiet NaN keeping the sign. */
XO_API uint16_t xo_f32_to_bf16(float x) {
  uint32_t u = f2u(x);
  if ((u & 0x7fffffffu) > 0x7f800000u) {
    return (uint16_t)(((u & 0xFFC00000u) | 0x00400000u) >> 16);
  }
  uint32_t lsb = (u >> 16) & 1u;
  return (uint16_t)((u + 0x7fffu + lsb) >> 16);
}

XO_API float xo_bf16_to_f32(uint16_t h) { return u2f((uint32_t)h << 16); }

/* Keep exponent range, round the significand to `mant` explicit bits, RNE
 * (llvm_util.cc EmitReducePrecisionIR, used by fptrunc.cc:395-402). */
static uint32_t reduce_mantissa_rne(uint32_t u, int mant) {
  const int drop = 23 - mant;
  uint32_t last = 1u << drop;
  uint32_t bias = ((u & last) >> drop) + (last >> 1) - 1u;
  uint32_t mask = ~(last - 1u);
  return (u + bias) & mask;
}

/* fptrunc.cc:375-509 specialised to f32 -> e4m3fn (bias 7, 3 mantissa bits,
 * no inf; overflow and inf/nan -> 0x7F with the sign kept), followed by the
 * subnormal path of llvm_util.cc:1034-1130 (round_to_even(|x| * 2^9)).
 * As written there, an input of exactly +-496.0 is not "overflow" (strict >)
 * yet rounds up to 2^9, whose shifted exponent truncates to 0x80; this
 * restatement keeps that result.  Inputs clamped to +-448 never reach it. */
XO_API uint8_t xo_f32_to_f8e4m3fn(float x) {
  const uint32_t u = f2u(x);
  const uint32_t a = u & 0x7fffffffu;
  const uint8_t sign = (uint8_t)((u >> 31) << 7);
  uint8_t bits;
  const int is_nan_in = a > 0x7f800000u;
  uint32_t r = is_nan_in ? a : (reduce_mantissa_rne(u, 3) & 0x7fffffffu);
  const uint32_t min_normal = (uint32_t)(120 + 1) << 23; /* 2^-6 */
  if (r < min_normal) r = min_normal;
  r -= (uint32_t)120 << 23;
  bits = (uint8_t)(r >> 20);
  /* largest source value that still rounds to a finite code: exponent field
   * 15+120, mantissa 111, plus half a step (fptrunc.cc:424-436). */
  const uint32_t max_repr = ((uint32_t)(15 + 120) << 23) | (7u << 20) | (1u << 19);
  const int special = (a > max_repr) || ((a & 0x7f800000u) == 0x7f800000u);
  if (special) bits = 0x7F;
  /* subnormal results: anything below 7.5 * 2^-9 */
  const float af = u2f(a);
  if (af < 7.5f * 0x1p-9f) {
    float scaled = af * 512.0f;
    bits = (uint8_t)(uint32_t)nearbyintf(scaled);
  }
  return bits | sign;
}

/* fptrunc.cc:131-230 */
XO_API uint16_t xo_f8e4m3fn_to_f16(uint8_t c) {
  static const uint16_t denorm[8] = {0x0000, 0x1800, 0x1C00, 0x1E00,
                                     0x2000, 0x2100, 0x2200, 0x2300};
  uint8_t a = c & 0x7F;
  uint16_t sign = (uint16_t)(c & 0x80) << 8;
  uint16_t e = (uint16_t)(((c & 0x78) >> 3) + 8) << 10;
  uint16_t m = (uint16_t)(c & 0x7) << 7;
  uint16_t h = e | m;
  if (a == 0x7F) h = 0x7E00;
  if (a < 8) h = denorm[a];
  return h | sign;
}

XO_API float xo_f16_to_f32(uint16_t h) {
  uint32_t sign = (uint32_t)(h & 0x8000) << 16;
  uint32_t e = (h >> 10) & 0x1F, m = h & 0x3FF;
  if (e == 0) {
    if (m == 0) return u2f(sign);
    float v = (float)m * 0x1p-24f;
    return sign ? -v : v;
  }
  if (e == 31) return u2f(sign | 0x7f800000u | (m << 13));
  return u2f(sign | ((e + 112) << 23) | (m << 13));
}

/* f32 -> f16, RNE (IEEE); needed for the f16 rows of the golden tables. */
XO_API uint16_t xo_f32_to_f16(float x) {
  uint32_t u = f2u(x), a = u & 0x7fffffffu;
  uint16_t sign = (uint16_t)((u >> 16) & 0x8000);
  if (a > 0x7f800000u) return sign | 0x7E00;
  if (a >= 0x47800000u) return sign | 0x7C00; /* >= 65536 -> inf (65520 rounds up too) */
  if (a < 0x38800000u) {                      /* below 2^-14: subnormal half */
    float v = u2f(a) * 0x1p24f;
    return sign | (uint16_t)(uint32_t)nearbyintf(v);
  }
  uint32_t r = reduce_mantissa_rne(a, 10);
  if (r >= 0x47800000u) return sign | 0x7C00;
  return sign | (uint16_t)(((r >> 23) - 112) << 10) | (uint16_t)((r >> 13) & 0x3FF);
}

XO_API float xo_f8e4m3fn_to_f32(uint8_t c) { return xo_f16_to_f32(xo_f8e4m3fn_to_f16(c)); }

/* f16 source path of the same emitter (fptrunc.cc:275-511 with fx = F16). */
XO_API uint8_t xo_f16_to_f8e4m3fn(uint16_t h) {
  /* every f16 is exact in f32 and both paths are single RNE roundings of the
   * same real number with the same overflow rule (max_repr scales with the
   * source format), so the f32 routine gives the f16 emitter's answer. */
  return xo_f32_to_f8e4m3fn(xo_f16_to_f32(h));
}

/* ir_array.cc:588-603: element i of the flat row-major index lives in byte
 * i/2, bits [4*(i%2), +4).  A trailing odd element leaves the high nibble 0. */
XO_API void xo_pack_s4(const int8_t* in, size_t n, uint8_t* out) {
  for (size_t i = 0; i < n / 2; ++i)
    out[i] = (uint8_t)((in[2 * i] & 0xF) | ((in[2 * i + 1] & 0xF) << 4));
  if (n & 1) out[n / 2] = (uint8_t)(in[n - 1] & 0xF);
}

/* ir_array.cc:618-639 + sign extension of the s4 -> s8 convert. */
XO_API void xo_unpack_s4(const uint8_t* in, size_t n, int8_t* out) {
  for (size_t i = 0; i < n; ++i) {
    uint8_t nib = (in[i / 2] >> (4 * (i & 1))) & 0xF;
    out[i] = (int8_t)((int8_t)(nib << 4) >> 4);
  }
}

/* xla/packing.cc UnpackIntN: raw nibbles, no sign extension (util_test.cc:420). */
XO_API void xo_unpack_u4(const uint8_t* in, size_t n, uint8_t* out) {
  for (size_t i = 0; i < n; ++i) out[i] = (in[i / 2] >> (4 * (i & 1))) & 0xF;
}

XO_API void xo_f32_to_bf16_n(const float* in, size_t n, uint16_t* out) {
  for (size_t i = 0; i < n; ++i) out[i] = xo_f32_to_bf16(in[i]);
}
XO_API void xo_f32_to_f8e4m3fn_n(const float* in, size_t n, uint8_t* out) {
  for (size_t i = 0; i < n; ++i) out[i] = xo_f32_to_f8e4m3fn(in[i]);
}
XO_API void xo_f8e4m3fn_to_f32_n(const uint8_t* in, size_t n, float* out) {
  for (size_t i = 0; i < n; ++i) out[i] = xo_f8e4m3fn_to_f32(in[i]);
}

/* ------------------------------------------------------- transcendental */

/* Multiply feeding an add inside one f32 kernel.  The CPU backend builds its
 * target machine with fused multiply-add allowed (cpu_aot_loader.cc:49-55,
 * used from cpu_compiler.cc:1364 and :2200: AllowFPOpFusion = Fast), so on a
 * host with an fma instruction such a pair is ONE rounding; on a host without
 * it is two.  xo_set_fp_contract(1) (the default: every x86-64 and aarch64
 * host of the last decade) gives the first, 0 the second. */
static int xo_fp_contract = 1;
XO_API void xo_set_fp_contract(int on) { xo_fp_contract = on != 0; }
XO_API int xo_get_fp_contract(void) { return xo_fp_contract; }
static inline float mul_add(float a, float b, float c) {
  if (xo_fp_contract) return fmaf(a, b, c);
  volatile float t = a * b;
  volatile float r = t + c;
  return r;
}

/* tanh.cc:48-108 then :33-46.  The emitter issues FMul then FAdd per Horner
 * step (mul_add above); the fma clamp constant is the default on x86 with FMA. */
XO_API float xo_tanh_f32(float x) {
  const float plus_clamp = 7.99881172180175781f;
  static const float num[7] = {-2.76076847742355e-16f, 2.00018790482477e-13f,
                               -8.60467152213735e-11f, 5.12229709037114e-08f,
                               1.48572235717979e-05f,  6.37261928875436e-04f,
                               4.89352455891786e-03f};
  static const float den[4] = {1.19825839466702e-06f, 1.18534705686654e-04f,
                               2.26843463243900e-03f, 4.89352518554385e-03f};
  float ax = fabsf(x);
  int use_approx = ax < 0.0004f; /* compared in double there: 0.0004 as f32 */
  float xc = x;
  if (!(xc >= -plus_clamp)) xc = -plus_clamp; /* fast max: NaN -> constant */
  if (!(xc <= plus_clamp)) xc = plus_clamp;
  if (x != x) xc = x;
  volatile float x2 = xc * xc;
  float p = num[0];
  for (int i = 1; i < 7; ++i) p = mul_add(x2, p, num[i]);
  volatile float n = xc * p;
  float q = den[0];
  for (int i = 1; i < 4; ++i) q = mul_add(x2, q, den[i]);
  float r = use_approx ? x : (n / q);
  if (ax >= 20.0f) r = copysignf(1.0f, x);
  return r;
}

/* polynomial_approximations.cc:173-296 (Cephes expf; its MulAdd is FMul then
 * FAdd, and in - C1*n is FMul then FSub: all mul_add above). */
XO_API float xo_exp_f32(float x) {
  const float C1 = 0.693359375f, C2 = -2.12194440e-4f;
  const float p0 = 1.9875691500E-4f, p1 = 1.3981999507E-3f, p2 = 8.3334519073E-3f,
              p3 = 4.1665795894E-2f, p4 = 1.6666665459E-1f, p5 = 5.0000001201E-1f;
  if (x != x) return x;
  float in = x;
  if (in < -87.8f) in = -87.8f;
  if (in > 88.8f) in = 88.8f;
  float n = floorf(mul_add(in, 1.44269504088896341f, 0.5f));
  if (n < -127.0f) n = -127.0f;
  if (n > 127.0f) n = 127.0f;
  float xr = mul_add(-C1, n, in);
  xr = mul_add(-C2, n, xr);
  float z = mul_add(xr, p0, p1);
  z = mul_add(z, xr, p2);
  z = mul_add(z, xr, p3);
  z = mul_add(z, xr, p4);
  z = mul_add(z, xr, p5);
  volatile float xx = xr * xr;
  z = mul_add(z, xx, xr);
  volatile float z1 = 1.0f + z;
  int32_t ni = (int32_t)n;
  float pow2 = u2f((uint32_t)(ni + 0x7f) << 23);
  return z1 * pow2;
}

/* a[i]*b[i] + c[i] as one elementwise kernel holds it (see mul_add). */
XO_API void xo_mul_add_f32_n(const float* a, const float* b, const float* c, size_t n, float* out) {
  for (size_t i = 0; i < n; ++i) out[i] = mul_add(a[i], b[i], c[i]);
}
XO_API void xo_tanh_f32_n(const float* in, size_t n, float* out) {
  for (size_t i = 0; i < n; ++i) out[i] = xo_tanh_f32(in[i]);
}
XO_API void xo_exp_f32_n(const float* in, size_t n, float* out) {
  for (size_t i = 0; i < n; ++i) out[i] = xo_exp_f32(in[i]);
}

/* --------------------------------------------------------------- epilogue */

enum { XO_F32 = 0, XO_BF16 = 1 };
enum { XO_EPI_NONE = 0, XO_EPI_RELU = 1, XO_EPI_GELU_TANH = 2, XO_EPI_SILU = 3 };

/* Result of an op whose HLO type is `ty`: f32 value re-rounded if bf16. */
static inline float rnd(float v, int ty) {
  return ty == XO_BF16 ? xo_bf16_to_f32(xo_f32_to_bf16(v)) : v;
}

/* One output element after the dot.  `acc` is the f32 accumulator; the dot
 * instruction has type dot_ty; bias add and activation are ops of type ep_ty
 * (a convert sits between them when the types differ); the result is finally
 * converted to bf16.  Op order of GELU follows gemm_rewriter_fp8_test.cc:1123-1141,
 * SiLU follows gemm_rewriter.cc:995-1002 after LogisticExpander. */
static inline float epilogue_value(float acc, int dot_ty, int ep_ty, int has_bias,
                                   float bias, int epi) {
  float x = rnd(acc, dot_ty);
  x = rnd(x, ep_ty); /* convert(dot) -> ep_ty; identity when equal or widening */
  if (has_bias) x = rnd(x + rnd(bias, ep_ty), ep_ty);
  switch (epi) {
    case XO_EPI_RELU:
      x = x > 0.0f ? x : (x != x ? x : 0.0f);
      break;
    case XO_EPI_GELU_TANH: {
      float c0 = rnd(0.044715f, ep_ty), c1 = rnd(0.797884583f, ep_ty);
      float m0 = rnd(x * x, ep_ty);
      float m1 = rnd(x * m0, ep_ty);
      /* f32-typed ops sit in one kernel: m1*c0 feeds only the add (mul_add);
       * bf16-typed ops round the product to bf16 in between, nothing fuses */
      float a0 = ep_ty == XO_BF16 ? rnd(x + rnd(m1 * c0, ep_ty), ep_ty) : mul_add(m1, c0, x);
      float m3 = rnd(a0 * c1, ep_ty);
      float th = rnd(xo_tanh_f32(m3), ep_ty);
      float a2 = rnd(th + 1.0f, ep_ty);
      float m4 = rnd(a2 * 0.5f, ep_ty);
      x = rnd(x * m4, ep_ty);
      break;
    }
    case XO_EPI_SILU: {
      float ng = -x;
      float ex = rnd(xo_exp_f32(ng), ep_ty);
      float dn = rnd(1.0f + ex, ep_ty);
      float sg = rnd(1.0f / dn, ep_ty);
      x = rnd(x * sg, ep_ty);
      break;
    }
    default:
      break;
  }
  return x;
}

static inline uint16_t epilogue(float acc, int dot_ty, int ep_ty, int has_bias,
                                float bias, int epi) {
  return xo_f32_to_bf16(epilogue_value(acc, dot_ty, ep_ty, has_bias, bias, epi));
}

/* The f8 result of a dot whose value v (f32-typed ops throughout) is scaled by a per-tensor
 * factor, clamped and converted: convert(clamp(-448, v / z | v * z, 448)), the tail of
 * gemm_rewriter_fp8_test.cc:1665-1690 (divide) and :1730-1748 (multiply).  Clamp is
 * min(max(x, lo), hi) with NaN passed on. */
static inline uint8_t scaled_f8_result(float v, float z, int divides) {
  volatile float t = divides ? v / z : v * z;
  float c = t;
  if (c == c) {
    if (c < -448.0f) c = -448.0f;
    if (c > 448.0f) c = 448.0f;
  }
  return xo_f32_to_f8e4m3fn(c);
}

XO_API uint16_t xo_epilogue_one(float acc, int dot_ty, int ep_ty, int has_bias,
                                float bias, int epi) {
  return epilogue(acc, dot_ty, ep_ty, has_bias, bias, epi);
}

/* ------------------------------------------------------------ dequant dot */

/*
 * out[b,m,n] = epilogue( sum_k f32(A[b,m,k]) * W'[b,k,n] ), with
 *   W'[b,k,n] = round_mul_ty( f32(w[b,k,n]) * round_mul_ty(scale[b,k/group,n]) )
 * A: bf16 [batch,M,K].  w: s8 [batch,K,N] (w_bits=8) or s4 packed low nibble
 * first over the flat row-major index (w_bits=4).  scale: [batch,K/group,N] of
 * scale_ty (group == K for per-output-channel scales).  bias: [N] of bias_ty
 * or NULL.  out: bf16 [batch,M,N].  Additions over k in increasing k, one
 * rounding per product and per sum.  Returns 0, or -1 on a bad argument.
 */
/* The same with 4-bit weights read as unsigned (w_unsigned != 0: u4, 0..15) and an optional zero
 * point per scale (zero_points: u4 [batch,K/group,N] packed like the weights, or NULL):
 *   W'[b,k,n] = round_mul_ty( round_mul_ty(f32(w) - f32(z)) * round_mul_ty(scale) )
 * -- convert, subtract, multiply, each an op of type mul_ty; the difference of two integers below
 * 16 is exact in either type. */
XO_API int xo_dequant_dot_zp(const uint16_t* A, const void* w, int w_bits, int w_unsigned,
                             const uint8_t* zero_points, const void* scale, int scale_ty, int mul_ty,
                             const void* bias, int bias_ty, int64_t batch, int64_t M,
                             int64_t K, int64_t N, int64_t group, int dot_ty,
                             int ep_ty, int epi, uint16_t* out);

XO_API int xo_dequant_dot(const uint16_t* A, const void* w, int w_bits,
                          const void* scale, int scale_ty, int mul_ty,
                          const void* bias, int bias_ty, int64_t batch, int64_t M,
                          int64_t K, int64_t N, int64_t group, int dot_ty,
                          int ep_ty, int epi, uint16_t* out) {
  return xo_dequant_dot_zp(A, w, w_bits, 0, NULL, scale, scale_ty, mul_ty, bias, bias_ty, batch, M, K, N,
                           group, dot_ty, ep_ty, epi, out);
}

/* out32, when given, receives the value before the final convert to bf16: the result of a module
 * whose root is the f32 dot (or f32-typed epilogue op) itself, as in
 * fusion_emitter_int4_device_test.cc:101,205,320,508; out may then be NULL. */
static int dequant_dot_impl(const uint16_t* A, const void* w, int w_bits, int w_unsigned,
                            const uint8_t* zero_points, const void* scale, int scale_ty, int mul_ty,
                            const void* bias, int bias_ty, int64_t batch, int64_t M,
                            int64_t K, int64_t N, int64_t group, int dot_ty,
                            int ep_ty, int epi, uint16_t* out, float* out32) {
  if (!(w_bits == 8 || w_bits == 4) || group <= 0 || K % group != 0) return -1;
  if ((w_unsigned || zero_points) && w_bits != 4) return -1;
  const int64_t G = K / group;
  int rc = 0;
#pragma omp parallel
  {
    float* col = (float*)malloc(sizeof(float) * (size_t)K);
    float* accs = (float*)malloc(sizeof(float) * (size_t)M);
    if (!col || !accs) rc = -1;
#pragma omp for collapse(2) schedule(static)
    for (int64_t b = 0; b < batch; ++b) {
      for (int64_t n = 0; n < N; ++n) {
        if (rc) continue;
        /* materialise the dequantised column once (the CPU backend
         * materialises the whole dequantised tensor before the dot). */
        for (int64_t k = 0; k < K; ++k) {
          size_t idx = ((size_t)b * K + k) * N + n;
          int wi;
          if (w_bits == 8) {
            wi = ((const int8_t*)w)[idx];
          } else {
            uint8_t nib = (((const uint8_t*)w)[idx >> 1] >> (4 * (idx & 1))) & 0xF;
            wi = w_unsigned ? (int)nib : (int8_t)(nib << 4) >> 4;
          }
          size_t sidx = ((size_t)b * G + k / group) * N + n;
          float s = scale_ty == XO_BF16 ? xo_bf16_to_f32(((const uint16_t*)scale)[sidx])
                                        : ((const float*)scale)[sidx];
          s = rnd(s, mul_ty);
          float wf = rnd((float)wi, mul_ty);
          if (zero_points) {
            float zf = rnd((float)((zero_points[sidx >> 1] >> (4 * (sidx & 1))) & 0xF), mul_ty);
            volatile float d = wf - zf;
            wf = rnd(d, mul_ty);
          }
          float prod = wf * s;
          col[k] = rnd(prod, mul_ty);
        }
        for (int64_t m = 0; m < M; ++m) {
          const uint16_t* a = A + ((size_t)b * M + m) * K;
          float acc = 0.0f;
          for (int64_t k = 0; k < K; ++k) {
            float p = xo_bf16_to_f32(a[k]) * col[k];
            acc = acc + p;
          }
          accs[m] = acc;
        }
        float bv = 0.0f;
        if (bias)
          bv = bias_ty == XO_BF16 ? xo_bf16_to_f32(((const uint16_t*)bias)[n])
                                  : ((const float*)bias)[n];
        for (int64_t m = 0; m < M; ++m) {
          const float v = epilogue_value(accs[m], dot_ty, ep_ty, bias != NULL, bv, epi);
          if (out) out[((size_t)b * M + m) * N + n] = xo_f32_to_bf16(v);
          if (out32) out32[((size_t)b * M + m) * N + n] = v;
        }
      }
    }
    free(col);
    free(accs);
  }
  return rc;
}

XO_API int xo_dequant_dot_zp(const uint16_t* A, const void* w, int w_bits, int w_unsigned,
                             const uint8_t* zero_points, const void* scale, int scale_ty, int mul_ty,
                             const void* bias, int bias_ty, int64_t batch, int64_t M,
                             int64_t K, int64_t N, int64_t group, int dot_ty,
                             int ep_ty, int epi, uint16_t* out) {
  return dequant_dot_impl(A, w, w_bits, w_unsigned, zero_points, scale, scale_ty, mul_ty, bias, bias_ty, batch, M,
                          K, N, group, dot_ty, ep_ty, epi, out, NULL);
}

XO_API int xo_dequant_dot_f32(const uint16_t* A, const void* w, int w_bits, int w_unsigned,
                              const uint8_t* zero_points, const void* scale, int scale_ty, int mul_ty,
                              const void* bias, int bias_ty, int64_t batch, int64_t M,
                              int64_t K, int64_t N, int64_t group, int dot_ty,
                              int ep_ty, int epi, float* out32) {
  return dequant_dot_impl(A, w, w_bits, w_unsigned, zero_points, scale, scale_ty, mul_ty, bias, bias_ty, batch, M,
                          K, N, group, dot_ty, ep_ty, epi, NULL, out32);
}

/* --------------------------------------------------------- fp8 scaled dot */

/*
 * out[m,n] = epilogue( sum_k A'[m,k] * B'[k,n] ),
 *   A'[m,k] = round_mul_ty(f32(A8[m,k]) * round_mul_ty(sa_m)), B'[k,n] likewise with sb_n.
 * A8: f8e4m3fn [M,K] row-major.  B8: f8e4m3fn, [K,N] row-major when
 * b_is_nk == 0, or [N,K] row-major (contracting dimension minor) when 1.
 * a_scale points at one value (a_rows == 0: the per-tensor scale of
 * gemm_rewriter_fp8_test.cc:1099-1135) or at M values (a_rows != 0: one per
 * row of A, the broadcast along dimension 0 that a row-wise quantizer's
 * scales are applied with); b_scale at one value or, with b_cols != 0, at N
 * values, one per output channel.  With out8 the result is f8e4m3fn after a
 * per-tensor scaling by *d_scale (see scaled_f8_result); out_value, if given,
 * receives the f32 value before that scaling, for tolerance checks.
 */
XO_API int xo_fp8_scaled_dot(const uint8_t* A8, const uint8_t* B8, int b_is_nk,
                             const float* a_scale, int a_rows, const float* b_scale,
                             int b_cols, int mul_ty, const void* bias, int bias_ty,
                             int64_t M, int64_t K, int64_t N, int dot_ty, int ep_ty,
                             int epi, uint16_t* out, const float* d_scale, int d_divides,
                             uint8_t* out8, float* out_value) {
  float f8v[256];
  for (int c = 0; c < 256; ++c) f8v[c] = xo_f8e4m3fn_to_f32((uint8_t)c);
  /* the dequantised A once: M*K floats */
  float* Ad = (float*)malloc(sizeof(float) * (size_t)(M > 0 ? M : 1) * (size_t)(K > 0 ? K : 1));
  if (!Ad) return -1;
  for (int64_t m = 0; m < M; ++m) {
    float sa = rnd(a_scale[a_rows ? m : 0], mul_ty);
    for (int64_t k = 0; k < K; ++k) {
      volatile float pa = f8v[A8[(size_t)m * K + k]] * sa;
      Ad[(size_t)m * K + k] = rnd(pa, mul_ty);
    }
  }
  int rc = 0;
#pragma omp parallel
  {
    float* col = (float*)malloc(sizeof(float) * (size_t)(K > 0 ? K : 1));
    if (!col) rc = -1;
#pragma omp for schedule(static)
    for (int64_t n = 0; n < N; ++n) {
      if (rc) continue;
      float sb = rnd(b_scale[b_cols ? n : 0], mul_ty);
      for (int64_t k = 0; k < K; ++k) {
        volatile float pb = f8v[b_is_nk ? B8[(size_t)n * K + k] : B8[(size_t)k * N + n]] * sb;
        col[k] = rnd(pb, mul_ty);
      }
      float bv = 0.0f;
      if (bias)
        bv = bias_ty == XO_BF16 ? xo_bf16_to_f32(((const uint16_t*)bias)[n])
                                : ((const float*)bias)[n];
      for (int64_t m = 0; m < M; ++m) {
        const float* a = Ad + (size_t)m * K;
        float acc = 0.0f;
        for (int64_t k = 0; k < K; ++k) {
          float p = a[k] * col[k];
          acc = acc + p;
        }
        if (out8) { /* f8 result: f32-typed ops, then scale, clamp, convert */
          float v = epilogue_value(acc, dot_ty, ep_ty, bias != NULL, bv, epi);
          if (out_value) out_value[(size_t)m * N + n] = v;
          out8[(size_t)m * N + n] = scaled_f8_result(v, *d_scale, d_divides);
        } else {
          out[(size_t)m * N + n] = epilogue(acc, dot_ty, ep_ty, bias != NULL, bv, epi);
        }
      }
    }
    free(col);
  }
  free(Ad);
  return rc;
}

/* -------------------------------------------------- block-scaled (MX) dot */

/* f8e8m0fnu -> f32: 2^(e-127); 0xFF is NaN; there is no zero and no sign
 * (convert_test.cc:2114-2140: 1.0 <-> 127, 2^127 <-> 254, 2^-126 <-> 1). */
XO_API float xo_f8e8m0fnu_to_f32(uint8_t e) {
  if (e == 0xFF) return u2f(0x7fc00000u);
  if (e == 0) return u2f(0x00400000u); /* 2^-127, a subnormal f32 */
  return u2f((uint32_t)e << 23);
}

/*
 * "__op$block_scaled_dot" as BlockScalingRewriter expands it when no library
 * kernel applies (block_scaling_rewriter.cc:194-219, :521-571): each operand
 * is converted to the result type and multiplied by its scale, one scale per
 * `block` consecutive elements of the contracting (minor) dimension, then the
 * two are contracted.  A8: f8e4m3fn [M,K]; B8: f8e4m3fn [N,K]; a_sc: f8e8m0fnu
 * [M,K/block]; b_sc: [N,K/block].  The scales are powers of two and an f8 value
 * has a 4-bit significand, so the multiplies are exact in f32 and in bf16
 * alike; the dot adds in f32 and the epilogue rounds as for the other dots.
 */
XO_API int xo_block_scaled_dot(const uint8_t* A8, const uint8_t* B8, const uint8_t* a_sc,
                               const uint8_t* b_sc, int64_t block, const void* bias, int bias_ty,
                               int64_t M, int64_t K, int64_t N, int dot_ty, int ep_ty, int epi,
                               uint16_t* out) {
  if (block <= 0 || K % block) return -2;
  const int64_t nb = K / block;
  float* Ad = (float*)malloc(sizeof(float) * (size_t)(M > 0 ? M : 1) * (size_t)(K > 0 ? K : 1));
  if (!Ad) return -1;
  for (int64_t m = 0; m < M; ++m)
    for (int64_t k = 0; k < K; ++k) {
      volatile float p = xo_f8e4m3fn_to_f32(A8[(size_t)m * K + k]) * xo_f8e8m0fnu_to_f32(a_sc[(size_t)m * nb + k / block]);
      Ad[(size_t)m * K + k] = p;
    }
  int rc = 0;
#pragma omp parallel
  {
    float* col = (float*)malloc(sizeof(float) * (size_t)(K > 0 ? K : 1));
    if (!col) rc = -1;
#pragma omp for schedule(static)
    for (int64_t n = 0; n < N; ++n) {
      if (rc) continue;
      for (int64_t k = 0; k < K; ++k) {
        volatile float p = xo_f8e4m3fn_to_f32(B8[(size_t)n * K + k]) * xo_f8e8m0fnu_to_f32(b_sc[(size_t)n * nb + k / block]);
        col[k] = p;
      }
      float bv = 0.0f;
      if (bias)
        bv = bias_ty == XO_BF16 ? xo_bf16_to_f32(((const uint16_t*)bias)[n]) : ((const float*)bias)[n];
      for (int64_t m = 0; m < M; ++m) {
        const float* a = Ad + (size_t)m * K;
        float acc = 0.0f;
        for (int64_t k = 0; k < K; ++k) {
          float p = a[k] * col[k];
          acc = acc + p;
        }
        out[(size_t)m * N + n] = epilogue(acc, dot_ty, ep_ty, bias != NULL, bv, epi);
      }
    }
    free(col);
  }
  free(Ad);
  return rc;
}

/* ------------------------------------------------- RMSNorm + fp8 quantize */

/* Sum of n values as TreeReductionRewriter(32) shapes it: windows of 32
 * (last one short), each added left to right, repeated until one value is
 * left.  buf is clobbered. */
static float tree32_sum(float* buf, int64_t n) {
  while (n > 1) {
    int64_t m = (n + 31) / 32;
    for (int64_t w = 0; w < m; ++w) {
      int64_t lo = w * 32, hi = lo + 32 < n ? lo + 32 : n;
      float s = 0.0f;
      for (int64_t i = lo; i < hi; ++i) s = s + buf[i];
      buf[w] = s;
    }
    n = m;
  }
  return n == 1 ? buf[0] : 0.0f;
}

XO_API float xo_tree32_sum(const float* v, int64_t n) {
  float* b = (float*)malloc(sizeof(float) * (size_t)(n > 0 ? n : 1));
  memcpy(b, v, sizeof(float) * (size_t)n);
  float r = tree32_sum(b, n);
  free(b);
  return r;
}

/*
 * Per row r of x (bf16 [rows, cols]):
 *   xf   = f32(x)
 *   ms   = tree32_sum(xf*xf) / cols          (f32 divide)
 *   rinv = 1 / sqrt(ms + eps)                (IEEE sqrt and divide)
 *   y    = bf16( (xf * rinv) * f32(gamma) )  (two f32 multiplies, one rounding)
 *   amax = max |y|                           (exact)
 *   s    = amax / 448                        (f32 divide)
 *   q    = f8e4m3fn( clamp(-448, f32(y) / s, 448) )
 * q: [rows, cols] codes, scales: f32 [rows].  A row of zeros gives s = 0 and
 * 0/0 = NaN, which clamp propagates and the cast turns into 0x7F, exactly as
 * the unguarded HLO does.
 */
XO_API int xo_rmsnorm_quantize_fp8(const uint16_t* x, const uint16_t* gamma,
                                   float eps, int64_t rows, int64_t cols,
                                   uint8_t* q, float* scales) {
  int rc = 0;
#pragma omp parallel
  {
    float* sq = (float*)malloc(sizeof(float) * (size_t)cols);
    float* y = (float*)malloc(sizeof(float) * (size_t)cols);
    if (!sq || !y) rc = -1;
#pragma omp for schedule(static)
    for (int64_t r = 0; r < rows; ++r) {
      if (rc) continue;
      const uint16_t* xr = x + (size_t)r * cols;
      for (int64_t c = 0; c < cols; ++c) {
        float v = xo_bf16_to_f32(xr[c]);
        float p = v * v;
        sq[c] = p;
      }
      float ssum = tree32_sum(sq, cols);
      volatile float ms = ssum / (float)cols;
      volatile float me = ms + eps;
      volatile float rt = sqrtf(me);
      volatile float rinv = 1.0f / rt;
      float amax = 0.0f;
      for (int64_t c = 0; c < cols; ++c) {
        float t = xo_bf16_to_f32(xr[c]) * rinv;
        float u = t * xo_bf16_to_f32(gamma[c]);
        float yy = xo_bf16_to_f32(xo_f32_to_bf16(u));
        y[c] = yy;
        float ay = fabsf(yy);
        if (ay > amax || ay != ay) amax = ay;
      }
      volatile float s = amax / 448.0f;
      scales[r] = s;
      for (int64_t c = 0; c < cols; ++c) {
        float d = y[c] / s;
        float v = d;
        if (v == v) { if (v < -448.0f) v = -448.0f; if (v > 448.0f) v = 448.0f; }
        q[(size_t)r * cols + c] = xo_f32_to_f8e4m3fn(v);
      }
    }
    free(sq);
    free(y);
  }
  return rc;
}

XO_API int xo_num_threads(void) {
#if defined(_OPENMP)
  return omp_get_max_threads();
#else
  return 1;
#endif
}
