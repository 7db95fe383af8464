// Device-side element-type helpers shared by the gfx950 kernels.
//
// The library is compiled with -ffp-contract=off: every `a * b + c` written
// below is two roundings, and a fused multiply-add appears only where
// __builtin_fmaf is spelled out.  Casts follow the XLA CPU backend's
// definitions: f32 -> bf16 is round-to-nearest-even with quiet NaNs
// (xla/codegen/intrinsic/fptrunc.cc:64-114), f32 -> f8e4m3fn is
// round-to-nearest-even with overflow to NaN (fptrunc.cc:275-511).
#ifndef XLA_AMD_CSRC_DEVICE_NUMERICS_H_
#define XLA_AMD_CSRC_DEVICE_NUMERICS_H_

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

namespace xla_amd {

typedef float floatx2 __attribute__((ext_vector_type(2)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef int intx8 __attribute__((ext_vector_type(8)));
typedef uint32_t uintx2 __attribute__((ext_vector_type(2)));
typedef uint32_t uintx4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ float bits_to_f32(uint32_t u) { return __builtin_bit_cast(float, u); }
__device__ __forceinline__ uint32_t f32_to_bits(float f) { return __builtin_bit_cast(uint32_t, f); }

// bf16 pair packed in one dword -> two f32 (exact)
__device__ __forceinline__ float bf16lo_to_f32(uint32_t w) { return bits_to_f32(w << 16); }
__device__ __forceinline__ float bf16hi_to_f32(uint32_t w) { return bits_to_f32(w & 0xffff0000u); }
__device__ __forceinline__ float bf16_to_f32(uint16_t h) { return bits_to_f32((uint32_t)h << 16); }

// two f32 -> packed bf16 pair, RNE, NaN -> quiet NaN with the sign kept: one v_cvt_pk_bf16_f32
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  floatx2 v = {lo, hi};
  bf16x2 b = __builtin_convertvector(v, bf16x2);
  return __builtin_bit_cast(uint32_t, b);
}
__device__ __forceinline__ uint16_t f32_to_bf16(float x) { return (uint16_t)(pack_bf16x2(x, 0.0f) & 0xffffu); }
// value of an f32 after a bf16-typed HLO op re-rounds it
__device__ __forceinline__ float round_bf16(float x) { return bf16lo_to_f32(pack_bf16x2(x, 0.0f)); }

// f8e4m3fn code -> f32 (exact; 0x7F/0xFF -> NaN), pure integer/f32 arithmetic
__device__ __forceinline__ float f8e4m3fn_to_f32(uint32_t c) {
  uint32_t mag = c & 0x7fu;
  // normal codes: move exponent+mantissa to the f32 fields and re-bias by 127-7;
  // subnormal codes (mag < 8) are mag * 2^-9.
  float v = mag < 8u ? (float)mag * 0x1p-9f : bits_to_f32((mag << 20) + (120u << 23));
  if (mag == 0x7fu) v = bits_to_f32(0x7fc00000u);
  return bits_to_f32(f32_to_bits(v) | ((c & 0x80u) << 24));
}

// Software f32 -> f8e4m3fn, all inputs (slow path; the hot loops use the
// hardware convert on values already clamped to +-448).
__device__ __forceinline__ uint32_t f32_to_f8e4m3fn_any(float x) {
  uint32_t u = f32_to_bits(x), a = u & 0x7fffffffu, sign = (u >> 24) & 0x80u;
  uint32_t code;
  if (a > 0x43e80000u) {  // |x| > 464 (0x43e80000), inf, NaN
    code = 0x7fu;
  } else if (a < 0x3c800000u) {  // below 2^-6: subnormal grid of 2^-9, ties to even
    code = (uint32_t)__builtin_rintf(bits_to_f32(a) * 512.0f);
  } else {
    uint32_t r = a + 0x7ffffu + ((a >> 20) & 1u);  // RNE at 3 mantissa bits
    code = (r >> 20) - (120u << 3);
  }
  return code | sign;
}

// 4 f32 (clamped to +-448, not NaN) -> 4 f8e4m3fn codes in one dword; gfx950's
// v_cvt_pk_fp8_f32 is OCP e4m3fn with round-to-nearest-even.
__device__ __forceinline__ uint32_t pack_f8x4(float a, float b, float c, float d) {
  int r = __builtin_amdgcn_cvt_pk_fp8_f32(a, b, 0, false);
  r = __builtin_amdgcn_cvt_pk_fp8_f32(c, d, r, true);
  return (uint32_t)r;
}

// y / s, correctly rounded, from the correctly rounded reciprocal rs = RN(1/s):
// q0 = RN(y*rs); r = y - q0*s exactly (fma); q1 = RN(q0 + r*rs).  With rs
// correctly rounded and no overflow/underflow in range this is RN(y/s)
// (Markstein); the caller takes the plain IEEE divide when ordinary_divisor(s) is false.
__device__ __forceinline__ float div_by_ordinary(float y, float s, float rs) {
  float q0 = y * rs;
  float r = __builtin_fmaf(-q0, s, y);
  // s > 0 here, so the quotient carries the sign of y even when it is zero (-0/s = -0, which the
  // correction step would turn into +0)
  return __builtin_copysignf(__builtin_fmaf(r, rs, q0), y);
}

// A positive divisor shared by many quotients for which div_by_ordinary is exact: a normal
// number well inside the exponent range whose significand is not all ones.
__device__ __forceinline__ bool ordinary_divisor(float s) {
  const uint32_t sb = f32_to_bits(s);
  return sb > 0x0d800000u && sb < 0x71800000u && (sb & 0x7fffffu) != 0x7fffffu;
}

// n / d for tanh_xla's numerator and denominator only: the reciprocal refined once and the quotient
// corrected once -- the f32 division as this target expands it, minus the operand scaling, the
// special-case fix-up (d is a normal number in [4.89e-3, 0.95], |n| <= 0.95) and the second
// correction.  That this equals the IEEE quotient for every pair tanh_xla can produce is not argued
// but checked: a self-check kernel compares both tanh spellings on all 2^32 inputs.
__device__ __forceinline__ float div_well_scaled(float n, float d) {
  float r = __builtin_amdgcn_rcpf(d);
  r = __builtin_fmaf(__builtin_fmaf(-d, r, 1.0f), r, r);
  const float q0 = n * r;
  return __builtin_fmaf(__builtin_fmaf(-d, q0, n), r, q0);
}

// The reference's CPU backend compiles every kernel with fused multiply-add allowed
// (xla/service/cpu/cpu_aot_loader.cc:49-55 and cpu_compiler.cc:1364: AllowFPOpFusion = Fast), so a
// multiply feeding an add inside these f32 polynomials contracts to one fma on any host that has
// the instruction.  The fused spelling is used here: one instruction per Horner step.
//
// xla/codegen/intrinsic/tanh.cc:48-108 rational, then the |x| >= 20 -> +-1 rule of :33-46.
// NaN in -> unspecified finite value out (the caller restores it): tanh_xla below is the full op.
__device__ __forceinline__ float tanh_xla_nan_unspecified(float x) {
  const float kClamp = 7.99881172180175781f;
  float ax = __builtin_fabsf(x);
  float xc = __builtin_fminf(__builtin_fmaxf(x, -kClamp), kClamp);
  float x2 = xc * xc;
  float p = -2.76076847742355e-16f;
  p = __builtin_fmaf(x2, p, 2.00018790482477e-13f);
  p = __builtin_fmaf(x2, p, -8.60467152213735e-11f);
  p = __builtin_fmaf(x2, p, 5.12229709037114e-08f);
  p = __builtin_fmaf(x2, p, 1.48572235717979e-05f);
  p = __builtin_fmaf(x2, p, 6.37261928875436e-04f);
  p = __builtin_fmaf(x2, p, 4.89352455891786e-03f);
  p = xc * p;
  float q = 1.19825839466702e-06f;
  q = __builtin_fmaf(x2, q, 1.18534705686654e-04f);
  q = __builtin_fmaf(x2, q, 2.26843463243900e-03f);
  q = __builtin_fmaf(x2, q, 4.89352518554385e-03f);
  // q is in [4.89e-3, 0.95] and |p| <= 0.95; below |x| = 4e-4 (|p| < 2e-6) the quotient is not used
  float r = ax < 0.0004f ? x : div_well_scaled(p, q);
  // The |x| >= 20 -> copysign(1, x) rule of tanh.cc:33-46 changes nothing here: the clamp was chosen
  // (tanh.cc:54-59) so that the fused rational is exactly +-1 at +-kClamp, which is where every
  // larger |x| lands.
  return r;
}

// A NaN comes out of the fmax/fmin clamp as -kClamp (the reference's select-based clamp keeps it,
// llvm_util.cc EmitFloatMax with fast min/max), so it is put back.
__device__ __forceinline__ float tanh_xla(float x) {
  const float r = tanh_xla_nan_unspecified(x);
  return x != x ? x : r;
}

// xla/backends/cpu/codegen/polynomial_approximations.cc:173-296 (Cephes expf)
__device__ __forceinline__ float exp_xla(float x) {
  float in = __builtin_fminf(__builtin_fmaxf(x, -87.8f), 88.8f);
  float n = __builtin_floorf(__builtin_fmaf(in, 1.44269504088896341f, 0.5f));
  n = __builtin_fminf(__builtin_fmaxf(n, -127.0f), 127.0f);
  float r = __builtin_fmaf(-0.693359375f, n, in);
  r = __builtin_fmaf(2.12194440e-4f, n, r);
  float z = __builtin_fmaf(r, 1.9875691500E-4f, 1.3981999507E-3f);
  z = __builtin_fmaf(z, r, 8.3334519073E-3f);
  z = __builtin_fmaf(z, r, 4.1665795894E-2f);
  z = __builtin_fmaf(z, r, 1.6666665459E-1f);
  z = __builtin_fmaf(z, r, 5.0000001201E-1f);
  z = __builtin_fmaf(z, r * r, r);
  z = 1.0f + z;
  float p2 = bits_to_f32((uint32_t)((int)n + 0x7f) << 23);
  float res = z * p2;
  return x != x ? x : res;
}

enum : int { kEpiDefault = 0, kEpiBias = 1, kEpiRelu = 2, kEpiBiasRelu = 3, kEpiGelu = 4,
             kEpiBiasGelu = 5, kEpiSilu = 6, kEpiBiasSilu = 7 };

// What follows the dot in the matched HLO, op by op.  BF16_DOT: the dot
// instruction is bf16-typed (accumulator rounded first).  BF16_OPS: bias add
// and activation ops are bf16-typed, each result re-rounded (what
// FloatNormalization makes of them, xla/service/cpu/cpu_compiler.cc:804-817);
// otherwise they run in f32 and only the final convert rounds.  GELU op order:
// gemm_rewriter_fp8_test.cc:1123-1141; SiLU: gemm_rewriter.cc:995-1002.
// The dot result as the epilogue sees it: rounded to the dot's type, then (optionally) the
// bias add in the epilogue's type.
template <bool BF16_DOT, bool BF16_OPS>
__device__ __forceinline__ float epilogue_pre(float acc, float bias, bool has_bias) {
  auto R = [](float v) { return BF16_OPS ? round_bf16(v) : v; };
  float x = BF16_DOT ? round_bf16(acc) : acc;
  x = R(x);
  const float xb = R(x + R(bias));
  return has_bias ? xb : x;
}

// The activation, every op rounded to the epilogue's type.  `act` is one of 0, kEpiRelu,
// kEpiGelu, kEpiSilu (2, 4, 6).
template <bool BF16_OPS>
__device__ __forceinline__ float epilogue_act(float x, int act) {
  auto R = [](float v) { return BF16_OPS ? round_bf16(v) : v; };
  switch (act) {
    case 2:  // relu; NaN passes through
      x = x > 0.0f ? x : (x != x ? x : 0.0f);
      break;
    case 4: {  // tanh-approximated gelu
      float m0 = R(x * x);
      float m1 = R(x * m0);
      // f32-typed ops: the multiply by 0.044715 feeds only the add, which contracts like the
      // polynomial steps above; bf16-typed ops round the product first, so nothing fuses
      float a0 = BF16_OPS ? R(x + R(m1 * R(0.044715f))) : __builtin_fmaf(m1, 0.044715f, x);
      float m3 = R(a0 * R(0.797884583f));
      float th = R(tanh_xla_nan_unspecified(m3));  // x * m4 below turns a NaN x back into NaN
      // (th + 1) * 0.5: the halving is exact, so for f32 ops one fma gives the same bits
      float m4 = BF16_OPS ? R(R(th + 1.0f) * 0.5f) : __builtin_fmaf(th, 0.5f, 0.5f);
      x = R(x * m4);
      break;
    }
    case 6: {  // silu
      float ex = R(exp_xla(-x));
      float dn = R(1.0f + ex);
      float sg = R(1.0f / dn);
      x = R(x * sg);
      break;
    }
    default:
      break;
  }
  return x;
}

// The same activations for f32-typed ops, straight from their closed forms with the hardware
// exponential and reciprocal: gelu_tanh(x) = x * sigmoid(2 * 0.797884583 * (x + 0.044715 x^3)),
// silu(x) = x * sigmoid(x), sigmoid(t) = 1 / (1 + 2^(-t * log2 e)).  About 8 instructions instead
// of 35 (no rational tanh, no IEEE divide), 9 % of the 8192^3 f8 dot with GELU.  Opt-in only: it is
// accurate to ~1e-6 of the true function, but the HLO's own sequence is not -- for x below about
// -4.5 its 0.5 * (1 + tanh) cancels down to a few f32 ulps of 1 (and to exactly 0 past the tanh
// clamp), so there this form and the reference disagree by more than 2 bf16 ulp of a result that
// is itself below 1e-5.
__device__ __forceinline__ float epilogue_act_direct(float x, int act) {
  switch (act) {
    case 2:
      return x > 0.0f ? x : (x != x ? x : 0.0f);
    case 4: {
      const float w = x * __builtin_fmaf(x * x, 0.044715f, 1.0f);
      const float e = __builtin_amdgcn_exp2f(w * (-2.0f * 0.797884583f * 1.44269504088896341f));
      return x * __builtin_amdgcn_rcpf(1.0f + e);
    }
    case 6: {
      const float e = __builtin_amdgcn_exp2f(x * -1.44269504088896341f);
      return x * __builtin_amdgcn_rcpf(1.0f + e);
    }
    default:
      return x;
  }
}

template <bool BF16_DOT, bool BF16_OPS>
__device__ __forceinline__ float epilogue_value(float acc, float bias, int epi) {
  return epilogue_act<BF16_OPS>(epilogue_pre<BF16_DOT, BF16_OPS>(acc, bias, (epi & 1) != 0), epi & ~1);
}

__device__ __forceinline__ float epilogue_dispatch(float acc, float bias, int epi, bool bf16_dot,
                                                   bool bf16_ops) {
  if (bf16_ops) {
    return bf16_dot ? epilogue_value<true, true>(acc, bias, epi)
                    : epilogue_value<false, true>(acc, bias, epi);
  }
  return bf16_dot ? epilogue_value<true, false>(acc, bias, epi)
                  : epilogue_value<false, false>(acc, bias, epi);
}

// COUNT values through one epilogue, chosen once: straight-line code for the one variant that
// runs, instead of a COUNT-fold copy of the whole dispatch.
template <bool BF16_DOT, bool BF16_OPS, int ACT, int COUNT>
__device__ __forceinline__ void epilogue_all(float* v, const float* bias, bool has_bias) {
#pragma unroll
  for (int i = 0; i < COUNT; ++i)
    v[i] = epilogue_act<BF16_OPS>(epilogue_pre<BF16_DOT, BF16_OPS>(v[i], bias[i], has_bias), ACT);
}

template <bool BF16_DOT, bool BF16_OPS, int COUNT>
__device__ __forceinline__ void epilogue_all_act(float* v, const float* bias, int epi) {
  const bool has_bias = (epi & 1) != 0;
  switch (epi & ~1) {
    case kEpiRelu: epilogue_all<BF16_DOT, BF16_OPS, kEpiRelu, COUNT>(v, bias, has_bias); break;
    case kEpiGelu: epilogue_all<BF16_DOT, BF16_OPS, kEpiGelu, COUNT>(v, bias, has_bias); break;
    case kEpiSilu: epilogue_all<BF16_DOT, BF16_OPS, kEpiSilu, COUNT>(v, bias, has_bias); break;
    default: epilogue_all<BF16_DOT, BF16_OPS, 0, COUNT>(v, bias, has_bias); break;
  }
}

template <int COUNT>
__device__ __forceinline__ void epilogue_all_dispatch(float* v, const float* bias, int epi, bool bf16_dot,
                                                      bool bf16_ops) {
  if (bf16_ops) {
    if (bf16_dot) epilogue_all_act<true, true, COUNT>(v, bias, epi);
    else epilogue_all_act<false, true, COUNT>(v, bias, epi);
  } else {
    if (bf16_dot) epilogue_all_act<true, false, COUNT>(v, bias, epi);
    else epilogue_all_act<false, false, COUNT>(v, bias, epi);
  }
}

// A normal power of two whose product with any finite f8e4m3fn value stays a normal bf16: scaling by it
// is exact, so a bf16-typed dequantise multiply rounds nothing.
__device__ __forceinline__ bool is_pow2_f32(float s) {
  const uint32_t u = f32_to_bits(s);
  const uint32_t e = (u >> 23) & 0xffu;
  return (u & 0x807fffffu) == 0u && e > 24u && e < 230u;
}

// f(std::integral_constant<int, I>) for I = 0 .. N-1, expanded at compile time: unlike a loop under
// `#pragma unroll`, which the compiler may decline for a large body, the index is a constant in
// every copy, so arrays indexed by it stay in registers.
template <int I, int N, class F>
__device__ __forceinline__ void static_for(F&& f) {
  if constexpr (I < N) {
    f(std::integral_constant<int, I>{});
    static_for<I + 1, N>(f);
  }
}

}  // namespace xla_amd
#endif  // XLA_AMD_CSRC_DEVICE_NUMERICS_H_
