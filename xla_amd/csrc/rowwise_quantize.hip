// Row-wise dynamic quantisation to f8e4m3fn, optionally preceded by RMSNorm,
// in one pass over the activation: one workgroup owns one row, keeps it in
// registers, and reads it from HBM exactly once.
//
//   xf   = f32(x)                                   x: bf16 [rows, cols]
//   ms   = sum(xf*xf) / cols ; rinv = 1 / sqrt(ms + eps)
//   y    = bf16((xf * rinv) * f32(gamma))           (y = x without RMSNorm)
//   amax = max |y| ; s = amax / 448
//   q    = f8e4m3fn(clamp(-448, y / s, 448))        q: [rows, cols], s: f32 [rows]
//
// The sum of squares is added in the order XLA's TreeReductionRewriter(32)
// gives it on the CPU backend (xla/hlo/transforms/simplifiers/tree_reduction_rewriter.cc:50-121,
// window from xla/service/cpu/cpu_compiler.cc:529-535): windows of 32
// consecutive elements added left to right, then windows of 32 of those sums,
// and so on.  Every other step is order-free or a single IEEE operation, so
// the output codes and scales are reproducible bit for bit.
//
// Bound: HBM.  Algorithmic bytes per row: cols*2 (x) + cols (q) + 4 (s); gamma
// (cols*2) is read once per row but stays in L2.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "device_numerics.h"
#include "launch.h"

namespace xla_amd {
namespace {

constexpr int kThreads = 256;

// res of lane-1 in the same row of 16 lanes (lanes 4i..4i+3 never straddle a row)
__device__ __forceinline__ float lane_shr1(float v) {
  return __builtin_bit_cast(
      float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x111 /*row_shr:1*/, 0xf,
                                         0xf, true));
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = __builtin_fmaxf(v, __shfl_xor(v, off));
  return v;
}

// CH: consecutive 8-element chunks owned by a lane inside one group;
// G: groups.  A group spans kThreads*CH*8 consecutive elements.  VEC: rows are
// 16-byte aligned and cols % 8 == 0, so chunks move as 128-bit accesses.
template <int CH, int G, bool VEC>
__global__ __launch_bounds__(kThreads) void rowwise_quantize_kernel(
    const uint16_t* __restrict__ x, const uint16_t* __restrict__ gamma, uint8_t* __restrict__ q,
    float* __restrict__ scales, int rows, int cols, float eps, int rmsnorm) {
  constexpr int LPW = 4 / CH;  // lanes that share one 32-element window
  __shared__ float lvl_a[kThreads * G / LPW];
  __shared__ float lvl_b[(kThreads * G / LPW + 31) / 32];
  __shared__ float red[kThreads / 64];

  const int tid = threadIdx.x;
  const int row = blockIdx.x;
  if (row >= rows) return;
  const uint16_t* xr = x + (size_t)row * cols;
  uint8_t* qr = q + (size_t)row * cols;

  float v[G][CH][8];
#pragma unroll
  for (int g = 0; g < G; ++g) {
#pragma unroll
    for (int c = 0; c < CH; ++c) {
      const int e0 = ((g * kThreads + tid) * CH + c) * 8;
      if (VEC) {
        uintx4 w = {0u, 0u, 0u, 0u};
        if (e0 < cols) w = *reinterpret_cast<const uintx4*>(xr + e0);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          v[g][c][2 * i] = bf16lo_to_f32(w[i]);
          v[g][c][2 * i + 1] = bf16hi_to_f32(w[i]);
        }
      } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) v[g][c][i] = e0 + i < cols ? bf16_to_f32(xr[e0 + i]) : 0.0f;
      }
    }
  }

  float rinv = 1.0f;
  if (rmsnorm) {
    // level 1: 32-element windows, left to right, chained across the LPW lanes of a window
    const int n1 = (cols + 31) / 32;
#pragma unroll
    for (int g = 0; g < G; ++g) {
      float sq[CH][8];
#pragma unroll
      for (int c = 0; c < CH; ++c)
#pragma unroll
        for (int i = 0; i < 8; ++i) sq[c][i] = v[g][c][i] * v[g][c][i];
      float res = 0.0f;
#pragma unroll
      for (int r = 0; r < LPW; ++r) {
        float carry = r == 0 ? 0.0f : lane_shr1(res);
        float acc = carry;
#pragma unroll
        for (int c = 0; c < CH; ++c)
#pragma unroll
          for (int i = 0; i < 8; ++i) acc = acc + sq[c][i];
        if ((tid % LPW) == r) res = acc;
      }
      const int w = (g * kThreads + tid) / LPW;
      if ((tid % LPW) == LPW - 1 && w < n1) lvl_a[w] = res;
    }
    __syncthreads();
    // upper levels in LDS: windows of 32 partial sums, left to right
    float* src = lvl_a;
    float* dst = lvl_b;
    int n = n1;
    while (n > 1) {
      const int m = (n + 31) / 32;
      if (tid < m) {
        const int lo = tid * 32, hi = min(lo + 32, n);
        float acc = 0.0f;
        for (int i = lo; i < hi; ++i) acc = acc + src[i];
        dst[tid] = acc;
      }
      __syncthreads();
      float* t = src;
      src = dst;
      dst = t;
      n = m;
    }
    const float ms = src[0] / (float)cols;
    rinv = 1.0f / __builtin_sqrtf(ms + eps);
  }

  // y and its absolute maximum
  float amax = 0.0f;
  bool has_nan = false;
#pragma unroll
  for (int g = 0; g < G; ++g) {
#pragma unroll
    for (int c = 0; c < CH; ++c) {
      const int e0 = ((g * kThreads + tid) * CH + c) * 8;
      if (rmsnorm) {
        float gm[8];
        if (VEC) {
          uintx4 w = {0u, 0u, 0u, 0u};
          if (e0 < cols) w = *reinterpret_cast<const uintx4*>(gamma + e0);
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            gm[2 * i] = bf16lo_to_f32(w[i]);
            gm[2 * i + 1] = bf16hi_to_f32(w[i]);
          }
        } else {
#pragma unroll
          for (int i = 0; i < 8; ++i) gm[i] = e0 + i < cols ? bf16_to_f32(gamma[e0 + i]) : 0.0f;
        }
#pragma unroll
        for (int i = 0; i < 8; i += 2) {
          float t0 = (v[g][c][i] * rinv) * gm[i];
          float t1 = (v[g][c][i + 1] * rinv) * gm[i + 1];
          uint32_t pk = pack_bf16x2(t0, t1);
          v[g][c][i] = bf16lo_to_f32(pk);
          v[g][c][i + 1] = bf16hi_to_f32(pk);
        }
      }
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        float a = __builtin_fabsf(v[g][c][i]);
        has_nan |= a != a;
        amax = __builtin_fmaxf(amax, a);
      }
    }
  }
  amax = wave_max(amax);
  const bool any_nan = __any(has_nan);
  if ((tid & 63) == 0) red[tid >> 6] = any_nan ? bits_to_f32(0x7fc00000u) : amax;
  __syncthreads();
  {
    float m = red[0];
    bool nan_seen = m != m;
#pragma unroll
    for (int i = 1; i < kThreads / 64; ++i) {
      float t = red[i];
      nan_seen |= t != t;
      m = __builtin_fmaxf(m, t);
    }
    amax = nan_seen ? bits_to_f32(0x7fc00000u) : m;  // maximum propagates NaN in XLA
  }
  const float s = amax / 448.0f;
  if (tid == 0) scales[row] = s;

  // The reciprocal shortcut is exact only for an ordinary s; otherwise (zero, NaN, huge,
  // tiny, all-ones significand) every quotient takes the IEEE divide and the software cast,
  // which also reproduces the NaN codes the unguarded HLO yields for an all-zero row.
  const bool fast = ordinary_divisor(s);
  const float rs = 1.0f / s;

#pragma unroll
  for (int g = 0; g < G; ++g) {
#pragma unroll
    for (int c = 0; c < CH; ++c) {
      const int e0 = ((g * kThreads + tid) * CH + c) * 8;
      uint32_t out[2];
      if (fast) {
        float d[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          float t = div_by_ordinary(v[g][c][i], s, rs);
          d[i] = __builtin_amdgcn_fmed3f(t, -448.0f, 448.0f);
        }
        out[0] = pack_f8x4(d[0], d[1], d[2], d[3]);
        out[1] = pack_f8x4(d[4], d[5], d[6], d[7]);
      } else {
        out[0] = out[1] = 0u;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          float t = v[g][c][i] / s;
          if (t == t) t = __builtin_fminf(__builtin_fmaxf(t, -448.0f), 448.0f);
          out[i >> 2] |= f32_to_f8e4m3fn_any(t) << (8 * (i & 3));
        }
      }
      if (VEC) {
        if (e0 < cols) {
          uintx2 o = {out[0], out[1]};
          *reinterpret_cast<uintx2*>(qr + e0) = o;
        }
      } else {
#pragma unroll
        for (int i = 0; i < 8; ++i)
          if (e0 + i < cols) qr[e0 + i] = (uint8_t)(out[i >> 2] >> (8 * (i & 3)));
      }
    }
  }
}

template <int CH, int G, bool VEC>
void launch_variant(const XlaAmdRowwiseQuantize& p, hipStream_t stream) {
  hipLaunchKernelGGL((rowwise_quantize_kernel<CH, G, VEC>), dim3((unsigned)p.rows), dim3(kThreads),
                     0, stream, (const uint16_t*)p.x, (const uint16_t*)p.gamma, (uint8_t*)p.q,
                     p.scales, (int)p.rows, (int)p.cols, p.eps, p.rmsnorm);
}

}  // namespace

int LaunchRowwiseQuantize(const XlaAmdRowwiseQuantize& p, hipStream_t stream, int variant) {
  if (p.rows < 0 || p.cols < 0 || p.rows > 0x7fffffff)
    return Fail(XLA_FFI_Error_Code_INVALID_ARGUMENT, "rowwise_quantize_fp8: bad shape");
  if (p.rows == 0 || p.cols == 0) {
    SetLastKernel("rowwise_quantize_fp8:empty");
    return 0;
  }
  if (!p.x || !p.q || !p.scales || (p.rmsnorm && !p.gamma))
    return Fail(XLA_FFI_Error_Code_INVALID_ARGUMENT, "rowwise_quantize_fp8: null buffer");
  constexpr int64_t kMaxCols = 256 * 8 * 8;  // 8 chunks of 8 per lane
  if (p.cols > kMaxCols)
    return Fail(XLA_FFI_Error_Code_UNIMPLEMENTED,
                "rowwise_quantize_fp8: rows longer than 16384 elements are not supported");
  const bool vec = p.cols % 8 == 0 && ((uintptr_t)p.x % 16 == 0) && ((uintptr_t)p.q % 8 == 0) &&
                   (!p.rmsnorm || (uintptr_t)p.gamma % 16 == 0);
  const int64_t chunks = (p.cols + 7) / 8;          // 8-element chunks in a row
  const int64_t per_lane = (chunks + 255) / 256;    // chunks a lane must own
  // variant: 0 = one chunk per lane per group (fully coalesced 128-bit accesses),
  //          1 = two consecutive chunks, 2 = four consecutive chunks (a lane owns whole windows)
  int ch = variant == 2 ? 4 : variant == 1 ? 2 : 1;
  if (!vec) ch = 1;
  const int g = (int)((per_lane + ch - 1) / ch);
#define XLA_AMD_Q_CASE(CH_, G_)                                                  \
  if (ch == CH_ && g <= G_) {                                                    \
    if (vec) launch_variant<CH_, G_, true>(p, stream);                           \
    else launch_variant<CH_, G_, false>(p, stream);                              \
    SetLastKernel("rowwise_quantize_fp8:ch" #CH_ "_g" #G_);                      \
    return CheckLaunch("rowwise_quantize_fp8");                                  \
  }
  XLA_AMD_Q_CASE(1, 1) XLA_AMD_Q_CASE(1, 2) XLA_AMD_Q_CASE(1, 4) XLA_AMD_Q_CASE(1, 8)
  XLA_AMD_Q_CASE(2, 1) XLA_AMD_Q_CASE(2, 2) XLA_AMD_Q_CASE(2, 4)
  XLA_AMD_Q_CASE(4, 1) XLA_AMD_Q_CASE(4, 2)
#undef XLA_AMD_Q_CASE
  return Fail(XLA_FFI_Error_Code_INTERNAL, "rowwise_quantize_fp8: no kernel variant for this shape");
}

}  // namespace xla_amd
