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

// ---------------------------------------------------------------------------------------------
// The kernel that serves 16-byte aligned rows.  Same arithmetic, organised around what the
// instructions cost on gfx950 (measured, wave64 per SIMD: v_add/v_mul/v_fma/v_and 2 cycles;
// shifts, v_max, compares, v_bfi, v_med3, DPP forms and v_cvt_pk_bf16_f32 4; v_cvt_pk_fp8_f32 8):
//  * level-1 sums: a window of 32 is owned by 4 neighbouring lanes (8 elements each) and must be
//    added left to right.  Round r adds the lane's 8 squares on top of what the left neighbour
//    held after round r-1, every round into a register of its own: lane p's value is right after
//    round p (its neighbour's was right one round earlier), so lane 3 ends with the window's sum
//    and no lane ever selects between rounds.
//  * levels 2 and 3 are done by every wave for itself straight after one barrier: lane l adds
//    window l of the level-1 sums (read as eight 128-bit LDS loads), then the at most 16 results
//    are added in order through readlane.
//  * y only lives as packed bf16 pairs: amax is a packed 16-bit integer maximum of the absolute
//    bit patterns (every NaN pattern is larger than every number, so NaN wins as in XLA's
//    maximum), one v_and and one v_pk_max_u16 per pair.
//  * quotients need no clamp when the scale is ordinary: |y| <= amax and s = RN(amax / 448) make
//    |y / s| <= 448 (1 + 2^-23), which rounds to the code of 448.  The sign of a zero quotient,
//    lost by the correction step of the division, comes back by copying the sign bits of y over
//    the four codes of a dword (s > 0, so the code always carries the sign of y).
__device__ __forceinline__ float chain_carry(float prev) {
  // what the left neighbour holds (lanes 0, 16, 32, 48 read nothing useful and start windows)
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, prev), 0x111 /*row_shr:1*/,
                                                               0xf, 0xf, false));
}

__device__ __forceinline__ uint32_t wave_max_u32(uint32_t x) {
  auto mx = [](uint32_t a, int b) { return a > (uint32_t)b ? a : (uint32_t)b; };
  x = mx(x, __builtin_amdgcn_update_dpp(0, (int)x, 0xb1 /*quad_perm:[1,0,3,2]*/, 0xf, 0xf, true));
  x = mx(x, __builtin_amdgcn_update_dpp(0, (int)x, 0x4e /*quad_perm:[2,3,0,1]*/, 0xf, 0xf, true));
  x = mx(x, __builtin_amdgcn_update_dpp(0, (int)x, 0x141 /*row_half_mirror*/, 0xf, 0xf, true));
  x = mx(x, __builtin_amdgcn_update_dpp(0, (int)x, 0x140 /*row_mirror*/, 0xf, 0xf, true));
  uint32_t m = (uint32_t)__builtin_amdgcn_readlane((int)x, 0);
  m = mx(m, __builtin_amdgcn_readlane((int)x, 16));
  m = mx(m, __builtin_amdgcn_readlane((int)x, 32));
  m = mx(m, __builtin_amdgcn_readlane((int)x, 48));
  return m;
}

// G: 8-element chunks per lane (1, 2, 4 or 8); a row has at most 2048 * G elements.
template <int G>
__global__ __launch_bounds__(kThreads) void rowwise_quantize_chain_kernel(
    const uint16_t* __restrict__ x, const uint16_t* __restrict__ gamma, uint8_t* __restrict__ q,
    float* __restrict__ scales, int rows, int cols, float eps, int rmsnorm) {
  typedef uint16_t u16x2 __attribute__((ext_vector_type(2)));
  constexpr int kWindows = 64 * G;  // level-1 sums of a full row; a multiple of 32
  __shared__ __attribute__((aligned(16))) float lvl_a[kWindows];
  __shared__ uint32_t red[kThreads / 64];

  const int tid = threadIdx.x;
  const int p = tid & 3;
  const int row = blockIdx.x;
  if (row >= rows) return;
  const uint16_t* xr = x + (size_t)row * cols;
  uint8_t* qr = q + (size_t)row * cols;

  int e0[G];
  uintx4 raw[G], gw[G];
#pragma unroll
  for (int j = 0; j < G; ++j) {
    e0[j] = (j * kThreads + tid) * 8;
    raw[j] = uintx4{0u, 0u, 0u, 0u};
    if (e0[j] < cols) raw[j] = *reinterpret_cast<const uintx4*>(xr + e0[j]);
  }
  if (rmsnorm) {  // requested now, needed only after the sums
#pragma unroll
    for (int j = 0; j < G; ++j) {
      gw[j] = uintx4{0u, 0u, 0u, 0u};
      if (e0[j] < cols) gw[j] = *reinterpret_cast<const uintx4*>(gamma + e0[j]);
    }
  }

  float rinv = 1.0f;
  if (rmsnorm) {
    const int n1 = (cols + 31) / 32;
    for (int i = n1 + tid; i < kWindows; i += kThreads) lvl_a[i] = 0.0f;  // a short last window adds zeros
#pragma unroll
    for (int j = 0; j < G; ++j) {
      float sq[8];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float lo = bf16lo_to_f32(raw[j][i]), hi = bf16hi_to_f32(raw[j][i]);
        sq[2 * i] = lo * lo;
        sq[2 * i + 1] = hi * hi;
      }
      float acc = 0.0f;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        acc = (r == 0 ? 0.0f : chain_carry(acc)) + sq[0];
#pragma unroll
        for (int i = 1; i < 8; ++i) acc = acc + sq[i];
      }
      const int w = j * 64 + (tid >> 2);
      if (p == 3 && w < n1) lvl_a[w] = acc;
    }
    __syncthreads();
    const int m2 = (n1 + 31) / 32;  // level-2 windows, at most 16
    const int lane = tid & 63;
    float s2 = 0.0f;
    if (lane < m2) {
      const floatx4* src = reinterpret_cast<const floatx4*>(lvl_a + lane * 32);
      floatx4 w[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) w[i] = src[i];
#pragma unroll
      for (int i = 0; i < 8; ++i) s2 = (((s2 + w[i][0]) + w[i][1]) + w[i][2]) + w[i][3];
    }
    float tot = 0.0f;  // level 3; with a single level-2 window this is 0 + s2 = s2
#pragma unroll
    for (int t = 0; t < 16; ++t)
      if (t < m2) tot = tot + __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, s2), t));
    const float ms = tot / (float)cols;
    rinv = 1.0f / __builtin_sqrtf(ms + eps);
  }

  // y as packed bf16 pairs, and the largest absolute bit pattern
  uint32_t pk[G][4];
  u16x2 mx = {0, 0};
#pragma unroll
  for (int j = 0; j < G; ++j) {
    if (rmsnorm) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float t0 = (bf16lo_to_f32(raw[j][i]) * rinv) * bf16lo_to_f32(gw[j][i]);
        const float t1 = (bf16hi_to_f32(raw[j][i]) * rinv) * bf16hi_to_f32(gw[j][i]);
        pk[j][i] = pack_bf16x2(t0, t1);
      }
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) pk[j][i] = raw[j][i];
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
      mx = __builtin_elementwise_max(mx, __builtin_bit_cast(u16x2, pk[j][i] & 0x7fff7fffu));
  }
  uint32_t m16 = mx[0] > mx[1] ? (uint32_t)mx[0] : (uint32_t)mx[1];
  m16 = wave_max_u32(m16);
  if ((tid & 63) == 0) red[tid >> 6] = m16;
  __syncthreads();
#pragma unroll
  for (int i = 0; i < kThreads / 64; ++i) m16 = red[i] > m16 ? red[i] : m16;
  // maximum propagates NaN in XLA: any NaN among y makes amax the canonical NaN
  const float amax = m16 > 0x7f80u ? bits_to_f32(0x7fc00000u) : bits_to_f32(m16 << 16);
  const float s = amax / 448.0f;
  if (tid == 0) scales[row] = s;

  const bool fast = ordinary_divisor(s);
  const float rs = 1.0f / s;
#pragma unroll
  for (int j = 0; j < G; ++j) {
    uint32_t out[2];
    if (fast) {
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const uint32_t pa = pk[j][2 * h], pb = pk[j][2 * h + 1];
        const float y[4] = {bf16lo_to_f32(pa), bf16hi_to_f32(pa), bf16lo_to_f32(pb), bf16hi_to_f32(pb)};
        float d[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float q0 = y[i] * rs;
          d[i] = __builtin_fmaf(__builtin_fmaf(-q0, s, y[i]), rs, q0);
        }
        const uint32_t codes = pack_f8x4(d[0], d[1], d[2], d[3]);
        const uint32_t signs = __builtin_amdgcn_perm(pb, pa, 0x07050301u);  // high bytes of the four bf16
        out[h] = (codes & 0x7f7f7f7fu) | (signs & 0x80808080u);
      }
    } else {
      out[0] = out[1] = 0u;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const uint32_t w = pk[j][i >> 1];
        float t = ((i & 1) ? bf16hi_to_f32(w) : bf16lo_to_f32(w)) / s;
        if (t == t) t = __builtin_fminf(__builtin_fmaxf(t, -448.0f), 448.0f);
        out[i >> 2] |= f32_to_f8e4m3fn_any(t) << (8 * (i & 3));
      }
    }
    if (e0[j] < cols) {
      uintx2 o = {out[0], out[1]};
      // streaming store: the codes are not read again by this kernel (measured 77 -> 66 us on
      // 16384 x 8192; streaming loads of x on top of it lose that again)
      __builtin_nontemporal_store(o, reinterpret_cast<uintx2*>(qr + e0[j]));
    }
  }
}

// Rows longer than the register-resident kernels take (more than 16384 elements): the same
// arithmetic in three walks over the row, which a workgroup re-reads from L2 instead of keeping it
// in registers -- sums of squares per 32-element window (left to right, as above) into LDS and the
// upper levels there; then y and its maximum; then the codes.  A row of up to 2^20 elements has at
// most 32768 first-level sums (128 KiB of LDS, sized by the launch).
template <bool VEC>
__global__ __launch_bounds__(kThreads) void rowwise_quantize_long_kernel(
    const uint16_t* __restrict__ x, const uint16_t* __restrict__ gamma, uint8_t* __restrict__ q,
    float* __restrict__ scales, int rows, int cols, float eps, int rmsnorm) {
  extern __shared__ float lvl[];  // [n1] first-level sums, then [ceil(n1 / 32)] for the level above
  __shared__ float red[kThreads / 64];
  const int tid = threadIdx.x;
  const int row = blockIdx.x;
  if (row >= rows) return;
  const uint16_t* xr = x + (size_t)row * cols;
  uint8_t* qr = q + (size_t)row * cols;

  // eight consecutive elements from e0 on (zeros past the end of the row)
  auto load8 = [&](const uint16_t* src, int e0, float* out) {
    if (VEC) {
      uintx4 w = {0u, 0u, 0u, 0u};
      if (e0 < cols) w = *reinterpret_cast<const uintx4*>(src + e0);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        out[2 * i] = bf16lo_to_f32(w[i]);
        out[2 * i + 1] = bf16hi_to_f32(w[i]);
      }
    } else {
#pragma unroll
      for (int i = 0; i < 8; ++i) out[i] = e0 + i < cols ? bf16_to_f32(src[e0 + i]) : 0.0f;
    }
  };

  float rinv = 1.0f;
  if (rmsnorm) {
    const int n1 = (cols + 31) / 32;
    for (int w = tid; w < n1; w += kThreads) {
      float acc = 0.0f;
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        float v[8];
        load8(xr, w * 32 + c * 8, v);
#pragma unroll
        for (int i = 0; i < 8; ++i) acc = acc + v[i] * v[i];
      }
      lvl[w] = acc;
    }
    __syncthreads();
    float* src = lvl;
    float* dst = lvl + n1;
    int n = n1;
    while (n > 1) {
      const int m = (n + 31) / 32;
      for (int w = tid; w < m; w += kThreads) {
        const int lo = w * 32, hi = min(lo + 32, n);
        float acc = 0.0f;
        for (int i = lo; i < hi; ++i) acc = acc + src[i];
        dst[w] = acc;
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

  // y = bf16((x * rinv) * gamma), or x itself
  auto y8 = [&](int e0, float* y) {
    load8(xr, e0, y);
    if (rmsnorm) {
      float gm[8];
      load8(gamma, e0, gm);
#pragma unroll
      for (int i = 0; i < 8; i += 2) {
        const uint32_t pk = pack_bf16x2((y[i] * rinv) * gm[i], (y[i + 1] * rinv) * gm[i + 1]);
        y[i] = bf16lo_to_f32(pk);
        y[i + 1] = bf16hi_to_f32(pk);
      }
    }
  };

  float amax = 0.0f;
  bool has_nan = false;
  for (int e0 = tid * 8; e0 < cols; e0 += kThreads * 8) {
    float y[8];
    y8(e0, y);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const float a = __builtin_fabsf(y[i]);
      has_nan |= a != a;
      amax = __builtin_fmaxf(amax, a);
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
      const float t = red[i];
      nan_seen |= t != t;
      m = __builtin_fmaxf(m, t);
    }
    amax = nan_seen ? bits_to_f32(0x7fc00000u) : m;  // maximum propagates NaN in XLA
  }
  const float s = amax / 448.0f;
  if (tid == 0) scales[row] = s;
  const bool fast = ordinary_divisor(s);
  const float rs = 1.0f / s;

  for (int e0 = tid * 8; e0 < cols; e0 += kThreads * 8) {
    float y[8];
    y8(e0, y);
    uint32_t out[2];
    if (fast) {
      float d[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) d[i] = __builtin_amdgcn_fmed3f(div_by_ordinary(y[i], s, rs), -448.0f, 448.0f);
      out[0] = pack_f8x4(d[0], d[1], d[2], d[3]);
      out[1] = pack_f8x4(d[4], d[5], d[6], d[7]);
    } else {
      out[0] = out[1] = 0u;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        float t = y[i] / s;
        if (t == t) t = __builtin_fminf(__builtin_fmaxf(t, -448.0f), 448.0f);
        out[i >> 2] |= f32_to_f8e4m3fn_any(t) << (8 * (i & 3));
      }
    }
    if (VEC) {
      *reinterpret_cast<uintx2*>(qr + e0) = uintx2{out[0], out[1]};
    } else {
#pragma unroll
      for (int i = 0; i < 8; ++i)
        if (e0 + i < cols) qr[e0 + i] = (uint8_t)(out[i >> 2] >> (8 * (i & 3)));
    }
  }
}

// Aligned rows of 16385 to 65536 elements: one workgroup of 1024 lanes per row, the row held in LDS
// (up to 128 KiB) instead of in registers, so x still crosses HBM once.  First the row is copied in
// (16 bytes per lane, consecutive lanes consecutive chunks); then a lane per 32-element window adds
// its squares left to right and the upper levels follow as above; then every chunk is replaced in
// place by y (gamma comes from L2 once) while the maximum is taken; then the codes are made from y.
constexpr int kLdsRowThreads = 1024;
__global__ __launch_bounds__(kLdsRowThreads) void rowwise_quantize_lds_row_kernel(
    const uint16_t* __restrict__ x, const uint16_t* __restrict__ gamma, uint8_t* __restrict__ q,
    float* __restrict__ scales, int rows, int cols, float eps, int rmsnorm) {
  extern __shared__ __attribute__((aligned(16))) uint8_t lds_raw[];
  __shared__ uint32_t red[kLdsRowThreads / 64];
  const int tid = threadIdx.x;
  const int row = blockIdx.x;
  if (row >= rows) return;
  const int chunks = cols >> 3;                       // cols % 8 == 0
  const int padded = (chunks + 3) & ~3;               // whole 32-element windows; the padding holds zeros
  uintx4* const rowv = reinterpret_cast<uintx4*>(lds_raw);
  float* const lvl = reinterpret_cast<float*>(lds_raw + (size_t)padded * 16);
  const uintx4* xr = reinterpret_cast<const uintx4*>(x + (size_t)row * cols);
  uint8_t* qr = q + (size_t)row * cols;

  for (int i = tid; i < padded; i += kLdsRowThreads) rowv[i] = i < chunks ? xr[i] : uintx4{0u, 0u, 0u, 0u};
  __syncthreads();

  auto unpack8 = [](const uintx4& w, float* out) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      out[2 * i] = bf16lo_to_f32(w[i]);
      out[2 * i + 1] = bf16hi_to_f32(w[i]);
    }
  };

  float rinv = 1.0f;
  if (rmsnorm) {
    const int n1 = padded >> 2;
    // every level is padded with zeros to whole windows of 32, so a window is always eight 16-byte
    // reads (adding the zeros changes nothing: the sums are not negative)
    const int n1p = (n1 + 31) & ~31;
    for (int w = n1 + tid; w < n1p; w += kLdsRowThreads) lvl[w] = 0.0f;
    for (int w = tid; w < n1; w += kLdsRowThreads) {
      uintx4 c4[4];
#pragma unroll
      for (int c = 0; c < 4; ++c) c4[c] = rowv[w * 4 + c];
      float acc = 0.0f;
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        float v[8];
        unpack8(c4[c], v);
#pragma unroll
        for (int i = 0; i < 8; ++i) acc = acc + v[i] * v[i];
      }
      lvl[w] = acc;
    }
    __syncthreads();
    float* src = lvl;
    int n = n1, np = n1p;
    while (n > 1) {
      const int m = (n + 31) / 32, mp = (m + 31) & ~31;
      float* dst = src + np;
      for (int w = tid; w < mp; w += kLdsRowThreads) {
        float acc = 0.0f;
        if (w < m) {
          const floatx4* win = reinterpret_cast<const floatx4*>(src + w * 32);
          floatx4 v[8];
#pragma unroll
          for (int i = 0; i < 8; ++i) v[i] = win[i];
#pragma unroll
          for (int i = 0; i < 8; ++i) acc = (((acc + v[i][0]) + v[i][1]) + v[i][2]) + v[i][3];
        }
        dst[w] = acc;
      }
      __syncthreads();
      src = dst;
      n = m;
      np = mp;
    }
    const float ms = src[0] / (float)cols;
    rinv = 1.0f / __builtin_sqrtf(ms + eps);
  }

  // y replaces x in place as packed bf16 pairs; the maximum is taken over the absolute bit patterns
  // (every NaN pattern exceeds every number, which is XLA's NaN-propagating maximum)
  typedef uint16_t u16x2 __attribute__((ext_vector_type(2)));
  u16x2 mx = {0, 0};
  const uintx4* gv = reinterpret_cast<const uintx4*>(gamma);
  for (int i = tid; i < chunks; i += kLdsRowThreads) {
    uintx4 w = rowv[i];
    if (rmsnorm) {
      const uintx4 g = gv[i];
#pragma unroll
      for (int e = 0; e < 4; ++e)
        w[e] = pack_bf16x2((bf16lo_to_f32(w[e]) * rinv) * bf16lo_to_f32(g[e]), (bf16hi_to_f32(w[e]) * rinv) * bf16hi_to_f32(g[e]));
      rowv[i] = w;  // the same lane reads this chunk again below: no barrier needed
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) mx = __builtin_elementwise_max(mx, __builtin_bit_cast(u16x2, w[e] & 0x7fff7fffu));
  }
  uint32_t m16 = mx[0] > mx[1] ? (uint32_t)mx[0] : (uint32_t)mx[1];
  m16 = wave_max_u32(m16);
  if ((tid & 63) == 0) red[tid >> 6] = m16;
  __syncthreads();
#pragma unroll
  for (int i = 0; i < kLdsRowThreads / 64; ++i) m16 = red[i] > m16 ? red[i] : m16;
  const float amax = m16 > 0x7f80u ? bits_to_f32(0x7fc00000u) : bits_to_f32(m16 << 16);
  const float s = amax / 448.0f;
  if (tid == 0) scales[row] = s;
  const bool fast = ordinary_divisor(s);
  const float rs = 1.0f / s;

  for (int i = tid; i < chunks; i += kLdsRowThreads) {
    const uintx4 w = rowv[i];
    uint32_t out[2];
    if (fast) {  // no clamp needed and the zero's sign restored, as in the kernel above
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const uint32_t pa = w[2 * h], pb = w[2 * h + 1];
        const float y[4] = {bf16lo_to_f32(pa), bf16hi_to_f32(pa), bf16lo_to_f32(pb), bf16hi_to_f32(pb)};
        float d[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const float q0 = y[e] * rs;
          d[e] = __builtin_fmaf(__builtin_fmaf(-q0, s, y[e]), rs, q0);
        }
        const uint32_t codes = pack_f8x4(d[0], d[1], d[2], d[3]);
        const uint32_t signs = __builtin_amdgcn_perm(pb, pa, 0x07050301u);  // high bytes of the four bf16
        out[h] = (codes & 0x7f7f7f7fu) | (signs & 0x80808080u);
      }
    } else {
      out[0] = out[1] = 0u;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const uint32_t v = w[e >> 1];
        float t = ((e & 1) ? bf16hi_to_f32(v) : bf16lo_to_f32(v)) / s;
        if (t == t) t = __builtin_fminf(__builtin_fmaxf(t, -448.0f), 448.0f);
        out[e >> 2] |= f32_to_f8e4m3fn_any(t) << (8 * (e & 3));
      }
    }
    __builtin_nontemporal_store(uintx2{out[0], out[1]}, reinterpret_cast<uintx2*>(qr + (size_t)i * 8));
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
  const bool vec = p.cols % 8 == 0 && ((uintptr_t)p.x % 16 == 0) && ((uintptr_t)p.q % 8 == 0) &&
                   (!p.rmsnorm || (uintptr_t)p.gamma % 16 == 0);
  if (p.cols > kMaxCols) {
    if (p.cols > (1 << 20))
      return Fail(XLA_FFI_Error_Code_UNIMPLEMENTED,
                  "rowwise_quantize_fp8: rows longer than 1048576 elements are not supported");
    const int64_t n1 = (p.cols + 31) / 32;
    if (vec && p.cols <= 65536 && variant == 0) {
      // the row (padded to whole windows) and two levels of window sums
      // the row (padded to whole windows) and the levels of window sums, each padded to whole windows
      const size_t lds_row = (size_t)n1 * 64 + (size_t)(((n1 + 31) & ~31) + 160) * sizeof(float);
      hipError_t e = hipFuncSetAttribute((const void*)rowwise_quantize_lds_row_kernel,
                                         hipFuncAttributeMaxDynamicSharedMemorySize, 144 * 1024);
      if (e != hipSuccess)
        return Fail(XLA_FFI_Error_Code_INTERNAL, "rowwise_quantize_fp8: cannot reserve LDS: %s", hipGetErrorString(e));
      hipLaunchKernelGGL(rowwise_quantize_lds_row_kernel, dim3((unsigned)p.rows), dim3(kLdsRowThreads), lds_row, stream,
                         (const uint16_t*)p.x, (const uint16_t*)p.gamma, (uint8_t*)p.q, p.scales, (int)p.rows,
                         (int)p.cols, p.eps, p.rmsnorm);
      SetLastKernel("rowwise_quantize_fp8:lds_row");
      return CheckLaunch("rowwise_quantize_fp8");
    }
    const size_t lds = p.rmsnorm ? (size_t)(n1 + (n1 + 31) / 32) * sizeof(float) : 0;
    const void* fn = vec ? (const void*)rowwise_quantize_long_kernel<true> : (const void*)rowwise_quantize_long_kernel<false>;
    if (lds > 48 * 1024) {
      // per kernel and device; setting it twice to the same value is harmless
      hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, 136 * 1024);
      if (e != hipSuccess)
        return Fail(XLA_FFI_Error_Code_INTERNAL, "rowwise_quantize_fp8: cannot reserve LDS: %s", hipGetErrorString(e));
    }
    if (vec)
      hipLaunchKernelGGL((rowwise_quantize_long_kernel<true>), dim3((unsigned)p.rows), dim3(kThreads), lds, stream,
                         (const uint16_t*)p.x, (const uint16_t*)p.gamma, (uint8_t*)p.q, p.scales, (int)p.rows,
                         (int)p.cols, p.eps, p.rmsnorm);
    else
      hipLaunchKernelGGL((rowwise_quantize_long_kernel<false>), dim3((unsigned)p.rows), dim3(kThreads), lds, stream,
                         (const uint16_t*)p.x, (const uint16_t*)p.gamma, (uint8_t*)p.q, p.scales, (int)p.rows,
                         (int)p.cols, p.eps, p.rmsnorm);
    SetLastKernel(vec ? "rowwise_quantize_fp8:long" : "rowwise_quantize_fp8:long_unaligned");
    return CheckLaunch("rowwise_quantize_fp8");
  }
  const int64_t chunks = (p.cols + 7) / 8;          // 8-element chunks in a row
  const int64_t per_lane = (chunks + 255) / 256;    // chunks a lane must own
  // variant 0: the chained kernel for aligned rows; 1, 2, 3: the earlier layouts below (kept for
  // rows that are not 16-byte aligned and for comparison)
  if (vec && variant == 0) {
    const int g2 = per_lane <= 1 ? 1 : per_lane <= 2 ? 2 : per_lane <= 4 ? 4 : 8;
#define XLA_AMD_QC_CASE(G_)                                                                     \
  if (g2 == G_) {                                                                               \
    hipLaunchKernelGGL((rowwise_quantize_chain_kernel<G_>), dim3((unsigned)p.rows), dim3(kThreads), \
                       0, stream, (const uint16_t*)p.x, (const uint16_t*)p.gamma, (uint8_t*)p.q,  \
                       p.scales, (int)p.rows, (int)p.cols, p.eps, p.rmsnorm);                     \
    SetLastKernel("rowwise_quantize_fp8:chain_g" #G_);                                          \
    return CheckLaunch("rowwise_quantize_fp8");                                                 \
  }
    XLA_AMD_QC_CASE(1) XLA_AMD_QC_CASE(2) XLA_AMD_QC_CASE(4) XLA_AMD_QC_CASE(8)
#undef XLA_AMD_QC_CASE
  }
  if (variant > 0) --variant;
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
