// Weight-streaming f8e4m3fn scaled dot for decode shapes (M <= 64):
//   out[b,m,n] = epilogue( a_scale[m] * b_scale[n] * sum_k A8[b,m,k] * B8[b,k,n] )
// -- the small-M end of the f8 matmul that GemmRewriter hands to the library
// (xla/backends/gpu/transforms/gemm_rewriter.cc:1178-1540; the dequantising multiplies by the
// scales are f32-typed, so factoring them out of the sum moves no rounding: every product of
// two f8e4m3fn numbers is exact in f32).
//
// At these sizes the rhs is the only large operand and the kernel is a stream over it, built
// like the integer-weight decode kernels next to it but with nothing to dequantise:
//  * rhs [K,N] (N minor): a lane pulls 8 bytes (8 channels) of 8 consecutive rows into
//    registers, so 16 lanes take one whole 128-byte line per row.  Four 4x4 byte transposes
//    (v_perm_b32) turn the 8 x 8 block into 8 operands of 8 consecutive k for
//    v_mfma_f32_16x16x32_fp8_fp8, whose 16 rows are 16 *output channels*; the activations are
//    the other operand (8 bytes per lane straight from memory), so an instruction yields a
//    [16 channels x 16 tokens] tile.
//  * rhs [N,K] (K minor): a load instruction takes whole 128-byte lines of 8 channels (8 lanes per
//    line, 16 bytes each); ds_bpermute_b32 then deals the pieces to the lanes that stand for
//    their channel in the matrix operand (lane (channel, kb) gets bytes 32 kb .. 32 kb + 31 of
//    the channel's line).  Which k a slot of the matrix instruction stands for is free as long
//    as both operands agree, so the activations are read 32 contiguous bytes per lane and
//    nothing is transposed.
// The waves of a workgroup split its rows of K and add their tiles through LDS in wave order;
// K may also be split over workgroups, whose f32 sums go through the workspace and a second
// small kernel, in slice order: results do not depend on scheduling.
//
// Bound: HBM.  Algorithmic bytes: K*N (rhs) + a, scales, bias and out once each.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <string.h>
#include <stdio.h>

#include "decode_common.h"
#include "device_numerics.h"
#include "launch.h"

namespace xla_amd {
namespace {

struct Fp8DecodeParams {
  const uint8_t* a;      // [batch, M, K]
  const uint8_t* b;      // [batch, K, N], or [batch, N, K]
  const float* a_scale;  // one value, or M (a_per_row)
  const float* b_scale;  // one value, or N (b_per_channel)
  // block scales instead (rhs [N,K] only): one f8e8m0fnu byte per 32 values of k,
  // [batch, M, K / 32] and [batch, N, K / 32]; K % 128 == 0
  const uint8_t* a_block_scales;
  const uint8_t* b_block_scales;
  const void* bias;      // [N] or null
  uint16_t* out;         // [batch, M, N] bf16, or
  uint8_t* out8;         // f8e4m3fn codes: convert(clamp(v / *d_scale)) (v * *d_scale unless d_divides)
  const float* d_scale;
  float* amax;           // optional: max |v| over an f8 result, folded in with atomics
  float* partial;        // slices > 1: [batch, slices, M, N] f32 sums
  int M, K, N;
  int a_per_row, b_per_channel, bias_is_bf16, d_divides;
  int bf16_dot, bf16_ops, epilogue;
  int slices, rows_per_slice, rows_per_wave;  // rows_per_wave: a multiple of the kernel's step
  int cols;                                   // consecutive strips a workgroup takes, one after the other
  // A bf16-typed dequantise multiply (per-tensor scales): with scales that are powers of two it rounds
  // nothing and these kernels serve the call; otherwise every workgroup returns at once and the kernels
  // launched behind them, which test the same condition the other way round, do.
  int require_pow2_scales;
  // The kernels that take over then (rhs [K,N]): every a * a_scale and b * b_scale rounded to bf16 on the way
  // into the bf16 matrix instruction, the scales therefore no longer on the sum; they return at once
  // when both scales are powers of two (1), or run whatever the scales are (2: per-row or per-channel
  // scales, which no single test covers: the f8 form is not launched then).
  int rounded_operands;
};

constexpr int kWaves = 8;
constexpr uint32_t kNowhere = 0x80000000u;  // a lane offset no buffer reaches: the load returns zeros

// One result value: the scales, the epilogue, and the store (bf16, or an f8 code with its amax).
__device__ __forceinline__ void finish_value(const Fp8DecodeParams& p, int batch, int m, int n, float sum, float alpha,
                                             uint32_t* amax_bits) {
  float v = sum;
  if (!p.rounded_operands) {
    if (p.a_per_row) v = v * p.a_scale[m];
    v = v * (p.b_per_channel ? alpha * p.b_scale[n] : alpha);
  }
  const float bias = p.bias ? load_scale(p.bias, n, p.bias_is_bf16) : 0.0f;
  v = epilogue_dispatch(v, bias, p.epilogue, p.bf16_dot, p.bf16_ops);
  const size_t idx = ((size_t)batch * p.M + m) * p.N + n;
  if (p.out8) {
    *amax_bits = max(*amax_bits, f32_to_bits(v) & 0x7fffffffu);  // a NaN pattern exceeds every number
    // op by op as the HLO does: an IEEE quotient (or product), clamp (a NaN stays one), cast
    float c = p.d_divides ? v / *p.d_scale : v * *p.d_scale;
    if (c == c) c = __builtin_fminf(__builtin_fmaxf(c, -448.0f), 448.0f);
    p.out8[idx] = (uint8_t)f32_to_f8e4m3fn_any(c);
  } else {
    p.out[idx] = f32_to_bf16(v);
  }
}

// One atomic per wave into the amax result, which a fill kernel zeroed before the launch.
__device__ __forceinline__ void fold_amax(const Fp8DecodeParams& p, uint32_t amax_bits) {
  if (!p.out8 || !p.amax) return;
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) amax_bits = max(amax_bits, (uint32_t)__shfl_xor((int)amax_bits, off));
  if ((threadIdx.x & 63) == 0) atomicMax(reinterpret_cast<unsigned*>(p.amax), amax_bits);
}

// Adds the waves' accumulator tiles through LDS, 32 registers (one 16-token tile) per pass, and
// finishes them.  rhs [K,N]: register r = t * 8 + j (acc[j][mt][t]) in lane (li, kb) is channel
// strip * 128 + (4 * kb + t) * 8 + j; rhs [N,K]: register r = 4 * g + t (acc[g][mt][t]) is channel
// strip * 128 + 16 * g + 4 * kb + t; token 16 * mt + li in both.  Wave w finishes registers
// 4w .. 4w+3 of every pass, four consecutive channels of one token.
template <int MT, bool NK>
__device__ __forceinline__ void reduce_and_store(const Fp8DecodeParams& p, float* lds, const floatx4 (&acc)[8][MT],
                                                 int strip, int slice, int batch) {
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int li = lane & 15, kb = lane >> 4;
  // (block scales went in with the matrix instructions)
  const float alpha = p.a_block_scales || p.rounded_operands
                          ? 1.0f : (p.a_per_row ? 1.0f : *p.a_scale) * (p.b_per_channel ? 1.0f : *p.b_scale);
  uint32_t amax_bits = 0u;
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    if (mt) __syncthreads();
#pragma unroll
    for (int r = 0; r < 32; ++r) lds[(wave * 32 + r) * 64 + lane] = NK ? acc[r >> 2][mt][r & 3] : acc[r & 7][mt][r >> 3];
    __syncthreads();
    constexpr int RPW = 32 / kWaves;
    float res[RPW];
#pragma unroll
    for (int u = 0; u < RPW; ++u) {
      float s = 0.0f;
#pragma unroll
      for (int w2 = 0; w2 < kWaves; ++w2) s = s + lds[(w2 * 32 + wave * RPW + u) * 64 + lane];
      res[u] = s;
    }
    const int m = 16 * mt + li;
    const int r0 = wave * RPW;  // the wave's first register of the pass
    const int n0 = strip * 128 + (NK ? 16 * (r0 >> 2) + 4 * kb + (r0 & 3) : (4 * kb + (r0 >> 3)) * 8 + (r0 & 7));
    if (m >= p.M || n0 >= p.N) continue;  // N % 8 == 0: an aligned run of four is inside N or not at all
    if (p.slices > 1) {
      float* dst = p.partial + (((size_t)batch * p.slices + slice) * p.M + m) * p.N + n0;
#pragma unroll
      for (int u = 0; u < RPW; ++u) dst[u] = res[u];
    } else {
#pragma unroll
      for (int u = 0; u < RPW; ++u) finish_value(p, batch, m, n0 + u, res[u], alpha, &amax_bits);
    }
  }
  if (p.slices == 1) fold_amax(p, amax_bits);
}

// rhs [K,N].  MT: 16-token tiles.  A workgroup owns 128 channels (one 128-byte line per row) and
// rows_per_slice rows, its waves rows_per_wave consecutive rows each, in steps of 32.
// ROUNDED: the operands are widened, scaled and rounded to bf16 (16 vector instructions per 8 values) and
// multiplied by v_mfma_f32_16x16x32_bf16, which takes the same 8 consecutive k per lane.
template <int MT, bool ROUNDED>
__device__ __forceinline__ void kn_strip(const Fp8DecodeParams& p, float* lds, int strip, int slice, int batch) {
  int lane = threadIdx.x & 63;
  // (opaque to the compiler, so that a strip's descriptors and offsets are made anew for every strip of
  // a caller's loop instead of staying in registers through the other strips' sums)
  asm volatile("" : "+v"(lane), "+s"(batch));
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int li = lane & 15, kb = lane >> 4;
  const int n_lane = strip * 128 + li * 8;
  const uint32_t pitch = (uint32_t)p.N;
  const __amdgpu_buffer_rsrc_t rw = make_rsrc(p.b + (size_t)batch * p.K * p.N, (uint32_t)p.K * pitch);
  // one descriptor per 16-token tile, each ending where the activations end: the lane offset is
  // then the same for every tile and still range-checks tokens >= M
  __amdgpu_buffer_rsrc_t ra[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int rows = max(p.M - 16 * mt, 0);
    ra[mt] = make_rsrc(p.a + ((size_t)batch * p.M + (rows ? 16 * mt : 0)) * p.K, (uint32_t)rows * p.K);
  }
  const uint32_t voff_w = n_lane < p.N ? (uint32_t)(8 * kb) * pitch + (uint32_t)n_lane : kNowhere;
  const uint32_t voff_a = (uint32_t)li * p.K + 8 * kb;
  // rows 1..7 of a lane's block of 8 are reached through the scalar offset: K % 8 == 0, so the
  // block is inside the rhs exactly when its first row is, which the lane offset checks
  uint32_t soff_w[8];
#pragma unroll
  for (int r = 0; r < 8; ++r) soff_w[r] = (uint32_t)r * pitch;

  floatx4 acc[8][MT];
#pragma unroll
  for (int j = 0; j < 8; ++j)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[j][mt] = floatx4{0.f, 0.f, 0.f, 0.f};

  const int slice_end = min((slice + 1) * p.rows_per_slice, p.K);
  const int k_begin = slice * p.rows_per_slice + wave * p.rows_per_wave;
  const int k_stop = min(k_begin + p.rows_per_wave, slice_end);

  // the lane's operands: token 16 mt + li of a, channels n_lane .. n_lane + 7 of the rhs
  float sa_r[MT], sb_r[8];
  if constexpr (ROUNDED) {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) sa_r[mt] = round_bf16(p.a_per_row ? p.a_scale[min(16 * mt + li, p.M - 1)] : *p.a_scale);
#pragma unroll
    for (int j = 0; j < 8; ++j) sb_r[j] = round_bf16(p.b_per_channel ? p.b_scale[min(n_lane + j, p.N - 1)] : *p.b_scale);
  }
  // 8 f8e4m3fn codes (k in byte order) -> bf16(code * s), one rounding each
  auto scaled_bf16 = [&](uint32_t lo, uint32_t hi, float s) {
    const floatx2 f0 = __builtin_amdgcn_cvt_pk_f32_fp8((int)lo, false), f1 = __builtin_amdgcn_cvt_pk_f32_fp8((int)lo, true);
    const floatx2 f2 = __builtin_amdgcn_cvt_pk_f32_fp8((int)hi, false), f3 = __builtin_amdgcn_cvt_pk_f32_fp8((int)hi, true);
    const uintx4 o = {pack_bf16x2(f0[0] * s, f0[1] * s), pack_bf16x2(f1[0] * s, f1[1] * s),
                      pack_bf16x2(f2[0] * s, f2[1] * s), pack_bf16x2(f3[0] * s, f3[1] * s)};
    return __builtin_bit_cast(bf16x8, o);
  };

  uintx2 wq[2][8];
  uintx2 aq[2][MT];
  auto load_step = [&](int buf, int k0) {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) aq[buf][mt] = __builtin_amdgcn_raw_buffer_load_b64(ra[mt], voff_a + (uint32_t)k0, 0, 0);
    const uint32_t vw = voff_w + (uint32_t)k0 * pitch;
#pragma unroll
    for (int r = 0; r < 8; ++r) wq[buf][r] = __builtin_amdgcn_raw_buffer_load_b64(rw, vw, soff_w[r], 0);
  };
  auto compute = [&](int buf, int k0) {
    uintx2 av[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) av[mt] = aq[buf][mt];
    if (k0 + 32 > p.K) {  // scalar: only a step that crosses the end of K (its rhs rows read as zeros)
      asm volatile("");
      const bool ok = k0 + 8 * kb < p.K;
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) av[mt] = uintx2{ok ? av[mt][0] : 0u, ok ? av[mt][1] : 0u};
    }
    bf16x8 ab[MT];
    if constexpr (ROUNDED) {
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) ab[mt] = scaled_bf16(av[mt][0], av[mt][1], sa_r[mt]);
    }
#pragma unroll
    for (int q = 0; q < 2; ++q) {
      // 4x4 byte transposes: t[h][e] = byte e of rows 4h .. 4h+3 of dword q
      uint32_t t[2][4];
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const uint32_t x0 = wq[buf][4 * h][q], x1 = wq[buf][4 * h + 1][q], x2 = wq[buf][4 * h + 2][q], x3 = wq[buf][4 * h + 3][q];
        const uint32_t p0 = __builtin_amdgcn_perm(x1, x0, 0x05010400u), p1 = __builtin_amdgcn_perm(x1, x0, 0x07030602u);
        const uint32_t q0 = __builtin_amdgcn_perm(x3, x2, 0x05010400u), q1 = __builtin_amdgcn_perm(x3, x2, 0x07030602u);
        t[h][0] = __builtin_amdgcn_perm(q0, p0, 0x05040100u);
        t[h][1] = __builtin_amdgcn_perm(q0, p0, 0x07060302u);
        t[h][2] = __builtin_amdgcn_perm(q1, p1, 0x05040100u);
        t[h][3] = __builtin_amdgcn_perm(q1, p1, 0x07060302u);
      }
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        if constexpr (ROUNDED) {
          const bf16x8 wb = scaled_bf16(t[0][e], t[1][e], sb_r[4 * q + e]);
#pragma unroll
          for (int mt = 0; mt < MT; ++mt)
            acc[4 * q + e][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wb, ab[mt], acc[4 * q + e][mt], 0, 0, 0);
        } else {
          const long wop = __builtin_bit_cast(long, uintx2{t[0][e], t[1][e]});
#pragma unroll
          for (int mt = 0; mt < MT; ++mt)
            acc[4 * q + e][mt] = __builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8(wop, __builtin_bit_cast(long, av[mt]),
                                                                            acc[4 * q + e][mt], 0, 0, 0);
        }
      }
    }
  };
  if (k_begin < k_stop) {
    load_step(0, k_begin);
    for (int k0 = k_begin; k0 < k_stop; k0 += 64) {
      if (k0 + 32 < k_stop) load_step(1, k0 + 32);
      compute(0, k0);
      if (k0 + 64 < k_stop) load_step(0, k0 + 64);
      if (k0 + 32 < k_stop) compute(1, k0 + 32);
    }
  }
  reduce_and_store<MT, false>(p, lds, acc, strip, slice, batch);
}

// WALK: a workgroup takes p.cols consecutive strips one after the other (more strips than CUs: one
// resident workgroup per CU that walks several strips finishes sooner than workgroups queueing for CUs;
// a kernel of its own, because the loop costs the one-strip form registers).
template <int MT, bool WALK, bool ROUNDED = false>
__global__ __launch_bounds__(kWaves * 64) void fp8_dot_decode_kn_kernel(Fp8DecodeParams p) {
  __shared__ float lds[kWaves * 32 * 64];
  if constexpr (ROUNDED) {
    if (p.rounded_operands == 1 && is_pow2_f32(*p.a_scale) && is_pow2_f32(*p.b_scale)) return;  // the f8 form has served the call
  } else {
    if (p.require_pow2_scales && !(is_pow2_f32(*p.a_scale) && is_pow2_f32(*p.b_scale))) return;
  }
  const int slice = blockIdx.x % p.slices;
  if constexpr (!WALK) {
    kn_strip<MT, ROUNDED>(p, lds, blockIdx.x / p.slices, slice, blockIdx.y);
  } else {
    const int first = (blockIdx.x / p.slices) * p.cols;
    for (int c = 0; c < p.cols && (first + c) * 128 < p.N; ++c) {
      if (c) __syncthreads();  // the sums of the strip before have left LDS
      kn_strip<MT, ROUNDED>(p, lds, first + c, slice, blockIdx.y);
    }
  }
}

// rhs [N,K].  A workgroup owns 128 channels (8 groups of 16) and rows_per_slice values of k, its
// waves rows_per_wave consecutive ones each, in steps of 128 (one line per channel), a step in two
// halves of four channel groups.  MX: block scales.  The matrix instruction takes the scale of the
// step's block j (32 values of k) from the lanes with kb = j and applies it to the first 16 bytes of
// the lanes kb = 2 (j & 1), 2 (j & 1) + 1 for j < 2 and to their second 16 bytes for j >= 2 (as
// measured on the 32x32x64 form: the first 16 bytes of all lanes of a row are k 0..63 in lane order,
// the second 16 bytes k 64..127).  So with block scales lane (., kb) holds pieces kb and kb + 4 of the
// line instead of 2 kb and 2 kb + 1; a step's four scales of a channel (or row of a) are one dword,
// of which lane (., kb) hands in byte kb.
// ROUNDED (no block scales, up to two token tiles): as in kn_strip, with four v_mfma_f32_16x16x32_bf16 per
// 32 bytes of either operand (instruction d takes bytes 8 d .. 8 d + 7 of every lane's 32).
template <int MT, bool MX, bool ROUNDED = false>
__device__ __forceinline__ void nk_strip(const Fp8DecodeParams& p, float* lds, int strip, int slice, int batch) {
  int lane = threadIdx.x & 63;
  asm volatile("" : "+v"(lane), "+s"(batch));  // as in kn_strip
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int li = lane & 15, kb = lane >> 4;
  const __amdgpu_buffer_rsrc_t rw = make_rsrc(p.b + (size_t)batch * p.K * p.N, (uint32_t)p.K * (uint32_t)p.N);
  __amdgpu_buffer_rsrc_t ra[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int rows = max(p.M - 16 * mt, 0);
    ra[mt] = make_rsrc(p.a + ((size_t)batch * p.M + (rows ? 16 * mt : 0)) * p.K, (uint32_t)rows * p.K);
  }
  // loading side: instruction (g, hh) takes channels 16 g + 8 hh + (lane >> 3), piece lane & 7 of
  // their lines; N % 8 == 0, so its 8 channels are inside N or not at all
  uint32_t voff_w[8][2];
#pragma unroll
  for (int g = 0; g < 8; ++g)
#pragma unroll
    for (int hh = 0; hh < 2; ++hh) {
      const int n = strip * 128 + 16 * g + 8 * hh + (lane >> 3);
      voff_w[g][hh] = n < p.N ? (uint32_t)n * p.K + 16u * (lane & 7) : kNowhere;
    }
  const uint32_t voff_a = (uint32_t)li * p.K + (MX ? 16 : 32) * kb;
  constexpr uint32_t kSecond = MX ? 64u : 16u;  // from a lane's first piece to its second
  // block scales: the dword of row li of a's tile, and of channel 16 g + li
  const uint32_t kblocks = (uint32_t)p.K >> 5;
  __amdgpu_buffer_rsrc_t rsa[MX ? MT : 1];
  const __amdgpu_buffer_rsrc_t rsb =
      make_rsrc(MX ? p.b_block_scales + (size_t)batch * p.N * kblocks : p.b, MX ? (uint32_t)p.N * kblocks : 0u);
  if (MX) {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      const int rows = max(p.M - 16 * mt, 0);
      rsa[mt] = make_rsrc(p.a_block_scales + ((size_t)batch * p.M + (rows ? 16 * mt : 0)) * kblocks, (uint32_t)rows * kblocks);
    }
  }
  const uint32_t voff_sa = (uint32_t)li * kblocks;
  const int n_li = strip * 128 + li;
  // consuming side: lane (li, kb) stands for channel 16 g + li and wants pieces 2 kb and 2 kb + 1,
  // which lanes 8 (li & 7) + 2 kb (+ 1) of instruction (g, li >> 3) hold
  const int src0 = 4 * (8 * (li & 7) + (MX ? kb : 2 * kb));
  constexpr int kSrcStep = MX ? 16 : 4;  // four lanes on, or the next one
  const bool upper = li >= 8;

  floatx4 acc[8][MT];
#pragma unroll
  for (int g = 0; g < 8; ++g)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[g][mt] = floatx4{0.f, 0.f, 0.f, 0.f};

  // ROUNDED: the lane's operands are token 16 mt + li of a and channel 16 g + li of the rhs
  float sa_r[MT], sb_r[8];
  if constexpr (ROUNDED) {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) sa_r[mt] = round_bf16(p.a_per_row ? p.a_scale[min(16 * mt + li, p.M - 1)] : *p.a_scale);
#pragma unroll
    for (int g = 0; g < 8; ++g) sb_r[g] = round_bf16(p.b_per_channel ? p.b_scale[min(n_li + 16 * g, p.N - 1)] : *p.b_scale);
  }
  auto scaled_bf16 = [&](uint32_t lo, uint32_t hi, float s) {
    const floatx2 f0 = __builtin_amdgcn_cvt_pk_f32_fp8((int)lo, false), f1 = __builtin_amdgcn_cvt_pk_f32_fp8((int)lo, true);
    const floatx2 f2 = __builtin_amdgcn_cvt_pk_f32_fp8((int)hi, false), f3 = __builtin_amdgcn_cvt_pk_f32_fp8((int)hi, true);
    const uintx4 o = {pack_bf16x2(f0[0] * s, f0[1] * s), pack_bf16x2(f1[0] * s, f1[1] * s),
                      pack_bf16x2(f2[0] * s, f2[1] * s), pack_bf16x2(f3[0] * s, f3[1] * s)};
    return __builtin_bit_cast(bf16x8, o);
  };

  const int slice_end = min((slice + 1) * p.rows_per_slice, p.K);
  const int k_begin = slice * p.rows_per_slice + wave * p.rows_per_wave;
  const int k_stop = min(k_begin + p.rows_per_wave, slice_end);

  uintx4 wq[2][4][2];   // [buffer][group of the half][hh]
  uintx4 aq[2][MT][2];  // [buffer][tile][16-byte half]
  uint32_t sbq[2][MX ? 4 : 1], saq[2][MX ? MT : 1];  // the step's block scales
  // A piece past the end of K (K % 16 == 0: pieces are whole) lies in the next row of its operand, not
  // past the buffer: such a load gets the offset no buffer reaches instead and returns zeros.
  auto load_a = [&](int buf, int k0) {
    const int piece = MX ? 16 * kb : 32 * kb;
    const uint32_t o0 = k0 + piece < p.K ? voff_a + (uint32_t)k0 : kNowhere;
    const uint32_t o1 = k0 + piece + (int)kSecond < p.K ? voff_a + (uint32_t)k0 + kSecond : kNowhere;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      aq[buf][mt][0] = __builtin_amdgcn_raw_buffer_load_b128(ra[mt], o0, 0, 0);
      aq[buf][mt][1] = __builtin_amdgcn_raw_buffer_load_b128(ra[mt], o1, 0, 0);
      if (MX) saq[buf][mt] = __builtin_amdgcn_raw_buffer_load_b32(rsa[mt], voff_sa + ((uint32_t)k0 >> 5), 0, 0);
    }
  };
  auto load_w = [&](int buf, int half, int k0) {
    const bool ok = k0 + 16 * (lane & 7) < p.K;
#pragma unroll
    for (int g = 0; g < 4; ++g)
#pragma unroll
      for (int hh = 0; hh < 2; ++hh)
        wq[buf][g][hh] = __builtin_amdgcn_raw_buffer_load_b128(rw, ok ? voff_w[4 * half + g][hh] + (uint32_t)k0 : kNowhere, 0, 0);
    if (MX) {
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int n = n_li + 16 * (4 * half + g);
        sbq[buf][g] = __builtin_amdgcn_raw_buffer_load_b32(rsb, n < p.N ? (uint32_t)n * kblocks + ((uint32_t)k0 >> 5) : kNowhere, 0, 0);
      }
    }
  };
  auto compute = [&](int buf, int abuf, int half) {
    uintx4 av[MT][2];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      av[mt][0] = aq[abuf][mt][0];
      av[mt][1] = aq[abuf][mt][1];
    }
    uintx4 wv[4][2];
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      wv[g][0] = wq[buf][g][0];
      wv[g][1] = wq[buf][g][1];
    }
    bf16x8 ab[ROUNDED ? MT : 1][4];
    if constexpr (ROUNDED) {
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int d = 0; d < 4; ++d)
          ab[mt][d] = scaled_bf16(av[mt][d >> 1][2 * (d & 1)], av[mt][d >> 1][2 * (d & 1) + 1], sa_r[mt]);
    }
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      uint32_t tg[8];
#pragma unroll
      for (int x = 0; x < 2; ++x)
#pragma unroll
        for (int d = 0; d < 4; ++d) {
          const uint32_t lo = (uint32_t)__builtin_amdgcn_ds_bpermute(src0 + kSrcStep * x, (int)wv[g][0][d]);
          const uint32_t hi = (uint32_t)__builtin_amdgcn_ds_bpermute(src0 + kSrcStep * x, (int)wv[g][1][d]);
          tg[4 * x + d] = upper ? hi : lo;
        }
      if constexpr (ROUNDED) {
#pragma unroll
        for (int d = 0; d < 4; ++d) {
          const bf16x8 wb = scaled_bf16(tg[2 * d], tg[2 * d + 1], sb_r[4 * half + g]);
#pragma unroll
          for (int mt = 0; mt < MT; ++mt)
            acc[4 * half + g][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wb, ab[mt][d], acc[4 * half + g][mt], 0, 0, 0);
        }
        if (g & 1) __builtin_amdgcn_sched_barrier(0);
        continue;
      }
      // 32 bytes of k per lane and operand: one v_mfma_f32_16x16x128_f8f6f4 (both formats e4m3, no block scales)
      const intx8 wop = {(int)tg[0], (int)tg[1], (int)tg[2], (int)tg[3], (int)tg[4], (int)tg[5], (int)tg[6], (int)tg[7]};
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        const intx8 aop = {(int)av[mt][0][0], (int)av[mt][0][1], (int)av[mt][0][2], (int)av[mt][0][3],
                           (int)av[mt][1][0], (int)av[mt][1][1], (int)av[mt][1][2], (int)av[mt][1][3]};
        if (MX)
          acc[4 * half + g][mt] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(
              wop, aop, acc[4 * half + g][mt], 0, 0, 0, (int)(sbq[buf][g] >> (8 * kb)), 0, (int)(saq[abuf][mt] >> (8 * kb)));
        else
          acc[4 * half + g][mt] =
              __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wop, aop, acc[4 * half + g][mt], 0, 0, 0, 0, 0, 0);
      }
      if (MX) {  // (with scale operands the compiler otherwise sinks all four groups' MFMAs below their permutes)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) asm volatile("" : "+v"(acc[4 * half + g][mt]));
      }
      if (g & 1) __builtin_amdgcn_sched_barrier(0);  // two groups' pieces on their way at a time, not all four
    }
  };
  if (k_begin < k_stop) {
    load_a(0, k_begin);
    load_w(0, 0, k_begin);
    for (int k0 = k_begin; k0 < k_stop; k0 += 256) {
      load_w(1, 1, k0);
      compute(0, 0, 0);
      if (k0 + 128 < k_stop) { load_a(1, k0 + 128); load_w(0, 0, k0 + 128); }
      compute(1, 0, 1);
      if (k0 + 128 < k_stop) {
        load_w(1, 1, k0 + 128);
        compute(0, 1, 0);
        if (k0 + 256 < k_stop) { load_a(0, k0 + 256); load_w(0, 0, k0 + 256); }
        compute(1, 1, 1);
      }
    }
  }
  reduce_and_store<MT, true>(p, lds, acc, strip, slice, batch);
}

template <int MT, bool MX, bool WALK, bool ROUNDED = false>
__global__ __launch_bounds__(kWaves * 64) void fp8_dot_decode_nk_kernel(Fp8DecodeParams p) {
  __shared__ float lds[kWaves * 32 * 64];
  if constexpr (ROUNDED) {
    if (p.rounded_operands == 1 && is_pow2_f32(*p.a_scale) && is_pow2_f32(*p.b_scale)) return;  // the f8 form has served the call
  } else {
    if (!MX && p.require_pow2_scales && !(is_pow2_f32(*p.a_scale) && is_pow2_f32(*p.b_scale))) return;
  }
  const int slice = blockIdx.x % p.slices;
  if constexpr (!WALK) {
    nk_strip<MT, MX, ROUNDED>(p, lds, blockIdx.x / p.slices, slice, blockIdx.y);
  } else {
    const int first = (blockIdx.x / p.slices) * p.cols;
    for (int c = 0; c < p.cols && (first + c) * 128 < p.N; ++c) {
      if (c) __syncthreads();
      nk_strip<MT, MX, ROUNDED>(p, lds, first + c, slice, blockIdx.y);
    }
  }
}

// Sums the K-slices in slice order and finishes the values.
__global__ __launch_bounds__(256) void fp8_dot_decode_finalize_kernel(Fp8DecodeParams p) {
  if (p.rounded_operands) {
    if (p.rounded_operands == 1 && is_pow2_f32(*p.a_scale) && is_pow2_f32(*p.b_scale)) return;
  } else if (p.require_pow2_scales && !(is_pow2_f32(*p.a_scale) && is_pow2_f32(*p.b_scale))) {
    return;
  }
  const size_t total = (size_t)p.M * p.N;
  const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
  const int batch = blockIdx.y;
  uint32_t amax_bits = 0u;
  if (idx < total) {
    const float* ws = p.partial + (size_t)batch * p.slices * total + idx;
    float v = 0.0f;
    for (int s = 0; s < p.slices; ++s) v = v + ws[(size_t)s * total];
    const float alpha = p.a_block_scales || p.rounded_operands
                            ? 1.0f : (p.a_per_row ? 1.0f : *p.a_scale) * (p.b_per_channel ? 1.0f : *p.b_scale);
    finish_value(p, batch, (int)(idx / p.N), (int)(idx % p.N), v, alpha, &amax_bits);
  }
  fold_amax(p, amax_bits);
}

// K-slices for the shape: more workgroups until every CU has one, as long as a wave keeps at
// least 128 values of k (four steps, or one of the [N,K] kernel) and the sums written and read
// again stay under a quarter of the rhs bytes.  A few workgroups more than CUs are worse than half
// as many (a second round for a quarter of the work: 80 strips take 19.8 us in 2 slices, 22.1 in 4).
int Slices(int64_t batch, int64_t M, int64_t K, int64_t N, bool nk) {
  if (int s = GetOption("fp8_decode_slices")) return s;
  const int64_t strips = (N + 127) / 128;
  int slices = 1;
  while (strips * batch * slices < 192 && slices < 16 && K / (slices * 2) >= 128 * kWaves &&
         2.0 * (slices * 2) * M * N * 4.0 <= 0.25 * (double)K * N)
    slices *= 2;
  if (slices > 1 && strips * batch * slices > 256 && strips * batch * slices < 400) slices /= 2;
  return slices;
}

}  // namespace

// More rows of a than one launch takes: the rows go through the streaming kernel in equal passes
// (every row of the result depends on its own row of a only).  rows: rows per pass, a multiple of 16.
static int Passes(int64_t M, bool nk, bool mx, int64_t* rows) {
  const int64_t most = mx ? 32 : nk ? 48 : 64;
  const int64_t passes = (M + most - 1) / most;
  *rows = passes > 0 ? ((M + passes - 1) / passes + 15) / 16 * 16 : 0;
  return (int)passes;
}

// Passes of the streaming kernel against the tiled kernel, in microseconds fitted on MI355X over
// matrices from 4096 x 4096 to 8192 x 28672: a pass 15 + 1.95e-7 K N (rhs [K,N], up to 64 rows) or
// 13 + 1.35e-7 K N (rhs [N,K], up to 48); the tiled kernel with at most one round of tiles
// 32 + 0.0071 K, 27 + 0.0052 K when it splits its tiles along K (at most 64 of them, 65 rows on).
// ([128,8192] x [8192,8192]: 69 us tiled, 46 in two passes; [64,14336] x [4096,14336]^T: 135 and 38.)
static bool PassesAreCheaper(int64_t M, int64_t K, int64_t N, bool nk, int passes, int64_t rows) {
  const int64_t tiles = ((M + 255) / 256) * ((N + 255) / 256);
  if (tiles > 256 || passes > 6) return false;
  const double kn = (double)K * (double)N;
  // (a [K,N] pass of 48 rows takes about 0.85 of one of 64)
  const double pass_us = nk ? 13.0 + 1.35e-7 * kn : (15.0 + 1.95e-7 * kn) * (0.4 + 0.6 * (double)rows / 64.0);
  const double tiled_us = tiles <= 64 && M >= 65 && K >= 2048 ? 27.0 + 0.0052 * (double)K : 32.0 + 0.0071 * (double)K;
  return (double)passes * pass_us <= tiled_us;
}

static size_t WorkspaceBytesFor(int64_t batch, int64_t M, int64_t K, int64_t N, bool nk, bool mx) {
  int64_t rows = M;
  if (M > (mx ? 32 : nk ? 48 : 64)) {  // passes follow each other on the stream and share the scratch
    if (batch > 1) return 0;
    const int passes = Passes(M, nk, mx, &rows);
    if (GetOption("fp8_dot_kernel") != 3 && !PassesAreCheaper(M, K, N, nk, passes, rows)) return 0;
  }
  size_t bytes = 0;
  for (const int64_t m : {rows, M % rows}) {  // (the last pass may have fewer rows and more slices)
    if (m <= 0) continue;
    const int slices = Slices(batch, m, K, N, nk);
    const size_t need = slices > 1 ? (size_t)batch * slices * m * N * 4 : 0;
    bytes = bytes > need ? bytes : need;
  }
  return bytes;
}

size_t Fp8DotDecodeWorkspaceBytes(int64_t batch, int64_t M, int64_t K, int64_t N, int rhs_contracting_dim) {
  if (M <= 0 || K <= 0 || N <= 0 || batch <= 0) return 0;
  const bool nk = rhs_contracting_dim == 1;
  size_t bytes = WorkspaceBytesFor(batch, M, K, N, nk, false);
  if (nk) {  // the call may come with block scales or a bf16-typed multiply (not known here): passes of 32 rows
    const size_t mx = WorkspaceBytesFor(batch, M, K, N, true, true);
    bytes = bytes > mx ? bytes : mx;
  }
  return bytes;
}

static int LaunchFp8DotDecodeRows(const XlaAmdFp8ScaledDot& p, hipStream_t stream, bool bf16_multiply, bool* any_scale);

// Returns -1 when the shape is not covered, else the launch status.
int LaunchFp8DotDecode(const XlaAmdFp8ScaledDot& p, hipStream_t stream, bool bf16_multiply, bool* any_scale) {
  const bool nk = p.rhs_contracting_dim == 1;
  const bool mx = p.a_block_scales != nullptr;
  bool dummy = false;
  if (!any_scale) any_scale = &dummy;
  *any_scale = false;
  // (the rounding form of the [N,K] kernel takes two token tiles, like the block-scaled one)
  const bool two_tiles = mx || (nk && bf16_multiply && p.dequant_type == XLA_FFI_DataType_BF16);
  if (p.M <= (two_tiles ? 32 : nk ? 48 : 64)) return LaunchFp8DotDecodeRows(p, stream, bf16_multiply, any_scale);
  if (p.batch > 1) return -1;
  int64_t rows = 0;
  const int passes = Passes(p.M, nk, two_tiles, &rows);
  if (GetOption("fp8_dot_kernel") != 3 && !PassesAreCheaper(p.M, p.K, p.N, nk, passes, rows)) return -1;
  const size_t out_bytes = p.out_dtype == XLA_FFI_DataType_F8E4M3FN ? 1 : 2;
  char name[64] = "";
  for (int64_t m0 = 0; m0 < p.M; m0 += rows) {
    XlaAmdFp8ScaledDot sub = p;
    sub.M = p.M - m0 < rows ? p.M - m0 : rows;
    sub.a = (const char*)p.a + (size_t)m0 * p.K;
    sub.out = (char*)p.out + (size_t)m0 * p.N * out_bytes;
    if (p.a_scale_per_row) sub.a_scale = p.a_scale + m0;
    if (mx) sub.a_block_scales = (const char*)p.a_block_scales + (size_t)m0 * (size_t)(p.K / 32);
    const int rc = LaunchFp8DotDecodeRows(sub, stream, bf16_multiply, any_scale);
    if (rc != 0) return rc;  // (-1 on the first pass: not covered; the passes differ in their row count only)
    if (!name[0]) {
      char base[48];
      snprintf(base, sizeof(base), "%s", xla_amd_last_kernel());
      if (char* bar = strchr(base, '|')) *bar = 0;
      snprintf(name, sizeof(name), "%s:x%d%s", base, (int)rows, *any_scale ? "|rounded" : "");
    }
  }
  SetLastKernel(name);
  return 0;
}

static int LaunchFp8DotDecodeRows(const XlaAmdFp8ScaledDot& p, hipStream_t stream, bool bf16_multiply, bool* any_scale) {
  const int64_t batch = p.batch > 1 ? p.batch : 1;
  const bool nk = p.rhs_contracting_dim == 1;
  const bool mx = p.a_block_scales != nullptr;
  const int align = nk ? 16 : 8;  // bytes a lane loads at once
  // (four token tiles of the [N,K] kernel do not fit the registers of two waves per SIMD: 48 rows there,
  // 32 with block scales)
  if (p.M <= 0 || p.M > (mx ? 32 : nk ? 48 : 64) || p.K <= 0 || p.K % align != 0 || p.N % 8 != 0) return -1;
  // a bf16-typed dequantise multiply: only as the caller says (for an [N,K] rhs it launches the kernels
  // that take over when a scale is no power of two); vectors of scales only on a [K,N] rhs, whose
  // rounding form then runs alone
  const bool vector_scales = p.a_scale_per_row || p.b_scale_per_channel;
  if (p.dequant_type != XLA_FFI_DataType_F32 &&
      !(bf16_multiply && p.dequant_type == XLA_FFI_DataType_BF16 && !mx && !(nk && p.M > 32)))
    return -1;
  const bool only_rounded = p.dequant_type == XLA_FFI_DataType_BF16 && vector_scales;
  // block scales: a step's four scales of a row move as one dword
  if (mx && (!nk || p.K % 128 != 0 || ((uintptr_t)p.a_block_scales % 4) || ((uintptr_t)p.b_block_scales % 4) ||
             (double)p.N * (p.K / 32) >= 2147483000.0))
    return -1;
  if (((uintptr_t)p.a % align) || ((uintptr_t)p.b % align) || (double)p.K * p.N >= 2147483000.0 || batch > 65535) return -1;
  const bool out_f8 = p.out_dtype == XLA_FFI_DataType_F8E4M3FN;
  Fp8DecodeParams dp{};
  dp.a = (const uint8_t*)p.a;
  dp.b = (const uint8_t*)p.b;
  dp.a_scale = p.a_scale;
  dp.b_scale = p.b_scale;
  dp.a_block_scales = (const uint8_t*)p.a_block_scales;
  dp.b_block_scales = (const uint8_t*)p.b_block_scales;
  dp.a_per_row = p.a_scale_per_row != 0;
  dp.b_per_channel = p.b_scale_per_channel != 0;
  dp.bias = (p.epilogue & 1) ? p.bias : nullptr;
  dp.bias_is_bf16 = p.bias_dtype == XLA_FFI_DataType_BF16;
  dp.out = out_f8 ? nullptr : (uint16_t*)p.out;
  dp.out8 = out_f8 ? (uint8_t*)p.out : nullptr;
  dp.d_scale = p.d_scale;
  dp.d_divides = p.d_scale_multiplies ? 0 : 1;
  dp.amax = out_f8 ? p.amax : nullptr;
  dp.M = (int)p.M; dp.K = (int)p.K; dp.N = (int)p.N;
  dp.bf16_dot = p.dot_type == XLA_FFI_DataType_BF16;
  dp.bf16_ops = p.epilogue_type == XLA_FFI_DataType_BF16;
  dp.epilogue = p.epilogue;
  dp.require_pow2_scales = p.dequant_type == XLA_FFI_DataType_BF16 ? 1 : 0;
  const int kStep = nk ? 128 : 32;
  int slices = Slices(batch, p.M, p.K, p.N, nk);
  const size_t need = (size_t)batch * slices * p.M * p.N * 4;
  if (slices > 1 && (!p.workspace || p.workspace_bytes < need || ((uintptr_t)p.workspace % 16))) slices = 1;
  dp.slices = slices;
  dp.partial = (float*)p.workspace;
  const int mt = (int)((p.M + 15) / 16);
  const int waves = kWaves;
  const int per = (int)((p.K + slices - 1) / slices);
  dp.rows_per_wave = ((per + waves - 1) / waves + kStep - 1) / kStep * kStep;
  dp.rows_per_slice = dp.rows_per_wave * waves;
  const int strips = (int)((p.N + 127) / 128);
  // more work items than CUs: a workgroup walks `cols` strips, as long as that leaves about 200 workgroups
  int cols = 1;
  const int64_t items = (int64_t)strips * slices * batch;
  if (items > 256) {
    const int c = (int)((items + 255) / 256);
    if ((strips + c - 1) / c * slices * batch >= 192) cols = c;
  }
  // (three token tiles of the walking [N,K] kernel spill: one strip per workgroup there)
  if (nk && !mx && mt >= 3) cols = 1;
  if (int c = GetOption("fp8_decode_cols")) cols = c;
  dp.cols = cols;
  const dim3 grid((unsigned)((strips + cols - 1) / cols * slices), (unsigned)batch);
  const dim3 block(kWaves * 64);
#define XLA_AMD_LAUNCH_FP8_DECODE(KERNEL, ...)                                                      \
  do {                                                                                              \
    if (cols > 1) hipLaunchKernelGGL((KERNEL<__VA_ARGS__, true>), grid, block, 0, stream, dp);      \
    else hipLaunchKernelGGL((KERNEL<__VA_ARGS__, false>), grid, block, 0, stream, dp);              \
  } while (0)
  if (only_rounded) {
    // (the f8 form cannot tell from one value whether a vector of scales rounds anything)
  } else if (nk && mx) {
    if (mt == 1) XLA_AMD_LAUNCH_FP8_DECODE(fp8_dot_decode_nk_kernel, 1, true);
    else XLA_AMD_LAUNCH_FP8_DECODE(fp8_dot_decode_nk_kernel, 2, true);
  } else if (nk) {
    if (mt == 1) XLA_AMD_LAUNCH_FP8_DECODE(fp8_dot_decode_nk_kernel, 1, false);
    else if (mt == 2) XLA_AMD_LAUNCH_FP8_DECODE(fp8_dot_decode_nk_kernel, 2, false);
    else XLA_AMD_LAUNCH_FP8_DECODE(fp8_dot_decode_nk_kernel, 3, false);
  } else {
    if (mt == 1) XLA_AMD_LAUNCH_FP8_DECODE(fp8_dot_decode_kn_kernel, 1);
    else if (mt == 2) XLA_AMD_LAUNCH_FP8_DECODE(fp8_dot_decode_kn_kernel, 2);
    else if (mt == 3) XLA_AMD_LAUNCH_FP8_DECODE(fp8_dot_decode_kn_kernel, 3);
    else XLA_AMD_LAUNCH_FP8_DECODE(fp8_dot_decode_kn_kernel, 4);
  }
#undef XLA_AMD_LAUNCH_FP8_DECODE
  int rc = CheckLaunch("fp8_dot_decode");
  if (rc) return rc;
  if (slices > 1 && !only_rounded) {
    dim3 fgrid((unsigned)(((size_t)p.M * p.N + 255) / 256), (unsigned)batch);
    hipLaunchKernelGGL(fp8_dot_decode_finalize_kernel, fgrid, dim3(256), 0, stream, dp);
    rc = CheckLaunch("fp8_dot_decode_finalize");
    if (rc) return rc;
  }
  // A bf16-typed multiply: the same launches again in the form that rounds the scaled operands to bf16,
  // for scales that are no powers of two (one strip per workgroup).
  if (dp.require_pow2_scales) {
    Fp8DecodeParams dr = dp;
    dr.require_pow2_scales = 0;
    dr.rounded_operands = only_rounded ? 2 : 1;
    dr.cols = 1;
    const dim3 rgrid((unsigned)(strips * slices), (unsigned)batch);
    if (nk && mt == 1) hipLaunchKernelGGL((fp8_dot_decode_nk_kernel<1, false, false, true>), rgrid, block, 0, stream, dr);
    else if (nk) hipLaunchKernelGGL((fp8_dot_decode_nk_kernel<2, false, false, true>), rgrid, block, 0, stream, dr);
    else if (mt == 1) hipLaunchKernelGGL((fp8_dot_decode_kn_kernel<1, false, true>), rgrid, block, 0, stream, dr);
    else if (mt == 2) hipLaunchKernelGGL((fp8_dot_decode_kn_kernel<2, false, true>), rgrid, block, 0, stream, dr);
    else if (mt == 3) hipLaunchKernelGGL((fp8_dot_decode_kn_kernel<3, false, true>), rgrid, block, 0, stream, dr);
    else hipLaunchKernelGGL((fp8_dot_decode_kn_kernel<4, false, true>), rgrid, block, 0, stream, dr);
    rc = CheckLaunch("fp8_dot_decode_rounded");
    if (rc) return rc;
    if (slices > 1) {
      dim3 fgrid((unsigned)(((size_t)p.M * p.N + 255) / 256), (unsigned)batch);
      hipLaunchKernelGGL(fp8_dot_decode_finalize_kernel, fgrid, dim3(256), 0, stream, dr);
      rc = CheckLaunch("fp8_dot_decode_finalize");
      if (rc) return rc;
    }
    *any_scale = true;
  }
  static const char* names[2][4] = {{"fp8_dot_decode_kn_m16", "fp8_dot_decode_kn_m32", "fp8_dot_decode_kn_m48", "fp8_dot_decode_kn_m64"},
                                    {"fp8_dot_decode_nk_m16", "fp8_dot_decode_nk_m32", "fp8_dot_decode_nk_m48", "fp8_dot_decode_nk_m64"}};
  static const char* mx_names[2] = {"fp8_dot_decode_mx_m16", "fp8_dot_decode_mx_m32"};
  char name[56];
  snprintf(name, sizeof(name), "%s%s%s", mx ? mx_names[mt - 1] : names[nk ? 1 : 0][mt - 1], cols > 1 ? ":walk" : "",
           *any_scale ? "|rounded" : "");
  SetLastKernel(name);
  return 0;
}

}  // namespace xla_amd
