// LDS-tiled MFMA dots for prefill shapes.
//
//   kFp8 : out[m,n] = epi( a_scale*b_scale * sum_k A8[m,k] * B8[n,k] )   f8e4m3fn x f8e4m3fn
//   kS8  : out[b,m,n] = epi( scale[b,n] * sum_k A[b,m,k] * W[b,k,n] )    bf16 x s8 (per channel)
//   kS4  : out[b,m,n] = epi( sum_k A[b,m,k] * bf16(W[b,k,n] * scale[b,k/g,n]) )   bf16 x s4, bf16 scales per
//          group of g rows, every dequantised weight rounded once (the bf16-typed multiply)
//   kS8NK, kS4NK : the same two with the weights stored [b,n,k] (K minor; scales [b,n] / [b,n,k/g])
//
// A workgroup of 8 waves (2x4, two per SIMD) owns a 256x256 output tile, each wave a 128x64
// part held in 128 accumulator registers, and walks K in stages of 128 bytes per activation
// row (128 fp8 or 64 bf16 values).  Both operand tiles of a stage sit in LDS with the contracting
// dimension contiguous (128-byte rows, 16-byte chunks XOR-swizzled by row so that the
// 128-bit fragment reads of 16 consecutive rows cover all 64 banks once).  The
// activation tile -- and the fp8 weight tile, stored [N,K] -- go from global memory
// straight into LDS (buffer_load ... lds: no staging registers, out-of-range rows arrive as
// zeros); the swizzle is applied by permuting which global chunk each lane fetches.  The s8
// weights are [K,N] with N minor: a lane reads 4 channels of 8 consecutive rows, converts
// (exactly) to bf16 and writes each channel's 8 values as one swizzled 16-byte chunk, so
// the transposition costs nothing beyond the convert.  Stage s+1 is in flight while stage
// s feeds the matrix cores.
//
// The 32-row MFMA operand is fed with *output channels* and the 32-column operand with
// tokens, so a lane ends up with runs of 4 consecutive channels of one token and stores
// each as one 8-byte piece of the bf16 output row.
//
// Bound: MFMA (fp8: v_mfma_f32_32x32x64_f8f6f4, bf16: v_mfma_f32_32x32x16_bf16).
// Algorithmic flops: 2*M*N*K per batch.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include <atomic>
#include <type_traits>

#include "decode_common.h"
#include "device_numerics.h"
#include "launch.h"

namespace xla_amd {
namespace {

// kFp8KN: fp8 with the weights given [K,N]; kFp8MX: fp8 [M,K] x [N,K] with one f8e8m0fnu scale per
// 32 elements of K on both operands (MXFP8), multiplied in by the matrix cores themselves
// kBf16: both operands bf16 with K minor, a [M,K] and b [N,K] -- the f8 operands of a dot whose
// dequantise multiply is bf16-typed, already scaled and rounded by a pre-pass
// kU4: kS4 with unsigned nibbles and, optionally, one u4 zero point per scale (packed like the weights).
// kS8NK, kS4NK: integer weights stored [N,K]: a thread fetches 32 consecutive k of one channel and
// writes them, dequantised, as four chunks of that channel's LDS row
enum : int { kFp8 = 0, kS8 = 1, kFp8KN = 2, kFp8MX = 3, kS4 = 4, kBf16 = 5, kS8NK = 6, kS4NK = 7, kU4 = 8 };

constexpr int kTM = 256, kTN = 256;  // output tile (tokens x channels)
constexpr int kRow = 128;            // bytes of K per LDS row per stage

struct TiledParams {
  const uint8_t* a;     // kFp8: f8 [M,K]; kS8: bf16 [batch,M,K]
  const uint8_t* b;     // kFp8: f8 [N,K]; kFp8KN: f8 [K,N]; kS8: s8 [batch,K,N]
  const float* a_scale; // kFp8: one value, or M (a_per_row)
  const float* b_scale; // kFp8: one value, or N (b_per_channel)
  const void* scales;   // kS8: [scale_batch, N]; kS4: bf16 [scale_batch, K/group, N]
  int group_shift;      // kS4: log2 of the scale group (rows of K)
  const uint8_t* zero_points;  // kU4: u4 [scale_batch, K/group, N], two per byte, or null (all zero)
  const void* bias;
  uint16_t* out;        // [batch, M, N]
  int M, K, N;
  int scale_is_bf16, bias_is_bf16, scale_batched;
  int bf16_dot, bf16_ops, epilogue;
  int tiles_m, tiles_n;
  int require_pow2_scales;  // kFp8 with a bf16-typed dequantise multiply: exact only then
  int a_per_row, b_per_channel;
  uint8_t* out8;         // kFp8 with an f8e4m3fn result: [M,N] codes (out is unused then)
  const float* d_scale;  // its per-tensor scale, a device scalar
  int d_divides;         // the value is divided by the scale (else multiplied)
  float* amax;           // optional f32 scalar result: max |v| over the f8 result's values
  const uint8_t* a_block_scales;  // kFp8MX: f8e8m0fnu [M, K/32]
  const uint8_t* b_block_scales;  // kFp8MX: f8e8m0fnu [N, K/32]
  int closed_form_epilogue;       // option "tiled_epilogue" = 1
  int skip_if_pow2_scales;        // kBf16: both scales powers of two -> the f8 kernel has done the call, return
  // Integer-weight kinds: the tiles of the last, at most half-full round of 256 are each split over
  // two workgroups along K (grid: tail_first whole tiles, then tail_tiles second halves, then
  // tail_tiles first halves; one dimension, batches flattened).  A second half leaves its f32
  // accumulators in tail_sums and raises its flag; the first half, dispatched after it, adds them
  // to its own (first half + second half) and finishes the tile.
  int tail_first, tail_tiles;
  float* tail_sums;                 // [tail_tiles][32][512] x 16 bytes
  unsigned long long* tail_flags;   // [tail_tiles] x {flag, generation}
  unsigned long long epoch;         // a raised flag holds HandOverTarget(epoch, the slot's generation)
  int handover_test;                // test aid: second halves never raise their flag, first halves give up at once
  // Integer-weight kinds, ragged dot: a is [M,K] with rows sorted by group, b [groups,K,N], out [M,N].
  // Group g owns rows [sum of the sizes before it, + its size), read on the device.  The grid holds
  // tiles_n x ragged_slots workgroups; slot s is the s-th 256-row tile counted over all groups (a
  // group of n rows has ceil(n / 256) of them), slots past the last tile return.
  const void* group_sizes;
  int group_sizes_64, ragged_groups, ragged_slots;
};

constexpr size_t kTailSumsBytes = (size_t)kTM * kTN * sizeof(float);  // per split tile

__device__ __forceinline__ float e8m0_to_f32(uint32_t e) {
  return e == 0xffu ? bits_to_f32(0x7fc00000u) : e == 0u ? bits_to_f32(0x00400000u) : bits_to_f32(e << 23);
}

__device__ __forceinline__ __amdgpu_buffer_rsrc_t tile_rsrc(const void* base, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)bytes, 0x00020000);
}

typedef __attribute__((address_space(3))) void* lds_ptr_t;

// 64 lanes x 16 bytes from the buffer into 1 KiB of LDS starting at `dst` (lane l lands at
// dst + 16*l); out-of-range lanes deposit zeros.
// Everything goes into the per-lane offset: that is the part the hardware range-checks.
constexpr uint32_t kOutOfRange = 0x80000000u;  // every buffer here is smaller than 2 GiB
__device__ __forceinline__ void load_to_lds(__amdgpu_buffer_rsrc_t r, uint8_t* dst, uint32_t voff) {
  __builtin_amdgcn_raw_ptr_buffer_load_lds(r, (lds_ptr_t)(uintptr_t)dst, 16, voff, 0, 0, 0);
}

// Read side of the staged epilogue: 16 iterations of one ds_read_b128, four epilogue values
// and an 8-byte store per lane.  The activation and the two rounding modes are template
// parameters, so the loop body is branch-free; the variant is picked once per pass.
struct DrainArgs {
  const float* stage;
  int rd_chunk, rd_row, m_base, n, M, N;
  uint16_t* out;  // start of this batch's [M,N] block
  uint8_t* out8;  // f8e4m3fn result instead (d_mode != 0)
  // 0: bf16 result; f8 result = convert(clamp(t)): 1: t = v * dz, 2: t = v / dz through the
  // shared reciprocal (dz ordinary), 3: t = v / dz by the IEEE divide
  int d_mode;
  float dz, drz, dlim;  // the scale, its reciprocal, and 1792 * dz
  bool want_amax;       // f8 result: also the largest |v| of the whole result
  bool closed_form;     // f32-typed gelu / silu from x * sigmoid(.) instead of the HLO's op sequence
  bool n_vec, has_bias;
  float sc[4], bs[4];
};

// Returns, for an f8 result, the largest |v| this lane produced as a bit pattern (NaN sorts above
// every number, which is how maximum propagates it); 0 otherwise.
template <bool BF16_DOT, bool BF16_OPS, int ACT, bool OUT_F8, bool DIRECT = false>
__device__ __forceinline__ uint32_t drain_rows(const DrainArgs& d) {
  uint32_t amax = 0u;
#pragma unroll 4
  for (int it = 0; it < 16; ++it) {
    const int ml = it * 4 + d.rd_row;
    const floatx4 x = *reinterpret_cast<const floatx4*>(d.stage + ml * 64 + ((d.rd_chunk ^ (ml & 15)) << 2));
    float v[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      const float pre = epilogue_pre<BF16_DOT, BF16_OPS>(x[t] * d.sc[t], d.bs[t], d.has_bias);
      v[t] = DIRECT ? epilogue_act_direct(pre, ACT) : epilogue_act<BF16_OPS>(pre, ACT);
    }
    const int m = d.m_base + ml;
    if (OUT_F8) {
      if (d.want_amax && m < d.M) {
#pragma unroll
        for (int t = 0; t < 4; ++t)
          if (d.n + t < d.N) amax = max(amax, f32_to_bits(v[t]) & 0x7fffffffu);
      }
      float q[4];
      bool special = d.d_mode == 3;
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        if (d.d_mode == 1) {
          q[t] = v[t] * d.dz;
        } else if (d.d_mode == 2) {
          // beyond +-1792*dz the quotient is clamped anyway; inside, the shortcut cannot overflow
          q[t] = div_by_ordinary(__builtin_amdgcn_fmed3f(v[t], -d.dlim, d.dlim), d.dz, d.drz);
        } else {
          q[t] = v[t] / d.dz;
        }
        special |= v[t] != v[t] || q[t] != q[t];
      }
      uint32_t codes;
      if (!special) {
        codes = pack_f8x4(__builtin_amdgcn_fmed3f(q[0], -448.0f, 448.0f), __builtin_amdgcn_fmed3f(q[1], -448.0f, 448.0f),
                          __builtin_amdgcn_fmed3f(q[2], -448.0f, 448.0f), __builtin_amdgcn_fmed3f(q[3], -448.0f, 448.0f));
      } else {  // NaN in or out, or a scale the shortcut does not cover: op by op, software cast
        codes = 0u;
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          float c = d.d_mode == 1 ? v[t] * d.dz : v[t] / d.dz;
          if (c == c) c = __builtin_fminf(__builtin_fmaxf(c, -448.0f), 448.0f);
          codes |= f32_to_f8e4m3fn_any(c) << (8 * t);
        }
      }
      if (m < d.M && d.n < d.N) {
        uint8_t* dst = d.out8 + (size_t)m * d.N + d.n;
        if (d.n_vec) {
          *reinterpret_cast<uint32_t*>(dst) = codes;
        } else {
#pragma unroll
          for (int t = 0; t < 4; ++t)
            if (d.n + t < d.N) dst[t] = (uint8_t)(codes >> (8 * t));
        }
      }
    } else if (m < d.M && d.n < d.N) {
      uint16_t* dst = d.out + (size_t)m * d.N + d.n;
      if (d.n_vec) {  // N % 4 == 0 and n % 4 == 0: the run of 4 is whole and 8-byte aligned
        const uintx2 o = {pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3])};
        *reinterpret_cast<uintx2*>(dst) = o;
      } else {
#pragma unroll
        for (int t = 0; t < 4; ++t)
          if (d.n + t < d.N) dst[t] = f32_to_bf16(v[t]);
      }
    }
  }
  return amax;
}

template <bool BF16_DOT, bool BF16_OPS, bool OUT_F8>
__device__ __forceinline__ uint32_t drain_act(const DrainArgs& d, int act) {
  if (!BF16_OPS && d.closed_form) {  // opt-in: f32-typed gelu / silu from their closed forms
    if (act == kEpiGelu) return drain_rows<BF16_DOT, BF16_OPS, kEpiGelu, OUT_F8, true>(d);
    if (act == kEpiSilu) return drain_rows<BF16_DOT, BF16_OPS, kEpiSilu, OUT_F8, true>(d);
  }
  switch (act) {
    case kEpiRelu: return drain_rows<BF16_DOT, BF16_OPS, kEpiRelu, OUT_F8>(d);
    case kEpiGelu: return drain_rows<BF16_DOT, BF16_OPS, kEpiGelu, OUT_F8>(d);
    case kEpiSilu: return drain_rows<BF16_DOT, BF16_OPS, kEpiSilu, OUT_F8>(d);
    default: return drain_rows<BF16_DOT, BF16_OPS, 0, OUT_F8>(d);
  }
}

template <bool OUT_F8>
__device__ __forceinline__ uint32_t drain_dispatch(const DrainArgs& d, int act, bool bf16_dot, bool bf16_ops) {
  if (OUT_F8) return drain_act<false, false, true>(d, act);  // f32-typed ops only (checked on the host)
  if (bf16_ops) {
    if (bf16_dot) drain_act<true, true, false>(d, act); else drain_act<false, true, false>(d, act);
  } else {
    if (bf16_dot) drain_act<true, false, false>(d, act); else drain_act<false, false, false>(d, act);
  }
  return 0u;
}

// SPLIT: the kernel can run tiles as two workgroups along K (tail_tiles > 0).  The integer-weight
// kinds always can; for the f8 kinds that is an instantiation of its own, because the one-workgroup
// form has no register to spare (254) for it.
template <int KIND, bool OUT_F8, bool SPLIT>
__global__ __launch_bounds__(512) void tiled_dot_kernel(TiledParams p) {
  constexpr bool WQ = KIND == kS8 || KIND == kS4 || KIND == kU4 || KIND == kS8NK || KIND == kS4NK;  // integer weights, dequantised on the way into LDS
  constexpr bool W4 = KIND == kS4 || KIND == kU4 || KIND == kS4NK;   // two weights per byte, bf16 group scales
  constexpr bool U4 = KIND == kU4;
  constexpr bool W8 = KIND == kS8 || KIND == kS8NK;   // one scale per channel, applied to the sums
  constexpr bool BB = KIND == kBf16;     // both operands bf16, K minor
  constexpr bool F8 = !WQ && !BB;        // both operands f8e4m3fn
  constexpr bool BKN = KIND == kFp8KN;   // weight tile staged K-major and transposed on the way out of LDS
  constexpr bool MX = KIND == kFp8MX;    // block scales ride along with every stage
  constexpr bool BNK = KIND == kFp8 || MX || BB;  // weights [N,K]: staged like the activations
  constexpr int ESZ = F8 ? 1 : 2;  // bytes per activation element
  constexpr int KS = kRow / ESZ;             // K elements per stage
  extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];  // [2][(kTM + kTN) * kRow]
  constexpr int kBufBytes = (kTM + kTN) * kRow;

  if (F8 && !MX && p.require_pow2_scales) {
    if (!(is_pow2_f32(*p.a_scale) && is_pow2_f32(*p.b_scale))) return;  // the bf16-operand (or the exact) kernel runs
  }
  if (BB && p.skip_if_pow2_scales) {
    if (is_pow2_f32(*p.a_scale) && is_pow2_f32(*p.b_scale)) return;
  }

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // 0..7, two per SIMD
  const int l32 = lane & 31, kb = lane >> 5;
  const int wm = wave >> 2, wn = wave & 3;  // wave tile: tokens [wm*128,+128) x channels [wn*64,+64)

  // Workgroup id -> tile: consecutive ids of one XCD take 8 neighbouring channel tiles of one
  // token tile, then the next token tile, so a token tile and 8 weight tiles stay hot in L2.
  int bid = blockIdx.x;
  int batch = blockIdx.y;
  int role = 0;       // 0: all of K; 1: second half of K, hands over; 2: first half of K, finishes
  int tail_slot = 0;
  const int tiles_per_batch = p.tiles_m * p.tiles_n;  // == gridDim.x unless the tail is split
  if (SPLIT && p.tail_tiles > 0) {
    int t = blockIdx.x;
    if (t >= p.tail_first) {
      t -= p.tail_first;
      role = t < p.tail_tiles ? 1 : 2;
      tail_slot = role == 1 ? t : t - p.tail_tiles;
      t = p.tail_first + tail_slot;
    }
    batch = t / tiles_per_batch;
    bid = t % tiles_per_batch;
  }
  const bool waited_for_tail = role == 2;  // (the role changes if the wait gives up)
  unsigned long long tail_target = 0;      // what the slot's raised flag holds in this run
  if (SPLIT && role != 0 && threadIdx.x == 0) tail_target = HandOverTarget(p.epoch, p.tail_flags + 2 * tail_slot + 1);
  const bool ragged = WQ && p.group_sizes != nullptr;
  int m0r = 0, m_limit = p.M;  // ragged: first row of the tile and the end of its group's rows
  if (ragged) {
    // consecutive ids share a row tile (and with it an activation tile in L2).  Slot s is the s-th
    // 256-row tile counted over all groups; every wave finds it with a scan over the lanes, 64 groups
    // at a time (a serial walk, one scalar load per group, cost a workgroup tens of microseconds at 64
    // groups and more).
    int g_sel, begin_sel, rows_sel, last_end;
    ragged_item<kTM, true>(p, bid / p.tiles_n, lane, &g_sel, &begin_sel, &rows_sel, &last_end);
    const bool found = g_sel >= 0;
    if (found) {
      batch = g_sel;
      m0r = begin_sel;
      m_limit = begin_sel + rows_sel;
    }
    if (!found) return;
  }
  if (!ragged) {
    const int total = tiles_per_batch;
    if (total % 8 == 0) bid = (bid % 8) * (total / 8) + bid / 8;
  }
  int tm, tn;
  if (ragged) {
    tm = 0;
    tn = bid % p.tiles_n;
  } else {
    const int G = 8;
    const int full = (p.tiles_n / G) * G;           // channel tiles covered by complete groups
    const int per_group = G * p.tiles_m;
    if (bid < (full / G) * per_group) {
      const int g = bid / per_group, r = bid % per_group;
      tn = g * G + r % G;
      tm = r / G;
    } else {
      const int r = bid - (full / G) * per_group, w = p.tiles_n - full;  // last, narrower group
      tn = full + r % w;
      tm = r / w;
    }
  }
  const int m0 = ragged ? m0r : tm * kTM, n0 = tn * kTN;
  const int a_batch = ragged ? 0 : batch;  // a ragged dot has one [M,K] activation and one [M,N] result

  const uint32_t a_pitch = (uint32_t)p.K * ESZ;
  const __amdgpu_buffer_rsrc_t ra =
      tile_rsrc(p.a + (size_t)a_batch * p.M * a_pitch, (uint32_t)p.M * a_pitch);
  const uint32_t b_bytes = W4 ? (uint32_t)(((size_t)p.K * p.N) >> 1) : (uint32_t)p.K * (uint32_t)p.N * (BB ? 2u : 1u);
  const __amdgpu_buffer_rsrc_t rb = tile_rsrc(p.b + (size_t)batch * b_bytes, b_bytes);  // bytes, either layout

  // kFp8MX: scales [rows, K/32]; lane l of wave w owns tile row (w & 3) * 64 + l of its operand
  const int nblk = p.K >> 5;
  const __amdgpu_buffer_rsrc_t rsa =
      tile_rsrc(MX ? p.a_block_scales + (size_t)batch * p.M * nblk : p.a, MX ? (uint32_t)p.M * (uint32_t)nblk : 0u);
  const __amdgpu_buffer_rsrc_t rsb =
      tile_rsrc(MX ? p.b_block_scales + (size_t)batch * p.N * nblk : p.a, MX ? (uint32_t)p.N * (uint32_t)nblk : 0u);
  const uint32_t sc_voff = (uint32_t)((wave < 4 ? m0 : n0) + (wave & 3) * 64 + lane) * (uint32_t)nblk;

  // ---- direct-to-LDS loads: one instruction moves 8 rows x 128 bytes; lane l fills slot l%8
  // of row l/8 with global chunk (l%8) ^ ((row >> 1) & 7): any 16 consecutive rows then cover
  // all 64 banks with one 16-byte chunk each, which is what ds_read_b128 needs for its full
  // rate (the hardware serves 16 lanes per clock).  Wave w owns rows [w*32, w*32+32) of a
  // 256-row tile: 4 instructions per tile per stage.
  const int ld_row = lane >> 3;                       // 0..7 within an instruction
  // rows of instruction j start at a multiple of 8: (row >> 1) & 7 == 4 * (j & 1) + ld_row / 2
  const int ld_chunk[2] = {(lane & 7) ^ (ld_row >> 1), (lane & 7) ^ (4 + (ld_row >> 1))};
  uint32_t voff_a[4], voff_b[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int r = wave * 32 + j * 8 + ld_row;
    voff_a[j] = (uint32_t)(m0 + r) * a_pitch + ld_chunk[j & 1] * 16;
    if (BNK) voff_b[j] = (uint32_t)(n0 + r) * a_pitch + ld_chunk[j & 1] * 16;  // K * ESZ bytes per row, as for a
    if (BKN) {
      // [K,N]: instruction j of this wave moves 4 rows of K x 256 channels; lane l fills slot l%16
      // of row l/16 with global chunk (l%16) ^ ((k & 7) << 1): eight consecutive rows then spread a
      // pair of neighbouring chunks over all 16 slots, which the transposing reads below need
      const int kr = wave * 16 + j * 4 + (lane >> 4);  // row of the stage (0..127)
      const int ch = (lane & 15) ^ ((kr & 7) << 1);
      const uint32_t col = (uint32_t)(n0 + ch * 16);
      voff_b[j] = col < (uint32_t)p.N ? (uint32_t)kr * (uint32_t)p.N + col : kOutOfRange;  // N % 16 == 0
    }
  }

  // ---- integer weights travel global -> registers -> (dequantised) LDS.  Two sets of registers: the
  // loads run three stages ahead of the MFMAs, the conversion one stage ahead, cut into four parts
  // that issue in the shadow of the current stage's matrix instructions (see the main loop).
  struct WSet {
    uint32_t w[8];   // the thread's weights of one stage
    uintx4 sc;       // kS4, kU4: the bf16 scales of its 8 channels
    uint32_t z;      // kU4: their zero points, one nibble each
    uint32_t nks;    // kS4NK: the scale of its 32 k
  };
  WSet ws0, ws1;
  // ---- s8 weights: a thread takes 4 channels (quad nq) of the 8 rows of block kblk
  const int w_nq = tid & 63, w_kblk = tid >> 6;
  auto s8_load = [&](int k0, WSet& w) {
    const uint32_t col = (uint32_t)(n0 + w_nq * 4);
    const uint32_t kfirst = (uint32_t)(k0 + w_kblk * 8);       // K % 8 == 0: the block is inside K or not at all
    // (one select for the block, not a branch per row: the loads sit between the matrix instructions)
    const bool live = col < (uint32_t)p.N && kfirst < (uint32_t)p.K;  // else it would alias other rows
    // the top bit puts an offset past the end of every buffer (all are smaller than 2 GiB)
    const uint32_t first = (kfirst * (uint32_t)p.N + col) | (live ? 0u : kOutOfRange);
#pragma unroll
    for (int r = 0; r < 8; ++r)
      w.w[r] = __builtin_amdgcn_raw_buffer_load_b32(rb, first + (uint32_t)r * (uint32_t)p.N, 0, 0);
  };
  auto s8_store = [&](uint8_t* bt, const WSet& w, int part) {  // part: the byte of each dword, one channel
    {
      const int e = part;
      float f[8];
#pragma unroll
      for (int r = 0; r < 8; ++r) f[r] = (float)(int8_t)((w.w[r] >> (8 * e)) & 0xffu);
      const uintx4 v = {pack_bf16x2(f[0], f[1]), pack_bf16x2(f[2], f[3]), pack_bf16x2(f[4], f[5]),
                        pack_bf16x2(f[6], f[7])};
      const int n = w_nq * 4 + e;
      *reinterpret_cast<uintx4*>(bt + n * kRow + ((w_kblk ^ ((n >> 1) & 7)) << 4)) = v;
    }
  };

  // ---- s4 weights: two per byte along N, so a dword is 8 channels of one row.  Lane l of wave w
  // takes block l >> 3 of 8 rows of octet (w & 3) * 8 + (l & 7): the four lanes of a quad read 16
  // contiguous bytes of one row (with the block index in the low lane bits instead, a quad touched
  // four rows and the kernel was 11 % slower), and the 8 lanes of a row block write 8 different
  // 16-byte chunks.  Waves 0-3 / 4-7 dequantise nibble pairs (0,4),(1,5) / (2,6),(3,7) of the same
  // dwords.  The group's 8 bf16 scales ride along.
  const int q_kblk = lane >> 3, q_oct = (wave & 3) * 8 + (lane & 7), q_half = wave >> 2;
  const uint32_t s4_pitch = (uint32_t)p.N >> 1;
  const __amdgpu_buffer_rsrc_t rsc4 =
      tile_rsrc(W4 ? (const uint8_t*)p.scales + (size_t)(p.scale_batched ? batch : 0) * (size_t)(p.K >> p.group_shift) * p.N * 2
                   : p.a,
                W4 ? (uint32_t)(p.K >> p.group_shift) * (uint32_t)p.N * 2u : 0u);
  // kU4: the zero points of the lane's 8 channels, one dword per group of rows; without zero points
  // the descriptor is empty and the loads return zero
  const bool has_zp = U4 && p.zero_points != nullptr;
  const __amdgpu_buffer_rsrc_t rzp =
      tile_rsrc(has_zp ? p.zero_points + (size_t)(p.scale_batched ? batch : 0) * (size_t)(p.K >> p.group_shift) * (p.N >> 1) : p.a,
                has_zp ? (uint32_t)(p.K >> p.group_shift) * ((uint32_t)p.N >> 1) : 0u);
  auto s4_load = [&](int k0, WSet& w) {
    const uint32_t col = (uint32_t)(n0 + q_oct * 8);
    const uint32_t kfirst = (uint32_t)(k0 + q_kblk * 8);       // K % 8 == 0: the block is inside K or not at all
    const bool live = col < (uint32_t)p.N && kfirst < (uint32_t)p.K;  // N % 8 == 0
    // (the top bit puts an offset past the end of the buffer: one select for the block, no branch per row)
    const uint32_t first = (kfirst * s4_pitch + (col >> 1)) | (live ? 0u : kOutOfRange);
#pragma unroll
    for (int r = 0; r < 8; ++r)
      w.w[r] = __builtin_amdgcn_raw_buffer_load_b32(rb, first + (uint32_t)r * s4_pitch, 0, 0);
    w.sc = __builtin_amdgcn_raw_buffer_load_b128(
        rsc4, live ? ((kfirst >> p.group_shift) * (uint32_t)p.N + col) * 2u : kOutOfRange, 0, 0);
    if constexpr (U4)
      w.z = __builtin_amdgcn_raw_buffer_load_b32(rzp, live ? ((kfirst >> p.group_shift) * (uint32_t)p.N + col) >> 1 : kOutOfRange, 0, 0);
  };
  auto s4_store = [&](uint8_t* bt, const WSet& w, int part) {  // part: (sl, hi), one channel
    typedef _Float16 halfx2 __attribute__((ext_vector_type(2)));
    {
      const int sl = part >> 1;
      // nibbles (e, e + 4), e = 2 * q_half + sl, as the f16 pair (1024 + u, 1024 + u) or, for odd
      // e, (1024 + 16 u, 1024 + 16 u), u = w + 8 (kU4: the nibble itself): see dequant_dot_decode.hip
      halfx2 pr[8];
#pragma unroll
      for (int r = 0; r < 8; ++r) {
        const uint32_t x = q_half ? w.w[r] >> 8 : w.w[r];
        pr[r] = __builtin_bit_cast(halfx2, sl ? __builtin_amdgcn_bitop3_b32(x, 0x00f000f0u, U4 ? 0x64006400u : 0x64806480u, 0x6a)
                                              : __builtin_amdgcn_bitop3_b32(x, 0x000f000fu, U4 ? 0x64006400u : 0x64086408u, 0x6a));
      }
      {
        const int hi = part & 1;
        const int e_lo = sl + 4 * hi;  // nibble index when q_half == 0; + 2 otherwise
        const uint32_t sw0 = w.sc[(e_lo) >> 1], sw1 = w.sc[(e_lo + 2) >> 1];
        const uint32_t sw = q_half ? sw1 : sw0;  // e and e + 2 have the same parity: same half of the dword
        const float v = (e_lo & 1) ? bf16hi_to_f32(sw) : bf16lo_to_f32(sw);
        const float sj = sl ? v * 0.0625f : v;
        float cj = sl ? v * -72.0f : v * -1032.0f;
        if constexpr (U4) {
          // the zero point in place of the 8: -(1024 + z) s, or -(64 + z) s next to 1024 + 16 u (exact in f32)
          const float z = (float)((w.z >> (4 * (e_lo + 2 * q_half))) & 0xfu);
          cj = v * (sl ? -64.0f - z : -1024.0f - z);
        }
        float f[8];
#pragma unroll
        for (int r = 0; r < 8; ++r) f[r] = __builtin_fmaf((float)pr[r][hi], sj, cj);
        const uintx4 o = {pack_bf16x2(f[0], f[1]), pack_bf16x2(f[2], f[3]), pack_bf16x2(f[4], f[5]),
                          pack_bf16x2(f[6], f[7])};
        const int n = q_oct * 8 + e_lo + 2 * q_half;
        *reinterpret_cast<uintx4*>(bt + n * kRow + ((q_kblk ^ ((n >> 1) & 7)) << 4)) = o;
      }
    }
  };
  // ---- weights stored [N,K].  s4: thread t takes channel t >> 1 and the half t & 1 of the stage's 64 k,
  // 16 contiguous bytes that become chunks 4 * half ... + 3 of the channel's LDS row.  s8: thread t
  // takes the 16-byte piece t & 3 of channels t >> 2 and (t >> 2) + 128 -- the four lanes of a quad
  // read the 64 contiguous bytes of one channel -- and each piece becomes chunks 2 * piece, + 1.
  // (K % 32 == 0 for s4 and % 16 for s8: a 16-byte piece lies inside its row or past it.)
  const int nk_n = KIND == kS8NK ? tid >> 2 : tid >> 1, nk_half = tid & 1, nk_piece = tid & 3;
  auto nk_load = [&](int k0, WSet& w) {
    const uint32_t ch = (uint32_t)(n0 + nk_n);
    const uint32_t k = (uint32_t)(k0 + nk_half * 32);
    if constexpr (KIND == kS8NK) {
      const uint32_t kp = (uint32_t)(k0 + nk_piece * 16);
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const uint32_t cj = ch + 128u * j;
        const bool live = cj < (uint32_t)p.N && kp < (uint32_t)p.K;
        const uintx4 v = __builtin_amdgcn_raw_buffer_load_b128(rb, live ? cj * (uint32_t)p.K + kp : kOutOfRange, 0, 0);
        w.w[4 * j] = v[0]; w.w[4 * j + 1] = v[1]; w.w[4 * j + 2] = v[2]; w.w[4 * j + 3] = v[3];
      }
    } else {
      const bool live = ch < (uint32_t)p.N && k < (uint32_t)p.K;
      const uintx4 v = __builtin_amdgcn_raw_buffer_load_b128(rb, live ? (ch * (uint32_t)p.K + k) >> 1 : kOutOfRange, 0, 0);
      w.w[0] = v[0]; w.w[1] = v[1]; w.w[2] = v[2]; w.w[3] = v[3];
      // the lane's 32 k share a scale (groups of at least 32, or one scale per channel: shift 31)
      w.nks = (uint32_t)(uint16_t)__builtin_amdgcn_raw_buffer_load_b16(
          rsc4, live ? (ch * (uint32_t)(p.K >> p.group_shift) + (k >> p.group_shift)) * 2u : kOutOfRange, 0, 0);
    }
  };
  auto nk_store = [&](uint8_t* bt, const WSet& w, int part) {  // part: one 16-byte chunk of the row
    {
      const int c = part;
      float f[8];
      if constexpr (KIND == kS8NK) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          f[e] = (float)(int8_t)((w.w[2 * c] >> (8 * e)) & 0xffu);
          f[4 + e] = (float)(int8_t)((w.w[2 * c + 1] >> (8 * e)) & 0xffu);
        }
      } else {
        typedef _Float16 halfx2 __attribute__((ext_vector_type(2)));
        // nibble pairs (0,4), (1,5) of x and (2,6), (3,7) of x >> 8 as f16 1024 + u or 1024 + 16 u,
        // u = w + 8; one fma each takes the offset out and the scale in: see dequant_dot_decode.hip
        const uint32_t x = w.w[c];
        const float v = bf16lo_to_f32(w.nks);
        const float s_even = v, c_even = v * -1032.0f, s_odd = v * 0.0625f, c_odd = v * -72.0f;
        const halfx2 p04 = __builtin_bit_cast(halfx2, __builtin_amdgcn_bitop3_b32(x, 0x000f000fu, 0x64086408u, 0x6a));
        const halfx2 p15 = __builtin_bit_cast(halfx2, __builtin_amdgcn_bitop3_b32(x, 0x00f000f0u, 0x64806480u, 0x6a));
        const halfx2 p26 = __builtin_bit_cast(halfx2, __builtin_amdgcn_bitop3_b32(x >> 8, 0x000f000fu, 0x64086408u, 0x6a));
        const halfx2 p37 = __builtin_bit_cast(halfx2, __builtin_amdgcn_bitop3_b32(x >> 8, 0x00f000f0u, 0x64806480u, 0x6a));
        f[0] = __builtin_fmaf((float)p04[0], s_even, c_even);
        f[1] = __builtin_fmaf((float)p15[0], s_odd, c_odd);
        f[2] = __builtin_fmaf((float)p26[0], s_even, c_even);
        f[3] = __builtin_fmaf((float)p37[0], s_odd, c_odd);
        f[4] = __builtin_fmaf((float)p04[1], s_even, c_even);
        f[5] = __builtin_fmaf((float)p15[1], s_odd, c_odd);
        f[6] = __builtin_fmaf((float)p26[1], s_even, c_even);
        f[7] = __builtin_fmaf((float)p37[1], s_odd, c_odd);
      }
      const uintx4 o = {pack_bf16x2(f[0], f[1]), pack_bf16x2(f[2], f[3]), pack_bf16x2(f[4], f[5]),
                        pack_bf16x2(f[6], f[7])};
      // s8: dwords (2c, 2c + 1) are half c & 1 of the piece of channel nk_n + 128 * (c >> 1)
      const int row = KIND == kS8NK ? nk_n + 128 * (c >> 1) : nk_n;
      const int chunk = KIND == kS8NK ? nk_piece * 2 + (c & 1) : nk_half * 4 + c;
      *reinterpret_cast<uintx4*>(bt + row * kRow + ((chunk ^ ((row >> 1) & 7)) << 4)) = o;
    }
  };
  auto wq_store = [&](uint8_t* bt, const WSet& w, int part) {
    if constexpr (KIND == kS8) s8_store(bt, w, part);
    if constexpr (KIND == kS4 || KIND == kU4) s4_store(bt, w, part);
    if constexpr (KIND == kS8NK || KIND == kS4NK) nk_store(bt, w, part);
  };
  auto wq_load = [&](int k0, WSet& w) {  // k0 past K: every load lands as zeros without touching memory
    if constexpr (KIND == kS8) s8_load(k0, w);
    if constexpr (KIND == kS4 || KIND == kU4) s4_load(k0, w);
    if constexpr (KIND == kS8NK || KIND == kS4NK) nk_load(k0, w);
  };

  auto issue_loads = [&](int buf, int k0) {
    uint8_t* at = lds + buf * kBufBytes;
    uint8_t* bt = at + kTM * kRow;
    const uint32_t kbyte = (uint32_t)k0 * ESZ;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const bool past_k = kbyte + ld_chunk[j & 1] * 16 >= a_pitch;  // chunks past K must read as 0
      load_to_lds(ra, at + (wave * 32 + j * 8) * kRow, past_k ? kOutOfRange : voff_a[j] + kbyte);
      if (BNK)
        load_to_lds(rb, bt + (wave * 32 + j * 8) * kRow, past_k ? kOutOfRange : voff_b[j] + kbyte);
      if (BKN) {
        // rows k0 + kr; a row past K lies past the end of the buffer by itself
        const uint32_t v = voff_b[j] == kOutOfRange ? kOutOfRange : voff_b[j] + (uint32_t)k0 * (uint32_t)p.N;
        load_to_lds(rb, bt + (wave * 16 + j * 4) * 256, v);
      }
    }
    if (MX) {
      // the stage's four scale bytes of every tile row, one dword per row: waves 0-3 fetch the
      // 256 token rows, waves 4-7 the 256 channel rows (64 lanes x 4 bytes land contiguously)
      const uint32_t blk = (uint32_t)k0 >> 5;
      const uint32_t v = blk < (uint32_t)nblk ? sc_voff + blk : kOutOfRange;  // K % 128 == 0
      __builtin_amdgcn_raw_ptr_buffer_load_lds(wave < 4 ? rsa : rsb, (lds_ptr_t)(uintptr_t)(lds + 2 * kBufBytes + buf * 2048 + wave * 256),
                                               4, v, 0, 0, 0);
    }
  };

  floatx16 acc[2][4];
#pragma unroll
  for (int x = 0; x < 2; ++x)
#pragma unroll
    for (int y = 0; y < 4; ++y)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[x][y][v] = 0.0f;

  // ---- main loop.  A stage is NKS MFMA steps of 8 MFMAs per wave; a step reads its six
  // fragments (4 token tiles, 2 channel tiles) and multiplies.  Nothing is software-pipelined
  // inside a wave: the two waves of a SIMD alternate, one multiplying while the other's LDS
  // reads are in flight.  Once per stage, between the reads and the MFMAs of its last step,
  // the workgroup synchronises: every wave's reads of the stage buffer are complete (so it
  // may be refilled) and the next stage's tiles have landed.  The refill for stage s+2 is
  // issued right behind that barrier, interleaved with the MFMAs.
  constexpr int NKS = F8 ? 2 : 4;
  const int frag_sw = (l32 >> 1) & 7;  // tile rows of a fragment start at multiples of 32
  const int row_a = (wm * 128 + l32) * kRow, row_b = kTM * kRow + (wn * 64 + l32) * kRow;
  typedef typename std::conditional<F8, intx8, bf16x8>::type frag_t;
  frag_t fa[4], fb[2];
  int sa_e[4] = {0, 0, 0, 0}, sb_e[2] = {0, 0};  // kFp8MX: f8e8m0fnu scale of each fragment
  // kFp8KN: per-lane parts of the transposing reads' addresses (see read_frags)
  const int tr_m = (lane & 15) >> 1, tr_par = lane & 1, tr_g = (lane >> 4) & 1;
  const int bkn_base = (32 * kb + tr_m) * 256 + 8 * tr_par;
  const int bkn_cx[2] = {((wn * 4 + 0 + tr_g) ^ (tr_m << 1)) << 4, ((wn * 4 + 2 + tr_g) ^ (tr_m << 1)) << 4};
  auto read_frags = [&](int buf, int ks) {
    const uint8_t* at = lds + buf * kBufBytes + row_a;
    const uint8_t* bt = lds + buf * kBufBytes + row_b;
    if constexpr (F8) {
      // The matrix core applies the scale handed in by lanes 0-31 to the first 16 bytes of every
      // lane of the row and the one from lanes 32-63 to the second 16 (measured; without scales
      // any split of the 64 k works as long as both operands use the same).  So with block scales
      // a lane takes 16 bytes of each of the step's two 32-element blocks, otherwise 32 in a run.
      const int c0 = ((MX ? 4 * ks + kb : 4 * ks + 2 * kb) ^ frag_sw) << 4;
      const int c1 = ((MX ? 4 * ks + 2 + kb : 4 * ks + 2 * kb + 1) ^ frag_sw) << 4;
      auto rd = [&](const uint8_t* base) {
        const uintx4 x0 = *reinterpret_cast<const uintx4*>(base + c0);
        const uintx4 x1 = *reinterpret_cast<const uintx4*>(base + c1);
        return intx8{(int)x0[0], (int)x0[1], (int)x0[2], (int)x0[3], (int)x1[0], (int)x1[1], (int)x1[2], (int)x1[3]};
      };
      if constexpr (BKN) {
        // Weight tile [k][256 channels] in LDS, read with the transposing 64-bit load: in every
        // group of 16 lanes, lane i hands in the address of 8 bytes (row i of a 16x8 block) and
        // lane j receives column j of the even rows (j < 8) or column j-8 of the odd rows.  Even
        // lanes point at 8 consecutive k of one channel octet, odd lanes at the same k of the next
        // octet, so the 16 lanes end up with 8 consecutive k of 16 consecutive channels: the MFMA
        // operand layout.  Four such loads give a lane its 32 values of k.
        typedef int intx2 __attribute__((ext_vector_type(2)));
        typedef __attribute__((address_space(3))) intx2* tr_ptr_t;
        const uint8_t* wt = lds + buf * kBufBytes + kTM * kRow + bkn_base + ks * (64 * 256);
        auto rdt = [&](int nt) {
          intx2 q[4];
#pragma unroll
          for (int i = 0; i < 4; ++i)
            q[i] = __builtin_amdgcn_ds_read_tr8_b64_v2i32((tr_ptr_t)(uintptr_t)(wt + bkn_cx[nt] + i * (8 * 256)));
          return intx8{q[0][0], q[0][1], q[1][0], q[1][1], q[2][0], q[2][1], q[3][0], q[3][1]};
        };
        fb[0] = rdt(0);
        fa[0] = rd(at);
        fb[1] = rdt(1);
      } else {
        fb[0] = rd(bt);
        fa[0] = rd(at);
        fb[1] = rd(bt + 32 * kRow);
      }
#pragma unroll
      for (int t = 1; t < 4; ++t) fa[t] = rd(at + t * 32 * kRow);
      if constexpr (MX) {
        // Lanes 0-31 hand in the scale of block 2*ks of the stage, lanes 32-63 that of block
        // 2*ks + 1.  A row's four bytes are read once per stage and shifted by the lane's half, so
        // that byte 0 serves step 0 and byte 2 step 1 (picked by the instruction's op_sel).
        if (ks == 0) {
          const uint32_t* sc = reinterpret_cast<const uint32_t*>(lds + 2 * kBufBytes + buf * 2048);
#pragma unroll
          for (int t = 0; t < 4; ++t) sa_e[t] = (int)(sc[wm * 128 + t * 32 + l32] >> (8 * kb));
#pragma unroll
          for (int t = 0; t < 2; ++t) sb_e[t] = (int)(sc[256 + wn * 64 + t * 32 + l32] >> (8 * kb));
        }
      }
    } else {
      const int c = ((2 * ks + kb) ^ frag_sw) << 4;
      fb[0] = *reinterpret_cast<const bf16x8*>(bt + c);
      fa[0] = *reinterpret_cast<const bf16x8*>(at + c);
      fb[1] = *reinterpret_cast<const bf16x8*>(bt + 32 * kRow + c);
#pragma unroll
      for (int t = 1; t < 4; ++t) fa[t] = *reinterpret_cast<const bf16x8*>(at + t * 32 * kRow + c);
    }
  };
  auto mfma_all = [&](int ks) {
#pragma unroll
    for (int mt = 0; mt < 4; ++mt)
#pragma unroll
      for (int nt = 0; nt < 2; ++nt) {
        if constexpr (MX) {
          if (ks == 0)
            acc[nt][mt] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fb[nt], fa[mt], acc[nt][mt], 0, 0, 0, sb_e[nt],
                                                                           0, sa_e[mt]);
          else
            acc[nt][mt] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fb[nt], fa[mt], acc[nt][mt], 0, 0, 2, sb_e[nt],
                                                                           2, sa_e[mt]);
        } else if constexpr (F8)
          acc[nt][mt] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fb[nt], fa[mt], acc[nt][mt], 0, 0, 0, 0, 0, 0);
        else
          acc[nt][mt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb[nt], fa[mt], acc[nt][mt], 0, 0, 0);
      }
  };

  const int stages = (p.K + KS - 1) / KS;
  const int half = (stages + 1) >> 1;
  int s_begin = role == 1 ? half : 0, s_end = role == 2 ? half : stages;
  bool add_sums = false;
  __shared__ int tail_arrived;
  // Integer-weight kinds: VMEM instructions of one stage's weight loads (the wait in front of the
  // stage barrier lets exactly those stay in flight)
  constexpr int kWLoads = KIND == kS8 ? 8 : KIND == kS4 ? 9 : KIND == kU4 ? 10 : 2;
  constexpr int kPastK = 0x40000000;  // a k0 no matrix reaches: the weight loads of such a stage fetch nothing
  for (;;) {
    if constexpr (WQ) {
      // Weights: loaded three stages ahead into one of two register sets, dequantised into the other
      // stage buffer one stage ahead, a quarter of the conversion behind each of the current stage's
      // first three MFMA steps (the last quarter rides with the third), where its VALU instructions
      // issue while the matrix pipe works.  Activations: DMA two stages ahead, as for the f8 kinds.
      uint8_t* const wt0 = lds + kTM * kRow;
      uint8_t* const wt1 = lds + kBufBytes + kTM * kRow;
      issue_loads(0, s_begin * KS);
      wq_load(s_begin * KS, ws0);
#pragma unroll
      for (int part = 0; part < 4; ++part) wq_store(wt0, ws0, part);
      asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
      __syncthreads();
      issue_loads(1, (s_begin + 1) * KS);  // past K: lands as zeros, never read
      __builtin_amdgcn_sched_barrier(0);   // the activation loads stay older than the weight loads
      wq_load(s_begin + 1 < s_end ? (s_begin + 1) * KS : kPastK, ws1);
      wq_load(s_begin + 2 < s_end ? (s_begin + 2) * KS : kPastK, ws0);
      auto stage = [&](int buf, uint8_t* wt_next, WSet& set, int s) __attribute__((always_inline)) {
        read_frags(buf, 0);
        mfma_all(0);
        wq_store(wt_next, set, 0);
        read_frags(buf, 1);
        mfma_all(1);
        wq_store(wt_next, set, 1);
        read_frags(buf, 2);
        mfma_all(2);
        wq_store(wt_next, set, 2);
        wq_store(wt_next, set, 3);
        read_frags(buf, 3);
        // the next stage's activations have landed (the weight loads issued after them may still fly),
        // this wave's LDS reads and writes are done
        asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"(kWLoads) : "memory");
        __syncthreads();
        issue_loads(buf, (s + 2) * KS);  // past this workgroup's stages in the last rounds: into a buffer nobody reads
        __builtin_amdgcn_sched_barrier(0);
        wq_load(s + 3 < s_end ? (s + 3) * KS : kPastK, set);
        mfma_all(3);
      };
      int s = s_begin;
      for (; s + 2 < s_end; s += 2) {
        stage(0, wt1, ws1, s);
        stage(1, wt0, ws0, s + 1);
      }
      if (s + 1 < s_end) {
        stage(0, wt1, ws1, s);
        ++s;
      }
      {  // last stage: nothing left to fetch or convert
        const int buf = (s - s_begin) & 1;
#pragma unroll
        for (int ks = 0; ks < NKS; ++ks) {
          read_frags(buf, ks);
          mfma_all(ks);
        }
      }
    } else {
      issue_loads(0, s_begin * KS);
      asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
      __syncthreads();
      issue_loads(1, (s_begin + 1) * KS);  // past K: lands as zeros, never read
      for (int s = s_begin; s + 1 < s_end; ++s) {
        const int buf = (s - s_begin) & 1;
#pragma unroll
        for (int ks = 0; ks + 1 < NKS; ++ks) {
          read_frags(buf, ks);
          mfma_all(ks);
        }
        read_frags(buf, NKS - 1);
        asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
        __syncthreads();
        issue_loads(buf, (s + 2) * KS);  // past this workgroup's stages in the last rounds: into a buffer nobody reads
        mfma_all(NKS - 1);
        if (F8) {
#pragma unroll
          for (int i = 0; i < 8; ++i) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // one MFMA
            __builtin_amdgcn_sched_group_barrier(0x010, 1, 0);  // one buffer load
          }
        }
      }
      {  // last stage: nothing left to fetch
        const int buf = (s_end - 1 - s_begin) & 1;
#pragma unroll
        for (int ks = 0; ks < NKS; ++ks) {
          read_frags(buf, ks);
          mfma_all(ks);
        }
      }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the loads issued past the end have landed
    __syncthreads();  // the epilogue (or another pass of this loop) reuses the stage buffers
    if (!SPLIT || role != 2) break;
    // first half done: wait (bounded) for the second half's flag.  That workgroup has a lower id,
    // so it was dispatched before this one and is running or done.
    if (tid == 0) {
      int ok = 0;
      const int spins = p.handover_test ? kHandOverTestSpins : kHandOverSpins;
      for (int spin = 0; spin < spins; ++spin) {
        if (__hip_atomic_load(p.tail_flags + 2 * tail_slot, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == tail_target) { ok = 1; break; }
        __builtin_amdgcn_s_sleep(4);
      }
      tail_arrived = ok;
    }
    __syncthreads();
    if (tail_arrived) { add_sums = true; break; }
    // the flag never showed: this workgroup does the second half as well, in K order
    role = 0;
    s_begin = half;
    s_end = stages;
  }
  constexpr int kDeviceScope = 16;  // sc1: performed where every XCD sees it
  const __amdgpu_buffer_rsrc_t rt =
      tile_rsrc(reinterpret_cast<const uint8_t*>(p.tail_sums) + (size_t)tail_slot * kTailSumsBytes,
                SPLIT && (role == 1 || add_sums) ? (uint32_t)kTailSumsBytes : 0u);
  if (SPLIT && role == 1) {
#pragma unroll
      for (int nt = 0; nt < 2; ++nt)
#pragma unroll
        for (int mt = 0; mt < 4; ++mt)
#pragma unroll
          for (int vq = 0; vq < 4; ++vq) {
            const floatx16& a = acc[nt][mt];
            __builtin_amdgcn_raw_buffer_store_b128(
                uintx4{f32_to_bits(a[vq * 4]), f32_to_bits(a[vq * 4 + 1]), f32_to_bits(a[vq * 4 + 2]), f32_to_bits(a[vq * 4 + 3])},
                rt, (uint32_t)((((nt * 4 + mt) * 4 + vq) * 512 + tid) * 16), 0, kDeviceScope);
          }
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      __syncthreads();
      if (tid == 0 && !p.handover_test)
        __hip_atomic_store(p.tail_flags + 2 * tail_slot, tail_target, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      return;
  }

  // ---- epilogue, staged through LDS (free now: every wave passed the last barrier).
  // Register v of tile (nt, mt) in lane (l32, kb) is token mt*32 + l32, channel
  // nt*32 + (v/4)*8 + kb*4 + v%4 of the wave's 128x64 tile.  Each wave owns 16 KiB of LDS and
  // handles 64 tokens per pass: it writes them as [64 tokens][16 chunks of 4 f32] (chunks
  // XOR-swizzled by token), then reads the block back with 16 lanes per token row, so that a
  // row leaves as 128 contiguous bytes of bf16 and the accumulators are only ever indexed
  // statically.  The rolled read loop carries the epilogue.
  float alpha = 1.0f;
  if (F8 && !MX) alpha = (p.a_per_row ? 1.0f : *p.a_scale) * (p.b_per_channel ? 1.0f : *p.b_scale);
  float* stage = reinterpret_cast<float*>(lds + wave * 16384);
  const int rd_chunk = lane & 15, rd_row = lane >> 4;  // read side: chunk of 4 channels, row within 4
  const bool n_vec = (p.N & 3) == 0;
  // channels of this lane on the read side: the same in both passes
  const int n = n0 + wn * 64 + rd_chunk * 4;
  DrainArgs d;
#pragma unroll
  for (int t = 0; t < 4; ++t) {
    const bool ok = n + t < p.N;
    d.sc[t] = alpha;
    if (F8 && !MX && p.b_per_channel) d.sc[t] = alpha * p.b_scale[ok ? n + t : 0];
    if (W8) {
      const size_t si = (size_t)(p.scale_batched ? batch : 0) * p.N + (ok ? n + t : 0);
      d.sc[t] = p.scale_is_bf16 ? bf16_to_f32(((const uint16_t*)p.scales)[si]) : ((const float*)p.scales)[si];
    }
    d.bs[t] = 0.0f;
    if (p.bias) {
      const int bi = ok ? n + t : 0;
      d.bs[t] = p.bias_is_bf16 ? bf16_to_f32(((const uint16_t*)p.bias)[bi]) : ((const float*)p.bias)[bi];
    }
  }
  d.stage = stage;
  d.rd_chunk = rd_chunk;
  d.rd_row = rd_row;
  d.n = n;
  d.M = m_limit;  // rows from here on belong to the next group (or lie past M): computed, never stored
  d.N = p.N;
  d.out = p.out + (size_t)a_batch * p.M * p.N;
  d.out8 = nullptr;
  d.want_amax = OUT_F8 && p.amax != nullptr;
  d.closed_form = p.closed_form_epilogue != 0;
  uint32_t amax_bits = 0u;
  d.d_mode = 0;
  d.dz = d.drz = d.dlim = 1.0f;
  if (OUT_F8) {
    d.out8 = p.out8 + (size_t)batch * p.M * p.N;
    d.dz = *p.d_scale;
    d.drz = 1.0f / d.dz;
    d.dlim = 1792.0f * d.dz;
    d.d_mode = !p.d_divides ? 1 : ordinary_divisor(d.dz) ? 2 : 3;
  }
  d.n_vec = n_vec;
  d.has_bias = p.bias != nullptr;
  float row_scale[4] = {1.0f, 1.0f, 1.0f, 1.0f};
  if (F8 && !MX && p.a_per_row) {
    // one scale per token row: all 16 registers of a tile belong to the lane's one token
#pragma unroll
    for (int mt = 0; mt < 4; ++mt) {
      const int m = m0 + wm * 128 + mt * 32 + l32;
      const float rs = p.a_scale[m < p.M ? m : p.M - 1];
      row_scale[mt] = rs;
#pragma unroll
      for (int nt = 0; nt < 2; ++nt) acc[nt][mt] *= rs;
    }
  }
#pragma unroll
  for (int pass = 0; pass < 2; ++pass) {
    if (SPLIT && add_sums) {
      // the other half of K: a pass's 16 chunks are fetched together (8 and 8 by the f8 kinds, which
      // have fewer registers free) and added on the way into LDS (first half + second half), so the
      // accumulators themselves are never rewritten (with one scale per row of a the accumulators
      // already carry it and the fetched sums take it here)
      auto fetch = [&](int mtl, uintx4 (&o)[2][4]) {
#pragma unroll
        for (int nt = 0; nt < 2; ++nt)
#pragma unroll
          for (int vq = 0; vq < 4; ++vq)
            o[nt][vq] = __builtin_amdgcn_raw_buffer_load_b128(
                rt, (uint32_t)((((nt * 4 + pass * 2 + mtl) * 4 + vq) * 512 + tid) * 16), 0, kDeviceScope);
      };
      auto add_and_stage = [&](int mtl, const uintx4 (&o)[2][4]) {
        const int m = mtl * 32 + l32;
        const float rs = F8 && !MX ? row_scale[pass * 2 + mtl] : 1.0f;
#pragma unroll
        for (int nt = 0; nt < 2; ++nt) {
#pragma unroll
          for (int vq = 0; vq < 4; ++vq) {
            const int c = nt * 8 + vq * 2 + kb;
            const floatx16& a = acc[nt][pass * 2 + mtl];
            const uintx4& q = o[nt][vq];
            const floatx4 v = {a[vq * 4] + bits_to_f32(q[0]) * rs, a[vq * 4 + 1] + bits_to_f32(q[1]) * rs,
                               a[vq * 4 + 2] + bits_to_f32(q[2]) * rs, a[vq * 4 + 3] + bits_to_f32(q[3]) * rs};
            *reinterpret_cast<floatx4*>(stage + m * 64 + ((c ^ (m & 15)) << 2)) = v;
          }
        }
      };
      if constexpr (WQ) {
        uintx4 o0[2][4], o1[2][4];
        fetch(0, o0);
        fetch(1, o1);
        add_and_stage(0, o0);
        add_and_stage(1, o1);
      } else {
        uintx4 o[2][4];
        fetch(0, o);
        add_and_stage(0, o);
        __builtin_amdgcn_sched_barrier(0);
        fetch(1, o);
        add_and_stage(1, o);
      }
    } else {
#pragma unroll
      for (int mtl = 0; mtl < 2; ++mtl) {
        const int m = mtl * 32 + l32;
#pragma unroll
        for (int nt = 0; nt < 2; ++nt) {
#pragma unroll
          for (int vq = 0; vq < 4; ++vq) {
            const int c = nt * 8 + vq * 2 + kb;
            const floatx16& a = acc[nt][pass * 2 + mtl];
            const floatx4 v = {a[vq * 4], a[vq * 4 + 1], a[vq * 4 + 2], a[vq * 4 + 3]};
            *reinterpret_cast<floatx4*>(stage + m * 64 + ((c ^ (m & 15)) << 2)) = v;
          }
        }
      }
    }
    d.m_base = m0 + wm * 128 + pass * 64;
    amax_bits = max(amax_bits, drain_dispatch<OUT_F8>(d, p.epilogue & ~1, p.bf16_dot, p.bf16_ops));
  }
  // the slot moves on to its next generation, whether the flag showed or not: the next run (also a
  // replay of this launch from a captured graph) waits for new sums
  if (SPLIT && waited_for_tail && tid == 0) HandOverNextGeneration(p.tail_flags + 2 * tail_slot + 1, tail_target);
  if (OUT_F8 && p.amax) {  // one atomic per wave into the result a fill kernel zeroed
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) amax_bits = max(amax_bits, (uint32_t)__shfl_xor((int)amax_bits, off));
    if (lane == 0) atomicMax(reinterpret_cast<unsigned*>(p.amax), amax_bits);
  }
}

// [K,N] -> [N,K] byte transpose through a 64x64 LDS tile (fp8 rhs given with N minor).
__global__ __launch_bounds__(256) void transpose_bytes_kernel(const uint8_t* __restrict__ src,
                                                              uint8_t* __restrict__ dst, int K, int N) {
  __shared__ uint8_t tile[64][64 + 4];
  const int k0 = blockIdx.y * 64, n0 = blockIdx.x * 64;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  for (int r = ty; r < 64; r += 4) {
    const int k = k0 + r, n = n0 + tx;
    tile[r][tx] = (k < K && n < N) ? src[(size_t)k * N + n] : 0;
  }
  __syncthreads();
  for (int r = ty; r < 64; r += 4) {
    const int n = n0 + r, k = k0 + tx;
    if (n < N && k < K) dst[(size_t)n * K + k] = tile[tx][r];
  }
}

// [K,N] -> [N,K] byte transpose, 128x128 tiles, for N % 4 == 0, K % 16 == 0 and aligned
// pointers.  A thread reads 4 rows x 4 bytes (lanes along N: 128 contiguous bytes per row and
// half wave), transposes the 4x4 block with byte permutes, and parks the four column dwords in
// LDS as [n][k/4], the dword index XOR-swizzled by n/4 so the 32 lanes of a row group hit 32
// banks.  Then two threads per output row gather its 32 dwords and store 128 contiguous bytes.
__global__ __launch_bounds__(256) void transpose_bytes_fast_kernel(const uint8_t* __restrict__ src,
                                                                   uint8_t* __restrict__ dst, int K, int N) {
  __shared__ uint32_t tile[128 * 32];
  const int k0 = blockIdx.y * 128, n0 = blockIdx.x * 128;
  const int tid = threadIdx.x;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int b = tid + 256 * i, nb = b & 31, kb = b >> 5;
    uint32_t r[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int k = k0 + 4 * kb + q, n = n0 + 4 * nb;
      r[q] = (k < K && n < N) ? *reinterpret_cast<const uint32_t*>(src + (size_t)k * N + n) : 0u;
    }
    // bytes of v_perm's pool: 0-3 = second operand, 4-7 = first operand
    const uint32_t a01 = __builtin_amdgcn_perm(r[1], r[0], 0x05010400u);  // r0b0 r1b0 r0b1 r1b1
    const uint32_t c01 = __builtin_amdgcn_perm(r[1], r[0], 0x07030602u);  // r0b2 r1b2 r0b3 r1b3
    const uint32_t a23 = __builtin_amdgcn_perm(r[3], r[2], 0x05010400u);
    const uint32_t c23 = __builtin_amdgcn_perm(r[3], r[2], 0x07030602u);
    const uint32_t col[4] = {__builtin_amdgcn_perm(a23, a01, 0x05040100u), __builtin_amdgcn_perm(a23, a01, 0x07060302u),
                             __builtin_amdgcn_perm(c23, c01, 0x05040100u), __builtin_amdgcn_perm(c23, c01, 0x07060302u)};
#pragma unroll
    for (int j = 0; j < 4; ++j) tile[(4 * nb + j) * 32 + (kb ^ nb)] = col[j];
  }
  __syncthreads();
  const int n = tid >> 1, half = tid & 1;
  if (n0 + n >= N) return;
  uint8_t* out = dst + (size_t)(n0 + n) * K + k0 + half * 64;
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    uintx4 v;
#pragma unroll
    for (int e = 0; e < 4; ++e) v[e] = tile[n * 32 + ((half * 16 + q * 4 + e) ^ (n >> 2))];
    if (k0 + half * 64 + q * 16 < K) *reinterpret_cast<uintx4*>(out + q * 16) = v;  // K % 16 == 0
  }
}

// Exact, slow f8 scaled dot for scales that are not powers of two under a bf16-typed
// dequantise multiply: each operand value is rounded to bf16 after its scale, as the HLO does.
__global__ __launch_bounds__(256) void fp8_dot_exact_kernel(TiledParams p, int b_is_nk, int deq_bf16,
                                                            int only_if_not_pow2) {
  if (only_if_not_pow2 && is_pow2_f32(*p.a_scale) && is_pow2_f32(*p.b_scale)) return;
  const size_t total = (size_t)p.M * p.N;
  // one batch per blockIdx.y
  p.a += (size_t)blockIdx.y * p.M * p.K;
  p.b += (size_t)blockIdx.y * p.K * p.N;
  if (p.out) p.out += (size_t)blockIdx.y * total;
  if (p.out8) p.out8 += (size_t)blockIdx.y * total;
  const bool mx = p.a_block_scales != nullptr;
  const int nblk = p.K >> 5;
  if (mx) {
    p.a_block_scales += (size_t)blockIdx.y * p.M * nblk;
    p.b_block_scales += (size_t)blockIdx.y * p.N * nblk;
  }
  // the grid is bounded (a call that returns at the first line costs a few workgroups, not one
  // per 256 outputs): each workgroup strides over the outputs
  for (size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x; idx < total; idx += (size_t)gridDim.x * 256) {
    const int n = (int)(idx % p.N), m = (int)(idx / p.N);
    float sa = 1.0f, sb = 1.0f;
    if (!mx) { sa = p.a_scale[p.a_per_row ? m : 0]; sb = p.b_scale[p.b_per_channel ? n : 0]; }
    if (deq_bf16) { sa = round_bf16(sa); sb = round_bf16(sb); }
    float acc = 0.0f;
    for (int k = 0; k < p.K; ++k) {
      if (mx && (k & 31) == 0) {
        sa = e8m0_to_f32(p.a_block_scales[(size_t)m * nblk + (k >> 5)]);
        sb = e8m0_to_f32(p.b_block_scales[(size_t)n * nblk + (k >> 5)]);
      }
      float av = f8e4m3fn_to_f32(p.a[(size_t)m * p.K + k]) * sa;
      float bv = f8e4m3fn_to_f32(b_is_nk ? p.b[(size_t)n * p.K + k] : p.b[(size_t)k * p.N + n]) * sb;
      if (deq_bf16) { av = round_bf16(av); bv = round_bf16(bv); }
      acc = acc + av * bv;
    }
    float bias = 0.0f;
    if (p.bias) bias = p.bias_is_bf16 ? bf16_to_f32(((const uint16_t*)p.bias)[n]) : ((const float*)p.bias)[n];
    const float v = epilogue_dispatch(acc, bias, p.epilogue, p.bf16_dot, p.bf16_ops);
    if (p.out8) {
      if (p.amax) atomicMax(reinterpret_cast<unsigned*>(p.amax), f32_to_bits(v) & 0x7fffffffu);
      float c = p.d_divides ? v / *p.d_scale : v * *p.d_scale;
      if (c == c) c = __builtin_fminf(__builtin_fmaxf(c, -448.0f), 448.0f);
      p.out8[idx] = (uint8_t)f32_to_f8e4m3fn_any(c);
    } else {
      p.out[idx] = f32_to_bf16(v);
    }
  }
}

// Pre-pass of the bf16-operand path: dst[r][c] = bf16(f32(src f8) * bf16(scale)), the dequantised operand
// exactly as a bf16-typed multiply leaves it.  src is [rows, cols] (TRANSPOSE: [cols, rows], i.e. a [K,N]
// rhs read so that dst is [N,K]); scale is one value or one per row of dst.  64 x 256 elements per
// workgroup.  With skip_if_pow2 the call belongs to the f8 kernel when both scales are powers of two.
template <bool TRANSPOSE>
__global__ __launch_bounds__(256) void f8_to_scaled_bf16_kernel(const uint8_t* __restrict__ src, uint16_t* __restrict__ dst,
                                                               int rows, int cols, const float* __restrict__ scale,
                                                               int per_row, const float* __restrict__ other_scale,
                                                               int skip_if_pow2) {
  if (skip_if_pow2 && is_pow2_f32(*scale) && is_pow2_f32(*other_scale)) return;
  __shared__ uint8_t tile[64][64 + 4];
  const int r0 = blockIdx.y * 64;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  for (int part = 0; part < 4; ++part) {   // four 64-column tiles per workgroup
    const int c0 = (blockIdx.x * 4 + part) * 64;
    if (c0 >= cols) break;
    if (TRANSPOSE) {
      // src row = c0 + i (a k of the rhs), src column = r0 + tx (a channel): read along the channels
      for (int i = ty; i < 64; i += 4) {
        const int c = c0 + i, r = r0 + tx;
        tile[i][tx] = (c < cols && r < rows) ? src[(size_t)c * rows + r] : 0;
      }
      __syncthreads();
    }
    for (int i = ty; i < 64; i += 4) {
      const int r = r0 + i, c = c0 + tx;
      if (r >= rows || c >= cols) continue;
      const uint8_t code = TRANSPOSE ? tile[tx][i] : src[(size_t)r * cols + c];
      const float s = round_bf16(scale[per_row ? r : 0]);
      dst[(size_t)r * cols + c] = f32_to_bf16(f8e4m3fn_to_f32(code) * s);
    }
    if (TRANSPOSE) __syncthreads();  // the tile is refilled by the next part
  }
}

__global__ void store_u32_kernel(uint32_t* dst, uint32_t value) { *dst = value; }

// Ragged dot: rows past the last group are a dot of nothing, epilogue(0).  Workgroup (x, y) takes 256
// channels and every gridDim.y-th of those rows; usually there are none and it returns at once.
__global__ __launch_bounds__(256) void ragged_tail_rows_kernel(TiledParams p) {
  long long start = 0;
  for (int g = 0; g < p.ragged_groups; ++g) {
    long long n = p.group_sizes_64 ? ((const long long*)p.group_sizes)[g] : (long long)((const int*)p.group_sizes)[g];
    n = n < 0 ? 0 : (n > p.M - start ? p.M - start : n);
    start += n;
  }
  const int n = blockIdx.x * 256 + threadIdx.x;
  if (n >= p.N) return;
  float bias = 0.0f;
  if (p.bias) bias = p.bias_is_bf16 ? bf16_to_f32(((const uint16_t*)p.bias)[n]) : ((const float*)p.bias)[n];
  const uint16_t v = f32_to_bf16(epilogue_dispatch(0.0f, bias, p.epilogue, p.bf16_dot, p.bf16_ops));
  for (long long m = start + blockIdx.y; m < p.M; m += gridDim.y) p.out[(size_t)m * p.N + n] = v;
}

template <int KIND, bool OUT_F8, bool SPLIT>
int launch_tiled_form(const TiledParams& tp, int batch, hipStream_t stream, const char* what) {
  constexpr size_t kLds = 2 * (size_t)(kTM + kTN) * kRow + (KIND == kFp8MX ? 4096 : 0);  // 128 KiB (+ scales)
  // per kernel instantiation and device: one bit per device ordinal; two threads that race both set
  // the attribute to the same value, which is harmless, and neither launches before it is set
  static std::atomic<unsigned long long> configured{0};
  int device = 0;
  (void)hipGetDevice(&device);
  const unsigned long long bit = 1ull << (device & 63);
  if (!(configured.load(std::memory_order_acquire) & bit)) {
    hipError_t e = hipFuncSetAttribute((const void*)tiled_dot_kernel<KIND, OUT_F8, SPLIT>,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)kLds);
    if (e != hipSuccess)
      return Fail(XLA_FFI_Error_Code_INTERNAL, "%s: cannot reserve %zu bytes of LDS: %s", what, kLds,
                  hipGetErrorString(e));
    configured.fetch_or(bit, std::memory_order_release);
  }
  dim3 grid((unsigned)(tp.tiles_m * tp.tiles_n), (unsigned)batch);
  if (tp.tail_tiles > 0) grid = dim3((unsigned)(tp.tail_first + 2 * tp.tail_tiles), 1u);
  hipLaunchKernelGGL((tiled_dot_kernel<KIND, OUT_F8, SPLIT>), grid, dim3(512), kLds, stream, tp);
  return CheckLaunch(what);
}

// The integer-weight kinds have one form, which can split tiles along K; the others a form for each.
template <int KIND, bool OUT_F8 = false>
int launch_tiled(const TiledParams& tp, int batch, hipStream_t stream, const char* what) {
  constexpr bool WQ = KIND == kS8 || KIND == kS4 || KIND == kU4 || KIND == kS8NK || KIND == kS4NK;
  if constexpr (WQ) return launch_tiled_form<KIND, OUT_F8, true>(tp, batch, stream, what);
  else if constexpr (KIND == kBf16) return launch_tiled_form<KIND, OUT_F8, false>(tp, batch, stream, what);
  else
    return tp.tail_tiles > 0 ? launch_tiled_form<KIND, OUT_F8, true>(tp, batch, stream, what)
                             : launch_tiled_form<KIND, OUT_F8, false>(tp, batch, stream, what);
}

}  // namespace

// Scratch for splitting the tiles of the last round along K: worth it when that round is at most
// half full and K is long enough for half of it to outweigh the hand-over (256 KiB per tile,
// written and read once).  0: no split for this shape.
// max_tiles: the most tiles the whole call may have (the f8 kinds split only calls that are all tail)
static size_t TailBytesFor(int64_t batch, int64_t M, int64_t K, int64_t N, int64_t min_rows, int64_t max_tiles = 0x7fffffff) {
  if (batch <= 0 || M < min_rows || K < 2048 || N <= 0) return 0;
  const int64_t tiles = batch * ((M + kTM - 1) / kTM) * ((N + kTN - 1) / kTN);
  const int64_t tail = tiles % 256;
  if (tail == 0 || tail > 128 || tiles > max_tiles || tiles + tail > 0x7fffffff) return 0;
  return (size_t)tail * (kTailSumsBytes + 2 * sizeof(unsigned long long));  // sums, flag, generation
}
// The f8 kinds' form that can split spills registers (the one-workgroup form sits at 254), which costs
// every tile of a launch: two spilling workgroups per tile still beat one when a quarter of the CUs or
// fewer have a tile at all (64 tiles: 88 -> 70 us at K = 8192), not when 112 have one (92 -> 95 us),
// and never when whole tiles run in the same launch.
constexpr int64_t kF8MaxTail = 64;
// (up to 64 rows the integer-weight dots run on the decode kernels)
size_t TiledTailWorkspaceBytes(int64_t batch, int64_t M, int64_t K, int64_t N) { return TailBytesFor(batch, M, K, N, 65); }

// More than 64 tokens of integer weights: the decode kernel, run once per 64 tokens, streams and
// dequantises the weights on every pass but fills the machine at any M; the tiled kernel dequantises
// once per 256 tokens but gives a CU nothing to do unless there are 256 tiles.  Estimates in
// microseconds fitted on MI355X over matrices from 4096 x 4096 to 8192 x 28672 and 80 to 1024 tokens:
//   decode, weights [K,N]: the first pass 14 + 1.4e-7 K N (s4; s8 2.0e-7), every further one of the
//     same launch 1 + 1.6e-7 K N (2.05e-7), a last pass of fewer than 64 tokens three quarters of a
//     first one, all of it once per batch (8192 x 28672 s4: 47 / 86 / 168 us at 64 / 128 / 256 tokens);
//   decode, weights [N,K]: one launch, 14 + 1.85e-7 K N per 64 tokens (s4 and s8 alike);
//   tiled: 25 + 0.025 K per round of 256 tiles, a last round of at most 128 tiles (split along K)
//     25 + 0.0125 K (K = 8192: 230 and 127); weights [N,K]: 25 + 0.0245 K and 20 + 0.01025 K.
static bool DecodePassesAreCheaper(int64_t batch, int64_t M, int64_t K, int64_t N, bool four_bit, bool k_minor) {
  const double kn = (double)K * (double)N;
  double decode_us;
  if (k_minor) {
    decode_us = (14.0 + (double)batch * (double)((M + 63) / 64) * 1.85e-7 * kn) / 1.05;  // (ties go to the passes)
  } else {
    const double first = 14.0 + kn * (four_bit ? 1.4e-7 : 2.0e-7);
    const double next = 1.0 + kn * (four_bit ? 1.6e-7 : 2.05e-7);
    const int64_t whole = M / 64, rest = M % 64;
    decode_us = (double)batch * ((whole > 0 ? first + (double)(whole - 1) * next : 0.0) + (rest > 0 ? 0.75 * first : 0.0));
  }
  const int64_t tiles = batch * ((M + kTM - 1) / kTM) * ((N + kTN - 1) / kTN);
  const int64_t tail = tiles % 256;
  const double round_us = k_minor ? 25.0 + 0.0245 * (double)K : 25.0 + 0.025 * (double)K;
  const double half_us = k_minor ? 20.0 + 0.01025 * (double)K : 25.0 + 0.0125 * (double)K;
  const double tiled_us = (double)(tiles / 256) * round_us + (tail == 0 ? 0.0 : tail <= 128 && K >= 2048 ? half_us : round_us);
  return decode_us <= tiled_us;
}

// bf16 x s8 per-channel prefill.  Returns -1 when the tiled kernel does not cover the shape
// (the caller then falls back), 0 on success, or an error code.
int LaunchDequantDotPrefill(const XlaAmdDequantDot& p, hipStream_t stream) {
  // s4 with bf16 scales per power-of-two group of rows and a bf16-typed dequantise multiply, or
  // s8 with per-channel scales and an f32-typed one; u4 (with or without zero points) as s4
  const bool u4 = p.weight_dtype == XLA_FFI_DataType_U4;
  if (u4 && p.zero_points && ((uintptr_t)p.zero_points % 4) != 0) return -1;  // a dword (8 channels) per load
  const bool s4 = (p.weight_dtype == XLA_FFI_DataType_S4 || u4) && p.dequant_type == XLA_FFI_DataType_BF16 &&
                  p.scale_dtype == XLA_FFI_DataType_BF16 && p.group >= 8 && (p.group & (p.group - 1)) == 0 &&
                  p.N % 8 == 0 && ((uintptr_t)p.scales % 16) == 0 &&
                  (double)(p.K / p.group) * p.N * 2 < 2147483000.0;
  const bool s8 = p.weight_dtype == XLA_FFI_DataType_S8 && p.group == p.K && p.dequant_type == XLA_FFI_DataType_F32;
  if (!s4 && !s8) return -1;
  const bool ragged = p.group_sizes != nullptr;  // the caller has decided that the rows per group make tiles worth it
  if (u4 && ragged) return -1;  // a ragged dot over u4 weights stays with the 64-row chunks of the decode kernel
  if (!ragged && GetOption("dequant_dot_kernel") != 3 && DecodePassesAreCheaper(p.batch, p.M, p.K, p.N, s4, false))
    return -1;
  if (p.K % 8 != 0 || p.N % 4 != 0 || ((uintptr_t)p.lhs % 16) || ((uintptr_t)p.weights % 4)) return -1;
  // 32-bit buffer offsets per batch
  if ((double)p.M * p.K * 2 >= 2147483000.0 || (double)p.K * p.N >= 2147483000.0) return -1;
  TiledParams tp{};
  tp.a = (const uint8_t*)p.lhs;
  tp.b = (const uint8_t*)p.weights;
  tp.scales = p.scales;
  tp.bias = (p.epilogue & 1) ? p.bias : nullptr;
  tp.out = (uint16_t*)p.out;
  tp.M = (int)p.M; tp.K = (int)p.K; tp.N = (int)p.N;
  tp.scale_is_bf16 = p.scale_dtype == XLA_FFI_DataType_BF16;
  tp.bias_is_bf16 = p.bias_dtype == XLA_FFI_DataType_BF16;
  tp.scale_batched = p.scale_batch == p.batch && p.batch > 1;
  tp.bf16_dot = p.dot_type == XLA_FFI_DataType_BF16;
  tp.bf16_ops = p.epilogue_type == XLA_FFI_DataType_BF16;
  tp.epilogue = p.epilogue;
  tp.tiles_m = (tp.M + kTM - 1) / kTM;
  tp.tiles_n = (tp.N + kTN - 1) / kTN;
  tp.closed_form_epilogue = GetOption("tiled_epilogue") == 1;
  if (s4) tp.group_shift = __builtin_ctzll((unsigned long long)p.group);  // sizes the scales' descriptor: set before any launch
  tp.zero_points = u4 ? (const uint8_t*)p.zero_points : nullptr;
  if (ragged) {
    // at most floor(M / 256) + groups tiles of rows, whatever the sizes turn out to be
    tp.group_sizes = p.group_sizes;
    tp.group_sizes_64 = p.group_sizes_dtype == XLA_FFI_DataType_S64;
    tp.ragged_groups = (int)p.batch;
    tp.ragged_slots = (int)(p.M / kTM + p.batch);
    if ((double)tp.ragged_slots * tp.tiles_n > 2147483000.0) return -1;
    tp.tiles_m = tp.ragged_slots;
    tp.scale_batched = p.scale_batch == p.batch;  // one set of scales per group, also for a single group
    const int rc = u4   ? launch_tiled<kU4>(tp, 1, stream, "dequant_dot_tiled_u4")
                   : s4 ? launch_tiled<kS4>(tp, 1, stream, "dequant_dot_tiled_s4")
                        : launch_tiled<kS8>(tp, 1, stream, "dequant_dot_tiled_s8");
    if (rc) return rc;
    hipLaunchKernelGGL(ragged_tail_rows_kernel, dim3((unsigned)((p.N + 255) / 256), 64u), dim3(256), 0, stream, tp);
    SetLastKernel(u4 ? "dequant_dot_tiled_u4_rounded:ragged" : s4 ? "dequant_dot_tiled_s4_rounded:ragged" : "dequant_dot_tiled_s8_factored:ragged");
    return CheckLaunch("dequant_dot_ragged_tail_rows");
  }
  // the last round of 256 workgroups, when at most half full, runs as two workgroups per tile
  {
    const size_t need = TiledTailWorkspaceBytes(p.batch, p.M, p.K, p.N);
    if (need && GetOption("tiled_tail") != 1 && p.workspace && ((uintptr_t)p.workspace % 16) == 0 &&
        p.workspace_bytes >= need) {
      const int64_t tiles = p.batch * (int64_t)tp.tiles_m * tp.tiles_n;
      tp.tail_tiles = (int)(tiles % 256);
      tp.tail_first = (int)(tiles - tp.tail_tiles);
      tp.tail_sums = (float*)p.workspace;
      tp.tail_flags = (unsigned long long*)((char*)p.workspace + (size_t)tp.tail_tiles * kTailSumsBytes);
      tp.epoch = NextHandOverEpoch();
      tp.handover_test = GetOption("handover_test");
    }
  }
  if (u4) {
    SetLastKernel(tp.tail_tiles ? "dequant_dot_tiled_u4_rounded:tail2" : "dequant_dot_tiled_u4_rounded");
    return launch_tiled<kU4>(tp, (int)p.batch, stream, "dequant_dot_tiled_u4");
  }
  if (s4) {
    SetLastKernel(tp.tail_tiles ? "dequant_dot_tiled_s4_rounded:tail2" : "dequant_dot_tiled_s4_rounded");
    return launch_tiled<kS4>(tp, (int)p.batch, stream, "dequant_dot_tiled_s4");
  }
  SetLastKernel(tp.tail_tiles ? "dequant_dot_tiled_s8_factored:tail2" : "dequant_dot_tiled_s8_factored");
  return launch_tiled<kS8>(tp, (int)p.batch, stream, "dequant_dot_tiled_s8");
}

// The same for weights stored [batch,N,K] (scales [batch,N] or [batch,N,K/group]): s8 with one scale per
// channel under an f32-typed multiply, s4 with bf16 scales per power-of-two group of at least 32 under
// a bf16-typed one.  -1: not taken (the token-chunked streaming kernel runs instead).
int LaunchDequantDotPrefillNk(const XlaAmdDequantDot& p, hipStream_t stream) {
  const bool s4 = p.weight_dtype == XLA_FFI_DataType_S4 && p.dequant_type == XLA_FFI_DataType_BF16 &&
                  p.scale_dtype == XLA_FFI_DataType_BF16 && p.group >= 32 && (p.group & (p.group - 1)) == 0 &&
                  p.K % 32 == 0 && (double)(p.K / p.group) * p.N * 2 < 2147483000.0;
  const bool s8 = p.weight_dtype == XLA_FFI_DataType_S8 && p.group == p.K && p.dequant_type == XLA_FFI_DataType_F32 &&
                  p.K % 16 == 0;
  if ((!s4 && !s8) || p.zero_points) return -1;
  const bool ragged = p.group_sizes != nullptr;  // the caller has decided that the rows per group make tiles worth it
  if (!ragged && GetOption("dequant_dot_kernel") != 3 && DecodePassesAreCheaper(p.batch, p.M, p.K, p.N, s4, true))
    return -1;
  if (p.N % 4 != 0 || ((uintptr_t)p.lhs % 16) || ((uintptr_t)p.weights % 16) || ((uintptr_t)p.scales % 2)) return -1;
  if ((double)p.M * p.K * 2 >= 2147483000.0 || (double)p.K * p.N >= 2147483000.0) return -1;
  TiledParams tp{};
  tp.a = (const uint8_t*)p.lhs;
  tp.b = (const uint8_t*)p.weights;
  tp.scales = p.scales;
  tp.bias = (p.epilogue & 1) ? p.bias : nullptr;
  tp.out = (uint16_t*)p.out;
  tp.M = (int)p.M; tp.K = (int)p.K; tp.N = (int)p.N;
  tp.scale_is_bf16 = p.scale_dtype == XLA_FFI_DataType_BF16;
  tp.bias_is_bf16 = p.bias_dtype == XLA_FFI_DataType_BF16;
  tp.scale_batched = p.scale_batch == p.batch && p.batch > 1;
  tp.bf16_dot = p.dot_type == XLA_FFI_DataType_BF16;
  tp.bf16_ops = p.epilogue_type == XLA_FFI_DataType_BF16;
  tp.epilogue = p.epilogue;
  tp.tiles_m = (tp.M + kTM - 1) / kTM;
  tp.tiles_n = (tp.N + kTN - 1) / kTN;
  tp.closed_form_epilogue = GetOption("tiled_epilogue") == 1;
  if (s4) tp.group_shift = __builtin_ctzll((unsigned long long)p.group);  // sizes the scales' descriptor
  if (ragged) {
    // at most floor(M / 256) + groups tiles of rows, whatever the sizes turn out to be
    if ((double)p.M * p.N * 2 >= 2147483000.0) return -1;
    tp.group_sizes = p.group_sizes;
    tp.group_sizes_64 = p.group_sizes_dtype == XLA_FFI_DataType_S64;
    tp.ragged_groups = (int)p.batch;
    tp.ragged_slots = (int)(p.M / kTM + p.batch);
    if ((double)tp.ragged_slots * tp.tiles_n > 2147483000.0) return -1;
    tp.tiles_m = tp.ragged_slots;
    tp.scale_batched = p.scale_batch == p.batch;  // one set of scales per group, also for a single group
    const int rc = s4 ? launch_tiled<kS4NK>(tp, 1, stream, "dequant_dot_tiled_nk_s4") : launch_tiled<kS8NK>(tp, 1, stream, "dequant_dot_tiled_nk_s8");
    if (rc) return rc;
    hipLaunchKernelGGL(ragged_tail_rows_kernel, dim3((unsigned)((p.N + 255) / 256), 64u), dim3(256), 0, stream, tp);
    SetLastKernel(s4 ? "dequant_dot_tiled_nk_s4_rounded:ragged" : "dequant_dot_tiled_nk_s8_factored:ragged");
    return CheckLaunch("dequant_dot_ragged_tail_rows");
  }
  const size_t need = TiledTailWorkspaceBytes(p.batch, p.M, p.K, p.N);
  if (need && GetOption("tiled_tail") != 1 && p.workspace && ((uintptr_t)p.workspace % 16) == 0 &&
      p.workspace_bytes >= need) {
    const int64_t tiles = p.batch * (int64_t)tp.tiles_m * tp.tiles_n;
    tp.tail_tiles = (int)(tiles % 256);
    tp.tail_first = (int)(tiles - tp.tail_tiles);
    tp.tail_sums = (float*)p.workspace;
    tp.tail_flags = (unsigned long long*)((char*)p.workspace + (size_t)tp.tail_tiles * kTailSumsBytes);
    tp.epoch = NextHandOverEpoch();
    tp.handover_test = GetOption("handover_test");
  }
  if (s4) {
    SetLastKernel(tp.tail_tiles ? "dequant_dot_tiled_nk_s4_rounded:tail2" : "dequant_dot_tiled_nk_s4_rounded");
    return launch_tiled<kS4NK>(tp, (int)p.batch, stream, "dequant_dot_tiled_nk_s4");
  }
  SetLastKernel(tp.tail_tiles ? "dequant_dot_tiled_nk_s8_factored:tail2" : "dequant_dot_tiled_nk_s8_factored");
  return launch_tiled<kS8NK>(tp, (int)p.batch, stream, "dequant_dot_tiled_nk_s8");
}

namespace {
size_t RoundUp256(size_t v) { return (v + 255) & ~(size_t)255; }
// the transposed copy of a [K,N] rhs that cannot go in as it is: N no multiple of 16, or the pre-pass forced
size_t TransposedCopyBytes(int64_t K, int64_t N, int rhs_contracting_dim) {
  return rhs_contracting_dim == 0 && (N % 16 != 0 || GetOption("fp8_dot_layout") == 1) ? (size_t)K * N : 0;
}
// both operands as bf16 with K minor (a dequantise multiply that is bf16-typed: see LaunchFp8ScaledDot);
// 0 when the bf16-operand kernel does not take the shape
size_t Bf16OperandBytes(int64_t M, int64_t K, int64_t N) {
  if (M <= 0 || N <= 0 || K <= 0 || K % 8 != 0 || (double)M * K * 2 >= 2147483000.0 || (double)N * K * 2 >= 2147483000.0)
    return 0;
  return RoundUp256((size_t)M * K * 2) + (size_t)N * K * 2;
}
}  // namespace

// Scratch of an f8 scaled dot: [transposed copy of the rhs, if it needs one][a as bf16][b as bf16, K minor],
// the last two only under a bf16-typed dequantise multiply.
size_t Fp8ScaledDotWorkspaceBytes(int64_t M, int64_t K, int64_t N, int rhs_contracting_dim, int dequant_type) {
  const size_t copy = TransposedCopyBytes(K, N, rhs_contracting_dim);
  const size_t ops = dequant_type == XLA_FFI_DataType_BF16 ? Bf16OperandBytes(M, K, N) : 0;
  size_t tiled = ops ? RoundUp256(copy) + ops : copy;
  // nothing else in the scratch: the tiles of a last round at most half full split along K (f32 sums)
  // (up to 64 rows the streaming kernels take the call, with the few exceptions that stay unsplit)
  if (!tiled) tiled = TailBytesFor(1, M, K, N, 65, kF8MaxTail);
  // up to 64 rows of a under f32-typed multiplies: the streaming kernels' K-slices instead
  const size_t decode = Fp8DotDecodeWorkspaceBytes(1, M, K, N, rhs_contracting_dim);
  return tiled > decode ? tiled : decode;
}

int LaunchFp8ScaledDot(const XlaAmdFp8ScaledDot& p, hipStream_t stream) {
  // Opt-in: a bf16-typed dequantise multiply computed the way the reference's GPU pipeline computes the
  // same HLO (GemmRewriter turns it into an FP8 matmul whose scales multiply the f32 sum,
  // gemm_rewriter.cc:1235-1591), not op by op: the f32-typed call.
  if (p.dequant_type == XLA_FFI_DataType_BF16 && GetOption("fp8_scales_on_sum") == 1) {
    XlaAmdFp8ScaledDot q = p;
    q.dequant_type = XLA_FFI_DataType_F32;
    return LaunchFp8ScaledDot(q, stream);
  }
  if (p.M < 0 || p.K < 0 || p.N < 0 || p.M > 0x7fffffff || p.K > 0x7fffffff || p.N > 0x7fffffff)
    return Fail(XLA_FFI_Error_Code_INVALID_ARGUMENT, "fp8_scaled_dot: bad shape");
  if (p.rhs_contracting_dim != 0 && p.rhs_contracting_dim != 1)
    return Fail(XLA_FFI_Error_Code_INVALID_ARGUMENT, "fp8_scaled_dot: rhs_contracting_dim must be 0 or 1");
  if (!IsF32OrBf16(p.dequant_type) || !IsF32OrBf16(p.dot_type) || !IsF32OrBf16(p.epilogue_type) ||
      (p.bias && !IsF32OrBf16(p.bias_dtype)))
    return Fail(XLA_FFI_Error_Code_INVALID_ARGUMENT, "fp8_scaled_dot: types must be F32 or BF16");
  if (p.epilogue < 0 || p.epilogue > XLA_AMD_EPI_BIAS_SILU)
    return Fail(XLA_FFI_Error_Code_INVALID_ARGUMENT, "fp8_scaled_dot: unknown epilogue %d", p.epilogue);
  if ((p.epilogue & 1) && !p.bias)
    return Fail(XLA_FFI_Error_Code_INVALID_ARGUMENT, "fp8_scaled_dot: BIAS epilogue without a bias");
  if (p.M == 0 || p.N == 0 || p.batch < 0) {
    if (p.amax && p.out_dtype == XLA_FFI_DataType_F8E4M3FN) {  // maximum over nothing: its init, -inf
      hipLaunchKernelGGL(store_u32_kernel, dim3(1), dim3(1), 0, stream, reinterpret_cast<uint32_t*>(p.amax), 0xff800000u);
      int rc = CheckLaunch("fp8_scaled_dot_amax_init");
      if (rc) return rc;
    }
    SetLastKernel("fp8_scaled_dot:empty");
    return 0;
  }
  const bool mx = p.a_block_scales || p.b_block_scales;
  if (mx) {
    if (!p.a_block_scales || !p.b_block_scales || p.block != 32 || p.K % 32 != 0)
      return Fail(XLA_FFI_Error_Code_INVALID_ARGUMENT,
                  "fp8_scaled_dot: block scales come for both operands, one per 32 elements of K");
    if (p.rhs_contracting_dim != 1)
      return Fail(XLA_FFI_Error_Code_INVALID_ARGUMENT, "fp8_scaled_dot: a block-scaled rhs is [N,K]");
    if (p.a_scale_per_row || p.b_scale_per_channel || p.out_dtype == XLA_FFI_DataType_F8E4M3FN ||
        p.dequant_type != XLA_FFI_DataType_F32)
      return Fail(XLA_FFI_Error_Code_UNIMPLEMENTED,
                  "fp8_scaled_dot: block scales go with a bf16 result and no other scales");
  }
  if (!p.a || !p.b || (!mx && (!p.a_scale || !p.b_scale)) || !p.out)
    return Fail(XLA_FFI_Error_Code_INVALID_ARGUMENT, "fp8_scaled_dot: null buffer");
  const bool out_f8 = p.out_dtype == XLA_FFI_DataType_F8E4M3FN;
  if (!out_f8 && p.out_dtype != 0 && p.out_dtype != XLA_FFI_DataType_BF16)
    return Fail(XLA_FFI_Error_Code_INVALID_ARGUMENT, "fp8_scaled_dot: the result is BF16 or F8E4M3FN");
  if (out_f8 && !p.d_scale)
    return Fail(XLA_FFI_Error_Code_INVALID_ARGUMENT, "fp8_scaled_dot: an F8E4M3FN result needs d_scale");
  if (out_f8 && (p.dot_type != XLA_FFI_DataType_F32 || p.epilogue_type != XLA_FFI_DataType_F32))
    return Fail(XLA_FFI_Error_Code_INVALID_ARGUMENT,
                "fp8_scaled_dot: an F8E4M3FN result is scaled from f32-typed dot and epilogue ops");

  TiledParams tp{};
  tp.a = (const uint8_t*)p.a;
  tp.b = (const uint8_t*)p.b;
  tp.a_scale = p.a_scale;
  tp.b_scale = p.b_scale;
  tp.a_per_row = p.a_scale_per_row != 0;
  tp.b_per_channel = p.b_scale_per_channel != 0;
  tp.bias = (p.epilogue & 1) ? p.bias : nullptr;
  tp.out = out_f8 ? nullptr : (uint16_t*)p.out;
  tp.out8 = out_f8 ? (uint8_t*)p.out : nullptr;
  tp.d_scale = p.d_scale;
  tp.d_divides = p.d_scale_multiplies ? 0 : 1;
  tp.a_block_scales = (const uint8_t*)p.a_block_scales;
  tp.b_block_scales = (const uint8_t*)p.b_block_scales;
  tp.amax = out_f8 ? p.amax : nullptr;
  if (tp.amax) {  // the kernels fold their maxima into it with atomics (a kernel, not a memset: graphs)
    hipLaunchKernelGGL(store_u32_kernel, dim3(1), dim3(1), 0, stream, reinterpret_cast<uint32_t*>(tp.amax), 0u);
    int rc = CheckLaunch("fp8_scaled_dot_amax_init");
    if (rc) return rc;
  }
  const int force = GetOption("fp8_dot_kernel");  // 0 auto, 1 exact (slow), 2 tiled, 3 streaming (up to 64 rows of a)
  // A call with a bf16-typed multiply that the streaming kernels took: they have served it if both
  // scales are powers of two; the kernels below that serve it otherwise are launched behind them.
  bool streamed_if_pow2 = false;
  char streamed_name[64] = "";
  if (force == 0 || force == 3) {
    const bool bf16_multiply = p.dequant_type == XLA_FFI_DataType_BF16;
    bool any_scale = false;
    const int rc = LaunchFp8DotDecode(p, stream, bf16_multiply, &any_scale);
    if (rc > 0 || (rc == 0 && (!bf16_multiply || any_scale))) return rc;
    if (rc == 0) {
      streamed_if_pow2 = true;
      snprintf(streamed_name, sizeof(streamed_name), "%s", xla_amd_last_kernel());
    } else if (force == 3)
      return Fail(XLA_FFI_Error_Code_FAILED_PRECONDITION,
                  "fp8_scaled_dot: the streaming kernels take K %% 8 == 0 and N %% 8 == 0, 8-byte aligned operands "
                  "and f32-typed multiplies; more than 64 rows of a (48 with the rhs [N,K], 32 with block scales) "
                  "only without a batch dimension");
  }
  tp.M = (int)p.M; tp.K = (int)p.K; tp.N = (int)p.N;
  tp.bias_is_bf16 = p.bias_dtype == XLA_FFI_DataType_BF16;
  tp.bf16_dot = p.dot_type == XLA_FFI_DataType_BF16;
  tp.bf16_ops = p.epilogue_type == XLA_FFI_DataType_BF16;
  tp.epilogue = p.epilogue;
  tp.tiles_m = (tp.M + kTM - 1) / kTM;
  tp.tiles_n = (tp.N + kTN - 1) / kTN;
  const bool deq_bf16 = p.dequant_type == XLA_FFI_DataType_BF16;
  tp.require_pow2_scales = deq_bf16;
  tp.closed_form_epilogue = GetOption("tiled_epilogue") == 1;
  // a vector of scales cannot be tested for powers of two in one place: with a bf16-typed
  // multiply it takes the exact kernel
  const bool vector_scales = tp.a_per_row || tp.b_per_channel;

  const bool nk = p.rhs_contracting_dim == 1;
  const int batch = p.batch > 1 ? (int)p.batch : 1;
  if (p.batch > 65535) return Fail(XLA_FFI_Error_Code_INVALID_ARGUMENT, "fp8_scaled_dot: more than 65535 batches");
  if (batch > 1 && vector_scales)
    return Fail(XLA_FFI_Error_Code_INVALID_ARGUMENT, "fp8_scaled_dot: a batched dot takes per-tensor scales");
  bool tiled_ok = p.K % 16 == 0 && p.K > 0 && ((uintptr_t)p.a % 16 == 0) && force != 1 &&
                  !(deq_bf16 && vector_scales) &&
                  (double)p.M * p.K < 2147483000.0 && (double)p.N * p.K < 2147483000.0;
  const uint8_t* b_nk = (const uint8_t*)p.b;
  // a [K,N] rhs with whole 16-channel chunks goes in as it is: the kernel stages it K-major and
  // transposes on the way out of LDS (fp8_dot_layout = 1 forces the transposing pre-pass instead)
  const bool kn_direct = tiled_ok && !nk && p.N % 16 == 0 && ((uintptr_t)p.b % 16 == 0) &&
                         GetOption("fp8_dot_layout") != 1;
  if (tiled_ok && !nk && !kn_direct && !streamed_if_pow2) {  // (streamed: no f8 tiled kernel will run)
    // (the pre-pass handles one matrix: a batched [K,N] rhs with ragged N takes the exact kernel)
    if (batch == 1 && p.workspace && p.workspace_bytes >= (size_t)p.K * p.N && ((uintptr_t)p.workspace % 16 == 0)) {
      if (p.N % 4 == 0 && ((uintptr_t)p.b % 4 == 0)) {
        dim3 tgrid((unsigned)((p.N + 127) / 128), (unsigned)((p.K + 127) / 128));
        hipLaunchKernelGGL(transpose_bytes_fast_kernel, tgrid, dim3(256), 0, stream, (const uint8_t*)p.b,
                           (uint8_t*)p.workspace, (int)p.K, (int)p.N);
      } else {
        dim3 tgrid((unsigned)((p.N + 63) / 64), (unsigned)((p.K + 63) / 64));
        hipLaunchKernelGGL(transpose_bytes_kernel, tgrid, dim3(256), 0, stream, (const uint8_t*)p.b,
                           (uint8_t*)p.workspace, (int)p.K, (int)p.N);
      }
      int rc = CheckLaunch("fp8_scaled_dot_transpose");
      if (rc) return rc;
      b_nk = (const uint8_t*)p.workspace;
    } else {
      tiled_ok = false;
    }
  }
  if (tiled_ok && ((uintptr_t)b_nk % 16 != 0)) tiled_ok = false;
  // the stage's scales move as one dword per row: K % 128 == 0 and 4-byte aligned scale tensors
  if (mx && (p.K % 128 != 0 || ((uintptr_t)p.a_block_scales % 4) || ((uintptr_t)p.b_block_scales % 4) ||
             (double)p.M * (p.K / 32) >= 2147483000.0 || (double)p.N * (p.K / 32) >= 2147483000.0))
    tiled_ok = false;
  if (force == 2 && !tiled_ok)
    return Fail(XLA_FFI_Error_Code_FAILED_PRECONDITION,
                "fp8_scaled_dot: the tiled kernel needs K %% 16 == 0, 16-byte aligned operands and, "
                "for a [K,N] rhs, a workspace of K*N bytes");
  if (p.K == 0) tiled_ok = false;

  const size_t eblocks = ((size_t)p.M * p.N + 255) / 256;
  dim3 egrid((unsigned)(eblocks < 8192 ? (eblocks ? eblocks : 1) : 8192), (unsigned)batch);

  // A bf16-typed dequantise multiply rounds every a * a_scale and b * b_scale to bf16.  With scales
  // that are powers of two that rounding changes nothing and the f8 kernel serves the call; otherwise
  // the rounded operands are bf16 numbers, so a pre-pass writes them out (b with K minor) and the
  // bf16 matrix cores multiply them -- decided on the device from the scale values, where both are
  // single values; vectors of scales always go this way.  Without the scratch: the exact kernel.
  const size_t ops_bytes = deq_bf16 && !mx && !out_f8 && batch == 1 && force != 1 ? Bf16OperandBytes(p.M, p.K, p.N) : 0;
  const size_t ops_at = RoundUp256(TransposedCopyBytes(p.K, p.N, p.rhs_contracting_dim));
  if (ops_bytes && p.workspace && ((uintptr_t)p.workspace % 256) == 0 && p.workspace_bytes >= ops_at + ops_bytes &&
      ((uintptr_t)p.out % 8) == 0) {
    int rc = 0;
    const bool by_value = !vector_scales;  // the f8 kernel may serve the call: both decide from the scale values
    if (by_value && tiled_ok && !streamed_if_pow2) {
      TiledParams tt = tp;
      tt.b = b_nk;
      rc = kn_direct ? launch_tiled<kFp8KN>(tt, 1, stream, "fp8_scaled_dot_tiled_kn") : launch_tiled<kFp8>(tt, 1, stream, "fp8_scaled_dot_tiled");
      if (rc) return rc;
    }
    uint16_t* a16 = (uint16_t*)((char*)p.workspace + ops_at);
    uint16_t* b16 = (uint16_t*)((char*)a16 + RoundUp256((size_t)p.M * p.K * 2));
    const int skip = (by_value && tiled_ok) || streamed_if_pow2 ? 1 : 0;
    hipLaunchKernelGGL(f8_to_scaled_bf16_kernel<false>, dim3((unsigned)((p.K + 255) / 256), (unsigned)((p.M + 63) / 64)), dim3(256), 0,
                       stream, (const uint8_t*)p.a, a16, (int)p.M, (int)p.K, p.a_scale, tp.a_per_row ? 1 : 0, p.b_scale, skip);
    if (nk)
      hipLaunchKernelGGL(f8_to_scaled_bf16_kernel<false>, dim3((unsigned)((p.K + 255) / 256), (unsigned)((p.N + 63) / 64)), dim3(256),
                         0, stream, (const uint8_t*)p.b, b16, (int)p.N, (int)p.K, p.b_scale, tp.b_per_channel ? 1 : 0, p.a_scale, skip);
    else
      hipLaunchKernelGGL(f8_to_scaled_bf16_kernel<true>, dim3((unsigned)((p.K + 255) / 256), (unsigned)((p.N + 63) / 64)), dim3(256),
                         0, stream, (const uint8_t*)p.b, b16, (int)p.N, (int)p.K, p.b_scale, tp.b_per_channel ? 1 : 0, p.a_scale, skip);
    rc = CheckLaunch("fp8_scaled_dot_bf16_operands_prepass");
    if (rc) return rc;
    TiledParams tb = tp;
    tb.a = (const uint8_t*)a16;
    tb.b = (const uint8_t*)b16;
    tb.require_pow2_scales = 0;
    tb.skip_if_pow2_scales = skip;
    tb.a_per_row = tb.b_per_channel = 0;  // already in the operands
    rc = launch_tiled<kBf16>(tb, 1, stream, "fp8_scaled_dot_bf16_operands");
    if (rc) return rc;
    if (streamed_if_pow2) {
      char name[96];
      snprintf(name, sizeof(name), "%s|bf16_operands", streamed_name);
      SetLastKernel(name);
      return 0;
    }
    SetLastKernel(skip ? (kn_direct ? "fp8_scaled_dot_tiled_kn|bf16_operands" : nk ? "fp8_scaled_dot_tiled|bf16_operands"
                                                                                    : "fp8_scaled_dot_tiled+transpose|bf16_operands")
                       : "fp8_scaled_dot_bf16_operands");
    return 0;
  }
  if (streamed_if_pow2) {  // (no scratch for the bf16 operands: the exact kernel, if a scale is no power of two)
    hipLaunchKernelGGL(fp8_dot_exact_kernel, egrid, dim3(256), 0, stream, tp, nk ? 1 : 0, 1, 1);
    const int rc = CheckLaunch("fp8_scaled_dot_exact");
    if (rc) return rc;
    SetLastKernel(streamed_name);
    return 0;
  }
  if (tiled_ok) {
    TiledParams tt = tp;
    tt.b = b_nk;
    int rc;
    // the last round of 256 workgroups, when at most half full, runs as two workgroups per tile (the
    // scratch then holds nothing else: no transposed copy, no bf16 operands)
    const size_t tail_need = (nk || kn_direct) && !deq_bf16 ? TailBytesFor(batch, p.M, p.K, p.N, 65, kF8MaxTail) : 0;
    if (tail_need && GetOption("tiled_tail") != 1 && p.workspace && ((uintptr_t)p.workspace % 16) == 0 &&
        p.workspace_bytes >= tail_need) {
      const int64_t tiles = (int64_t)batch * tt.tiles_m * tt.tiles_n;
      tt.tail_tiles = (int)(tiles % 256);
      tt.tail_first = (int)(tiles - tt.tail_tiles);
      tt.tail_sums = (float*)p.workspace;
      tt.tail_flags = (unsigned long long*)((char*)p.workspace + (size_t)tt.tail_tiles * kTailSumsBytes);
      tt.epoch = NextHandOverEpoch();
      tt.handover_test = GetOption("handover_test");
    }
    const char* const split = tt.tail_tiles ? ":tail2" : "";
    if (mx)
      rc = launch_tiled<kFp8MX>(tt, batch, stream, "fp8_scaled_dot_tiled_mx");
    else if (out_f8)
      rc = kn_direct ? launch_tiled<kFp8KN, true>(tt, batch, stream, "fp8_scaled_dot_tiled_kn_f8")
                     : launch_tiled<kFp8, true>(tt, batch, stream, "fp8_scaled_dot_tiled_f8");
    else
      rc = kn_direct ? launch_tiled<kFp8KN>(tt, batch, stream, "fp8_scaled_dot_tiled_kn")
                     : launch_tiled<kFp8>(tt, batch, stream, "fp8_scaled_dot_tiled");
    if (rc) return rc;
    if (deq_bf16) {
      // runs only if a scale is not a power of two (decided on the device, no host read)
      hipLaunchKernelGGL(fp8_dot_exact_kernel, egrid, dim3(256), 0, stream, tp, nk ? 1 : 0, 1, 1);
      rc = CheckLaunch("fp8_scaled_dot_exact");
      if (rc) return rc;
    }
    char name[64];
    snprintf(name, sizeof(name), "%s%s",
             mx       ? "fp8_scaled_dot_tiled_mx"
             : out_f8 ? (nk ? "fp8_scaled_dot_tiled_f8" : kn_direct ? "fp8_scaled_dot_tiled_kn_f8" : "fp8_scaled_dot_tiled+transpose_f8")
                      : (nk ? "fp8_scaled_dot_tiled" : kn_direct ? "fp8_scaled_dot_tiled_kn" : "fp8_scaled_dot_tiled+transpose"),
             split);
    SetLastKernel(name);
    return 0;
  }
  hipLaunchKernelGGL(fp8_dot_exact_kernel, egrid, dim3(256), 0, stream, tp, nk ? 1 : 0, deq_bf16 ? 1 : 0, 0);
  SetLastKernel("fp8_scaled_dot_exact");
  return CheckLaunch("fp8_scaled_dot_exact");
}

}  // namespace xla_amd
