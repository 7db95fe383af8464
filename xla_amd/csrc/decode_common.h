// Declarations shared by the decode (weight-streaming) dequantize-dot kernels.
#ifndef XLA_AMD_CSRC_DECODE_COMMON_H_
#define XLA_AMD_CSRC_DECODE_COMMON_H_

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

#include "device_numerics.h"
#include "launch.h"

namespace xla_amd {

enum : int { kRounded = 0, kFactored = 1, kGroupFactored = 2 };

struct DecodeParams {
  const uint16_t* lhs;   // [batch, M, K]
  const uint8_t* w;      // [batch, K, N] packed
  const void* scales;    // [scale_batch, K/group, N]
  const void* bias;      // [N] or null
  uint16_t* out;         // [batch, M, N]
  float* workspace;      // [batch, slices, M, N] when slices > 1
  int M, K, N, group;
  int scale_is_bf16, bias_is_bf16, scale_batched;
  int bf16_dot, bf16_ops, epilogue;
  int strips, slices, rows_per_slice;  // rows_per_slice: multiple of 32 * WAVES
  // Rows of a slice that a wave of age class c (wave index / 4) takes, multiples of 64: the
  // waves w, w+4, w+8, ... share a SIMD, which serves the oldest wave first.
  int class_rows[4];
  int weights_shared;  // every batch reads the same weights and scales (token chunks of one matrix)
  // s4x kernels: a unit is four scale groups of rows; a SIMD's waves take class_units[age class]
  // consecutive units each, SIMD b starting at unit b * units_per_simd of the slice
  int units_per_simd;
  int class_units[4];
  // s4x kernels, two workgroups per strip handing over inside the kernel: the producer's sums go to
  // workspace[batch * strips + strip][16 x 256 floats], then its flag is raised to
  // HandOverTarget(epoch, generation of the strip): flags[2 * (batch * strips + strip)] is the flag,
  // the word after it the generation.  s8x kernels: slices - 1 producers per strip, each with sums
  // and a flag, then the strip's generation word.
  int pair;
  int rows_first;       // rows the producer takes; the finisher takes rows_per_slice from there on
  int units_per_simd2;  // the finisher's units per SIMD; its class split is class_units[2..3]
  unsigned long long* flags;
  unsigned long long epoch;
  // s8x kernels with 64-channel strips and 1, 2 or 4 slices: workgroup ids are laid out so that the
  // two strips that share a 128-byte line of every weight row lie 8 ids apart (the same XCD and L2
  // when workgroups go round the XCDs in turn): id = 16 * G + 8 * half + pair_in_group * slices + slice,
  // strip = 2 * (G * pairs_per_group + pair_in_group) + half.  0: strip = id / slices as usual.
  int pairs_per_group;
  // Test aid (option "handover_test" = 1): producers never raise their flags and the waiting
  // workgroup gives up after a few polls, so that its own fallback computes the result.
  int handover_test;
  // 4-bit weights are unsigned (u4, 0..15) and zero_points, if not null, holds one u4 value per
  // scale ([scale_batch, K/group, N], packed like the weights): W' = (w - z) * scale
  int w_unsigned;
  const uint8_t* zero_points;
  // Ragged dot (lhs [M,K] with its rows sorted by group, weights [groups,K,N]): group_sizes holds
  // `batch` row counts (s32, or s64 when group_sizes_64) in device memory; grid.y walks the groups,
  // group g takes rows [sum of the sizes before it, + its size) of lhs and out, rows past the last
  // group get epilogue(0).  Null for an ordinary (batched) dot.
  const void* group_sizes;
  int group_sizes_64;
  int ragged_groups;  // number of groups (the kernels that do not carry it in grid.y)
  int ragged_chunks;  // (kernels that spread a group's rows over grid.z; the decode kernel walks work items in grid.y)
  // Result and activation layouts beyond bf16 [batch,M,N] / [batch,M,K] (the kernels that honour them
  // store through StoreResult; the launcher keeps every other kernel away from such calls):
  int out_f32;         // out holds f32, not bf16
  int out_transposed;  // out is [batch,N,M]: the dequantised weights were the lhs of the dot
  int lhs_k_major;     // lhs is [batch,K,M] (one-thread-per-output kernels only)
  // out holds f8e4m3fn codes: convert(clamp(-448, v / *d_scale, 448)), or v * *d_scale with d_multiplies
  int out_f8;
  const float* d_scale;
  int d_multiplies;
};

// One result element: row m of batch `batch` (a ragged dot: batch 0, m over all rows), channel n.
static __device__ __forceinline__ void StoreResult(const DecodeParams& p, int batch, int m, int n, float v) {
  size_t idx = ((size_t)batch * (size_t)p.M + (size_t)m) * (size_t)p.N + (size_t)n;
  if (p.out_transposed) idx = ((size_t)batch * (size_t)p.N + (size_t)n) * (size_t)p.M + (size_t)m;
  if (p.out_f8) {
    // op by op as the HLO does: an IEEE quotient (or product), clamp (a NaN stays one), cast
    float c = p.d_multiplies ? v * *p.d_scale : v / *p.d_scale;
    if (c == c) c = __builtin_fminf(__builtin_fmaxf(c, -448.0f), 448.0f);
    reinterpret_cast<uint8_t*>(p.out)[idx] = (uint8_t)f32_to_f8e4m3fn_any(c);
  } else if (p.out_f32) {
    reinterpret_cast<float*>(p.out)[idx] = v;
  } else {
    p.out[idx] = f32_to_bf16(v);
  }
}

// Rows of a ragged dot that group g covers, read on the device: [*begin, *begin + *rows), clamped to
// [0, M] so that sizes that do not add up cannot reach outside the operands.
static __device__ __forceinline__ void ragged_rows(const DecodeParams& p, int g, int* begin, int* rows) {
  long long start = 0;
  for (int i = 0; i < g; ++i)
    start += p.group_sizes_64 ? ((const long long*)p.group_sizes)[i] : (long long)((const int*)p.group_sizes)[i];
  long long n = p.group_sizes_64 ? ((const long long*)p.group_sizes)[g] : (long long)((const int*)p.group_sizes)[g];
  start = start < 0 ? 0 : (start > p.M ? p.M : start);
  n = n < 0 ? 0 : (n > p.M - start ? p.M - start : n);
  *begin = (int)start;
  *rows = (int)n;
}

// Work items of a ragged dot on the streaming kernels: the chunks of ROWS rows of every group, in group
// order (a group of r rows has ceil(r / ROWS) of them: fewer than groups + ceil(M / ROWS) in all).  Every
// wave finds item `item` by itself, 64 groups at a time: lane l reads the size of group g0 + l, two scans
// over the lanes give the rows and the chunks before each group (a serial walk over the sizes, one
// scalar load per group, took longer than the dot itself once there were 64 groups and more).  All 64
// lanes must be active.  *group < 0: the item lies past the last chunk; *last_end: where the rows that
// the groups own end.  Sizes are clamped as in ragged_rows.
// NONNEG: negative sizes count as zero before the rows are summed (the grouped GEMM of the tiled kernel).
template <int ROWS, bool NONNEG = false, class Params = DecodeParams>
static __device__ __forceinline__ void ragged_item(const Params& p, int item, int lane, int* group, int* begin,
                                                   int* rows, int* last_end_out) {
  int seen = 0, g_sel = -1, begin_sel = 0, rows_sel = 0, last_end = 0;
  long long raw_base = 0;  // rows before group g0 as the sizes say
  for (int g0 = 0; g0 < p.ragged_groups; g0 += 64) {
    const int g = g0 + lane;
    const bool valid = g < p.ragged_groups;
    long long n = !valid ? 0 : p.group_sizes_64 ? ((const long long*)p.group_sizes)[g] : (long long)((const int*)p.group_sizes)[g];
    if (NONNEG && n < 0) n = 0;
    long long incl = n;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
      const int lo = __shfl_up((int)(uint32_t)(unsigned long long)incl, off), hi = __shfl_up((int)(uint32_t)((unsigned long long)incl >> 32), off);
      if (lane >= off) incl += (long long)(((unsigned long long)(uint32_t)hi << 32) | (uint32_t)lo);
    }
    const long long raw = raw_base + incl - n;
    const long long first = raw < 0 ? 0 : (raw > p.M ? p.M : raw);
    n = n < 0 ? 0 : (n > p.M - first ? p.M - first : n);
    const int chunks = valid ? ((int)n + ROWS - 1) / ROWS : 0;
    int cincl = chunks;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
      const int t = __shfl_up(cincl, off);
      if (lane >= off) cincl += t;
    }
    const int before = seen + cincl - chunks;
    const bool mine = item >= before && item < before + chunks;
    const unsigned long long hit = __ballot(mine);
    if (hit != 0ull && g_sel < 0) {
      const int src = __builtin_ctzll(hit);
      g_sel = g0 + src;
      begin_sel = __shfl((int)first + (item - before) * ROWS, src);
      rows_sel = __shfl(min((int)n - (item - before) * ROWS, ROWS), src);
    }
    const int last = min(63, p.ragged_groups - 1 - g0);   // the block's last group
    last_end = __shfl((int)(first + n), last);
    seen += __shfl(cincl, 63);
    const int lo = __shfl((int)(uint32_t)(unsigned long long)incl, 63), hi = __shfl((int)(uint32_t)((unsigned long long)incl >> 32), 63);
    raw_base += (long long)(((unsigned long long)(uint32_t)hi << 32) | (uint32_t)lo);
  }
  *group = __builtin_amdgcn_readfirstlane(g_sel);
  *begin = __builtin_amdgcn_readfirstlane(begin_sel);
  *rows = __builtin_amdgcn_readfirstlane(rows_sel);
  *last_end_out = __builtin_amdgcn_readfirstlane(last_end);
}

static __device__ __forceinline__ float load_scale(const void* s, size_t idx, int is_bf16) {
  return is_bf16 ? bf16_to_f32(((const uint16_t*)s)[idx]) : ((const float*)s)[idx];
}

// Buffer descriptor over [base, base+bytes): loads through it return 0 past the end, which is
// how rows beyond K and tokens beyond M drop out of the main loop without any branch.
static __device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* base, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)bytes, 0x00020000);
}

// N32 consecutive dwords (1, 2 or a multiple of 4) at voff + soff.  The hardware range-checks
// the per-lane offset only, so soff must be 0 wherever running past the end is possible.
template <int N32>
static __device__ __forceinline__ void buffer_load_words(__amdgpu_buffer_rsrc_t r, uint32_t voff, uint32_t soff,
                                                  uint32_t* dst) {
  if constexpr (N32 >= 4) {
#pragma unroll
    for (int q = 0; q < N32 / 4; ++q) {
      uintx4 v = __builtin_amdgcn_raw_buffer_load_b128(r, voff + 16 * q, soff, 0);
      dst[4 * q] = v[0]; dst[4 * q + 1] = v[1]; dst[4 * q + 2] = v[2]; dst[4 * q + 3] = v[3];
    }
  } else if constexpr (N32 == 2) {
    uintx2 v = __builtin_amdgcn_raw_buffer_load_b64(r, voff, soff, 0);
    dst[0] = v[0]; dst[1] = v[1];
  } else {
    dst[0] = __builtin_amdgcn_raw_buffer_load_b32(r, voff, soff, 0);
  }
}


// What a raised hand-over flag holds: the launch's epoch in the upper half and the slot's
// generation in the lower.  The generation is a word in the workspace next to the flag(s) that the
// workgroup which waits on the slot increments as the last thing it does, whether the flags showed
// or it gave up waiting: a flag raised late in one run (after the waiting side gave up) can then
// not be taken for the flag of the next run, also when that run is a replay of the same captured
// launch with the same epoch.  Every workgroup reads the generation as it starts (the one that
// increments it does so after its bounded wait, by when every producer has long started).
static __device__ __forceinline__ unsigned long long HandOverTarget(unsigned long long epoch,
                                                                    const unsigned long long* generation) {
  return (epoch << 32) | (__hip_atomic_load(generation, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) & 0xffffffffull);
}
static __device__ __forceinline__ void HandOverNextGeneration(unsigned long long* generation, unsigned long long target) {
  __hip_atomic_store(generation, (target + 1) & 0xffffffffull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
constexpr int kHandOverSpins = 1 << 22;  // polls before the waiting side computes everything itself
constexpr int kHandOverTestSpins = 16;

// A value no earlier launch of this process used and never 0: what the workgroups of one launch
// write into their hand-over flags (HandOverTarget), so that whatever an earlier call (or nobody)
// left in the workspace cannot be mistaken for it.
inline unsigned long long NextHandOverEpoch() {
  static std::atomic<unsigned long long> counter{0};
  static const unsigned long long nonce =
      0x9e3779b97f4a7c15ull * (unsigned long long)(uintptr_t)&counter ^ 0xd1b54a32d192ed03ull;
  return (nonce + 2 * counter.fetch_add(1, std::memory_order_relaxed)) | 1ull;
}

// Sums the K-slices of dp.workspace in slice order and applies scale, bias and activation
// (dequant_dot_decode.hip); mode: kRounded or kFactored.
int LaunchDecodeFinalize(const DecodeParams& dp, int batch, hipStream_t stream, int mode);

// Scratch the tiled prefill kernel uses to split the tiles of its last round along K
// (tiled_dot_mfma.hip); 0 when the shape is not split.
size_t TiledTailWorkspaceBytes(int64_t batch, int64_t M, int64_t K, int64_t N);

// K-slices a decode launch uses for this shape, and the f32 partial sums they need.
int DecodeSlices(int64_t batch, int64_t M, int64_t K, int64_t N, int strips, int64_t row_bytes, int waves);
size_t DequantDotWorkspaceBytes(int64_t batch, int64_t M, int64_t N, int slices);

// s4 weights with bf16 group scales under a bf16-typed multiply (dequant_dot_decode_s4x.hip).
// Returns -1 when the shape is not covered, else the launch status.  dp comes filled except for
// the strip / slice layout.
int LaunchDequantDotDecodeS4x(DecodeParams dp, const XlaAmdDequantDot& p, hipStream_t stream);
// Whether LaunchDequantDotDecodeS4x would split the rows of this shape over two workgroups that hand
// over inside the kernel, and the workspace that takes.
bool S4xPairShape(int64_t batch, int64_t M, int64_t K, int64_t N, int64_t group);
size_t S4xPairWorkspaceBytes(int64_t batch, int64_t M, int64_t N);

// s8 weights with per-channel scales under an f32-typed multiply, up to 16 tokens, small matrices:
// one launch whose K-slices add up inside the kernel (dequant_dot_decode_s8x.hip).  Returns -1 when
// the shape is not covered or the workspace is smaller than S8xWorkspaceBytes (0: shape not covered
// or nothing needed).
int LaunchDequantDotDecodeS8x(DecodeParams dp, const XlaAmdDequantDot& p, hipStream_t stream);
size_t S8xWorkspaceBytes(int64_t batch, int64_t M, int64_t K, int64_t N);

// Weights stored [N,K] (the contracting dimension minor), scales [N] or [N, K/group], any number of
// tokens (dequant_dot_nk.hip).  dp comes filled except for the strip / slice layout.
int LaunchDequantDotNk(DecodeParams dp, const XlaAmdDequantDot& p, hipStream_t stream);
size_t DequantDotNkWorkspaceBytes(int64_t batch, int64_t M, int64_t K, int64_t N, bool four_bit);

}  // namespace xla_amd
#endif  // XLA_AMD_CSRC_DECODE_COMMON_H_
