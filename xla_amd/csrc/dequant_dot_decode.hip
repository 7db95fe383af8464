// Weight-streaming dequantize-dot for decode shapes (M <= 64):
//   out[b,m,n] = epilogue( sum_k lhs[b,m,k] * W'[b,k,n] ),  W' = dequant(w, scale)
// lhs bf16 [M,K]; w s4 (two per byte, low nibble first) or s8, [K,N] with N
// minor; scales per output channel or per group of rows.
//
// The packed weights are the only large operand, so the kernel is a stream
// over W with everything else fused around it: each lane pulls VEC bytes of 8
// consecutive rows straight into registers, dequantises them there, and feeds
// them to v_mfma_f32_16x16x32_bf16 as the 16x32 operand whose 16 rows are 16
// *output channels*; the activations are the 32x16 operand, so one
// instruction produces a [16 channels x 16 tokens] tile.  A lane owns NV
// adjacent channels (the NV values of its VEC-byte chunk), hence NV
// instructions and NV*4 accumulator registers per 16 tokens.  The waves of a
// workgroup split the K range and add their tiles through LDS; an optional
// split of K across workgroups goes through an f32 workspace and a finalize
// kernel, in a fixed order, so results do not depend on scheduling.
//
// Bound: HBM.  Algorithmic bytes: K*N*bits/8 (weights) + scale, bias, lhs and
// out once each.
//
// Two dequantisation modes, following where the matched HLO rounds:
//  * kRounded : multiply(convert(w), broadcast(scale)) is bf16-typed, so every
//    dequantised weight is one RNE rounding of the exact product
//    (fusion_emitter_int4_device_test.cc:93-104 pattern; FloatNormalization,
//    xla/service/cpu/cpu_compiler.cc:804-817).  Done per weight, in registers.
//  * kFactored: the multiply is f32-typed and the scale is constant along K
//    (per output channel).  Integers go through the MFMA exactly and the scale
//    multiplies the f32 sum once.
//  * kGroupFactored: the multiply is f32-typed and the scales change every `group` rows of K
//    (a multiple of 32).  The integers of one group go through the MFMA exactly into a sum of
//    their own, which is folded into the result as sum * scale at the group's last step.  The
//    reference rounds every product w * s to f32 before it adds; factoring the scale out moves
//    each term by at most 2^-24 of itself, the size of the summation-order differences the
//    comparison rule already carries (the bf16-typed multiply rounds to 2^-9 and is never
//    factored).
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include <algorithm>
#include <mutex>

#include "decode_common.h"
#include "device_numerics.h"
#include "launch.h"

namespace xla_amd {
namespace {

// WBITS: 4 or 8.  VEC: bytes a lane reads per row (4, 8, 16).  MT: 16-token tiles.  WAVES: waves
// per workgroup, splitting the workgroup's rows.  SCALE_BF16: element type of the scales.
// GROUP32: the scale group size is a multiple of 32, so the 32 rows of a step share one group
// and the scales are reloaded only when a step starts a new group.
//
// The main loop has no per-lane control flow and no per-lane address arithmetic: every load is
// a buffer load whose lane offset is fixed for the whole kernel and whose row offset is a scalar.
template <int WBITS, int VEC, int MT, int WAVES, int MODE, bool SCALE_BF16, bool GROUP32>
__global__ __launch_bounds__(WAVES * 64) void dequant_dot_decode_kernel(DecodeParams p) {
  constexpr int NV = VEC * 8 / WBITS;   // channels per lane
  constexpr int WORDS = VEC / 4;        // dwords per lane per row
  constexpr int NPW = 32 / WBITS;       // channels per dword
  constexpr int R = NV * 4 * MT;        // accumulator registers per lane
  constexpr int TN = 16 * NV;           // channels per wave tile
  constexpr int SSZ = SCALE_BF16 ? 2 : 4;
  // the waves' tiles are added through LDS kChunk accumulator registers at a time: 64 KiB where
  // the split of a chunk over the waves allows it, so a 64-token tile needs four passes
  constexpr int kChunk = (WAVES == 8 && NV % 4 == 0 && R % 32 == 0) ? 32 : 16;
  __shared__ float lds[WAVES * kChunk * 64];

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // wave-uniform, in an SGPR
  const int li = lane & 15, kb = lane >> 4;
  // Consecutive workgroup ids land on different XCDs (round robin over 8); give each XCD a
  // contiguous range of strips so neighbouring strips, which share cache lines, share an L2.
  int bid = blockIdx.x;
  {
    const int total = gridDim.x;
    if (total % 8 == 0) bid = (bid % 8) * (total / 8) + bid / 8;
  }
  const int slice = bid % p.slices;
  const int strip = bid / p.slices;
  int batch = blockIdx.y;
  // rows of lhs / out this workgroup works on: batch b of an ordinary dot owns rows [b*M, (b+1)*M) of
  // the flattened [batch*M] rows; group b of a ragged dot owns the rows its group sizes say
  int m_begin = batch * p.M, m_rows = p.M, tail_begin = -1;
  if (p.group_sizes) {
    // grid.y walks work items: the chunks of 16 * MT rows of every group, in group order (a group of r
    // rows has ceil(r / (16 MT)) of them: fewer than groups + ceil(M / (16 MT)) in all, which is the
    // grid); an item past the last chunk has nothing to do, and the last item of the grid -- always one
    // of those -- fills the rows no group owns.  The sizes are only known here, on the device.
    int g_sel, begin_sel, rows_sel, last_end;
    ragged_item<16 * MT>(p, (int)blockIdx.y, lane, &g_sel, &begin_sel, &rows_sel, &last_end);
    const int item = blockIdx.y;
    if (item == (int)gridDim.y - 1) tail_begin = last_end;
    batch = g_sel < 0 ? 0 : g_sel;
    m_begin = begin_sel;
    m_rows = rows_sel;
    if (m_rows == 0 && (tail_begin < 0 || tail_begin >= p.M)) return;
  }

  const int n_lane = strip * TN + li * NV;   // first channel of this lane (may be >= N: discarded)
  const uint32_t pitch = (uint32_t)(((size_t)p.N * WBITS) >> 3);  // bytes per row of W
  const __amdgpu_buffer_rsrc_t rw =
      make_rsrc(p.w + (p.weights_shared ? (size_t)0 : (size_t)batch * p.K * pitch), (uint32_t)p.K * pitch);
  // one descriptor per 16-token tile, each ending where the activations end: the per-lane offset
  // is then the same for every tile (token li of the tile) and still range-checks tokens >= M
  __amdgpu_buffer_rsrc_t ra[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int rows = max(m_rows - 16 * mt, 0);
    ra[mt] = make_rsrc(p.lhs + ((size_t)m_begin + (rows ? 16 * mt : 0)) * p.K, (uint32_t)rows * p.K * 2u);
  }
  const int groups = p.K / p.group;
  const __amdgpu_buffer_rsrc_t rs =
      make_rsrc((const char*)p.scales + (size_t)(p.scale_batched ? batch : 0) * groups * p.N * SSZ,
                (uint32_t)groups * p.N * SSZ);
  // a lane whose channels lie beyond N (last strip) gets an offset no buffer reaches: all its
  // loads return zeros and nothing is read outside the operands
  constexpr uint32_t kNowhere = 0x80000000u;
  const bool lane_live = n_lane < p.N;
  const uint32_t voff_w = lane_live ? (uint32_t)(8 * kb) * pitch + (uint32_t)((n_lane * WBITS) >> 3) : kNowhere;
  const uint32_t voff_a = ((uint32_t)li * p.K + 8 * kb) * 2u;
  // rows r = 1..7 of a lane's block of 8 are reached through the scalar offset: K % 8 == 0, so
  // the block is inside the weights exactly when its first row is, which the lane offset checks
  uint32_t soff_w[8];
#pragma unroll
  for (int r = 0; r < 8; ++r) soff_w[r] = (uint32_t)r * pitch;
  const uint32_t voff_s = lane_live ? (uint32_t)n_lane * SSZ : kNowhere;
  // u4 zero points: one nibble per scale, packed like the weights; the lane's NV channels are NV / 8
  // dwords (4-bit weights give a lane at least 8 channels)
  constexpr int ZW = WBITS == 4 ? (NV / 8 > 0 ? NV / 8 : 1) : 1;
  const bool has_zp = WBITS == 4 && p.zero_points != nullptr;
  const __amdgpu_buffer_rsrc_t rz =
      make_rsrc(has_zp ? p.zero_points + (size_t)(p.scale_batched ? batch : 0) * groups * (p.N >> 1) : p.w,
                has_zp ? (uint32_t)groups * (uint32_t)(p.N >> 1) : 0u);
  const uint32_t voff_z = lane_live ? (uint32_t)(n_lane >> 1) : kNowhere;
  // 4-bit values arrive as the f16 number 1024 + u (or 1024 + 16 u): u = w + 8 for s4 (one XOR also
  // flips the nibble's sign bit), u = w for u4; what is subtracted again is 1024 + 8 resp. 1024 + z
  const uint32_t c_even = p.w_unsigned ? 0x64006400u : 0x64086408u;
  const uint32_t c_odd = p.w_unsigned ? 0x64006400u : 0x64806480u;

  floatx4 acc[NV][MT];
#pragma unroll
  for (int j = 0; j < NV; ++j)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[j][mt] = floatx4{0.f, 0.f, 0.f, 0.f};
  // kGroupFactored: acc holds the current group's sum of integers, tot the scaled sums so far; the
  // scales are wanted in the accumulators' layout (register t of instruction j in lane (li, kb) is
  // channel (4 * kb + t) * NV + j of the strip): four runs of NV consecutive channels per lane
  constexpr bool GF = MODE == kGroupFactored;
  static_assert(!GF || GROUP32, "group-factored sums need whole steps per group");
  constexpr int SWG = NV * SSZ / 4;
  floatx4 tot[GF ? NV : 1][GF ? MT : 1];
  uint32_t graw[GF ? 4 : 1][GF ? SWG : 1];
  uint32_t voff_g[4];
  if (GF) {
#pragma unroll
    for (int j = 0; j < NV; ++j)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) tot[j][mt] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      const int n = strip * TN + (4 * kb + t) * NV;
      voff_g[t] = n < p.N ? (uint32_t)n * SSZ : kNowhere;   // N % NV == 0: a run is inside N or not at all
    }
  }

  // the slice is cut into four blocks, one per SIMD; inside a block the age classes follow each other
  const int cls = wave >> 2;
  int k_begin = slice * p.rows_per_slice + (wave & 3) * (p.rows_per_slice >> 2);
#pragma unroll
  for (int c = 0; c < WAVES / 4; ++c)
    if (c < cls) k_begin += p.class_rows[c];
  const int rows_per_wave = p.class_rows[cls];
  const int k_stop = k_begin + rows_per_wave;           // may run past K: those rows load zeros

  // ---- software pipeline: everything step k0+32 needs from memory -- weights, activations
  // and (when it opens a new scale group) the scales -- is requested before the arithmetic
  // of step k0 starts, so a step never waits for a load issued after its own.
  constexpr int SW = NV * SSZ / 4;  // dwords of raw scales per lane
  uint32_t wq[2][8][WORDS];
  uintx4 aq[2][MT];
  uint32_t sraw[2][SW];
  uint32_t zraw[2][ZW];
  float sc[NV];  // kRounded: scale of each owned channel for the current group (s4: see compute)
  float cc[NV];  // s4: the constant term that removes the conversion offset

  // GROUP32: a step opens a new group every `steps_per_group` steps (and at the wave's first)
  const int steps_per_group = GROUP32 ? p.group / 32 : 1;
  auto opens_group = [&](int k0) {  // scalar
    return !GROUP32 || k0 == k_begin || ((k0 >> 5) % steps_per_group) == 0;
  };
  auto closes_group = [&](int k0) {  // scalar: the next step opens a group, or there is no next step
    return k0 + 32 >= k_stop || (((k0 >> 5) + 1) % steps_per_group) == 0;
  };
  auto load_step = [&](int buf, int k0) {
    const uint32_t va = voff_a + (uint32_t)k0 * 2u;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) aq[buf][mt] = __builtin_amdgcn_raw_buffer_load_b128(ra[mt], va, 0, 0);
    if (MODE == kRounded || (WBITS == 4 && has_zp)) {
      if (GROUP32) {
        if (opens_group(k0)) {
          const uint32_t g = (uint32_t)min(k0, p.K - 1) / (uint32_t)p.group;  // scalar
          if (MODE == kRounded) buffer_load_words<SW>(rs, voff_s, g * (uint32_t)p.N * SSZ, sraw[buf]);
          if (WBITS == 4 && has_zp) buffer_load_words<ZW>(rz, voff_z, g * (uint32_t)(p.N >> 1), zraw[buf]);
        }
      } else {
        const uint32_t g = (uint32_t)min(k0 + 8 * kb, p.K - 1) / (uint32_t)p.group;  // per lane
        if (MODE == kRounded) buffer_load_words<SW>(rs, voff_s + g * (uint32_t)p.N * SSZ, 0, sraw[buf]);
        if (WBITS == 4 && has_zp) buffer_load_words<ZW>(rz, voff_z + g * (uint32_t)(p.N >> 1), 0, zraw[buf]);
      }
    }
    const uint32_t vw = voff_w + (uint32_t)k0 * pitch;
#pragma unroll
    for (int r = 0; r < 8; ++r) buffer_load_words<WORDS>(rw, vw, soff_w[r], wq[buf][r]);
  };

  auto compute = [&](int buf, int k0) {
    // activations: 8 consecutive k of token (16*mt + li); tokens >= M read past the buffer -> 0
    uintx4 av[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) av[mt] = aq[buf][mt];
    if (k0 + 32 > p.K) {  // scalar condition: only a step that crosses the end of K
      asm volatile("");   // keeps this one branch: as selects it would cost 4 per tile in every step
      const bool ok = k0 + 8 * kb < p.K;
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
        av[mt] = uintx4{ok ? av[mt][0] : 0u, ok ? av[mt][1] : 0u, ok ? av[mt][2] : 0u, ok ? av[mt][3] : 0u};
    }
    bf16x8 bop[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) bop[mt] = __builtin_bit_cast(bf16x8, av[mt]);
    if (GF && opens_group(k0)) {  // the group's scales: wanted at its last step, four steps of latency to hide in
      asm volatile("");
      const uint32_t g = (uint32_t)min(k0, p.K - 1) / (uint32_t)p.group;
#pragma unroll
      for (int t = 0; t < 4; ++t) buffer_load_words<SWG>(rs, voff_g[t], g * (uint32_t)p.N * SSZ, graw[t]);
    }
    if ((MODE == kRounded || (WBITS == 4 && has_zp)) && opens_group(k0)) {
      asm volatile("");  // a branch, not 2*NV selects per step
#pragma unroll
      for (int j = 0; j < NV; ++j) {
        const uint32_t* raw = sraw[buf];
        float v = 1.0f;  // kFactored: the integers go through as they are
        if (MODE == kRounded)
          v = SCALE_BF16 ? ((j & 1) ? bf16hi_to_f32(raw[j / 2]) : bf16lo_to_f32(raw[j / 2]))
                         : bits_to_f32(raw[SCALE_BF16 ? 0 : j]);
        if (WBITS == 4) {
          // nibble j of a dword arrives as the f16 value 1024 + u (even j) or 1024 + 16u (odd j);
          // with zero point z (8 for s4, where u = w + 8):
          // (u - z)*s = (1024 + u)*s - (1024 + z)*s = (1024 + 16u)*(s/16) - (64 + z)*s, one fma each,
          // exact for any scale with an 8-bit significand and |1040*s| finite
          const float z = has_zp ? (float)((zraw[buf][j / 8] >> (4 * (j % 8))) & 0xfu) : (p.w_unsigned ? 0.0f : 8.0f);
          sc[j] = (j & 1) ? v * 0.0625f : v;
          cc[j] = (j & 1) ? v * -(64.0f + z) : v * -(1024.0f + z);
        } else {
          sc[j] = v;
        }
      }
    }
#pragma unroll
    for (int q = 0; q < WORDS; ++q) {
      if constexpr (WBITS == 4) {
        // Two nibbles become the two f16 halves of one dword in a single three-input bit
        // operation: where the mask is set the result is x ^ C (the nibble with its sign bit
        // flipped: offset binary), elsewhere C (the f16 exponent of 1024).  Masks 0x000f000f /
        // 0x00f000f0 pick nibbles (0,4) / (1,5) of x and (2,6) / (3,7) of x >> 8.  The product
        // with the scale and the removal of the offset are one v_fma_mix_f32 per weight.
        typedef _Float16 halfx2 __attribute__((ext_vector_type(2)));
#pragma unroll
        for (int sel = 0; sel < 4; ++sel) {  // nibble pairs (0,4), (1,5) of x, then (2,6), (3,7) of x >> 8
          halfx2 pr[8];
#pragma unroll
          for (int r = 0; r < 8; ++r) {
            const uint32_t x = sel < 2 ? wq[buf][r][q] : wq[buf][r][q] >> 8;
            pr[r] = __builtin_bit_cast(halfx2, (sel & 1) ? __builtin_amdgcn_bitop3_b32(x, 0x00f000f0u, c_odd, 0x6a)
                                                         : __builtin_amdgcn_bitop3_b32(x, 0x000f000fu, c_even, 0x6a));
          }
#pragma unroll
          for (int half = 0; half < 2; ++half) {
            const int e = sel + 4 * half;
            const int j = q * 8 + e;
            // (a factored multiply without zero points keeps its constants out of registers)
            const bool from_regs = MODE == kRounded || has_zp;
            const float z0 = p.w_unsigned ? 0.0f : 8.0f;
            const float sj = from_regs ? sc[j] : ((e & 1) ? 0.0625f : 1.0f);
            const float cj = from_regs ? cc[j] : ((e & 1) ? -(64.0f + z0) : -(1024.0f + z0));
            float f[8];
#pragma unroll
            for (int r = 0; r < 8; ++r) f[r] = __builtin_fmaf((float)pr[r][half], sj, cj);
            uintx4 a = {pack_bf16x2(f[0], f[1]), pack_bf16x2(f[2], f[3]), pack_bf16x2(f[4], f[5]),
                        pack_bf16x2(f[6], f[7])};
            const bf16x8 aop = __builtin_bit_cast(bf16x8, a);
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
              acc[j][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(aop, bop[mt], acc[j][mt], 0, 0, 0);
          }
        }
      } else {
        uint32_t lo[8];
#pragma unroll
        for (int r = 0; r < 8; ++r) lo[r] = wq[buf][r][q];
#pragma unroll
        for (int e = 0; e < NPW; ++e) {
          const int j = q * NPW + e;
          float f[8];
#pragma unroll
          for (int r = 0; r < 8; ++r) {
            f[r] = (float)(int8_t)((lo[r] >> (8 * e)) & 0xffu);
            if (MODE == kRounded) f[r] = f[r] * sc[j];
          }
          uintx4 a = {pack_bf16x2(f[0], f[1]), pack_bf16x2(f[2], f[3]), pack_bf16x2(f[4], f[5]),
                      pack_bf16x2(f[6], f[7])};
          const bf16x8 aop = __builtin_bit_cast(bf16x8, a);
#pragma unroll
          for (int mt = 0; mt < MT; ++mt)
            acc[j][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(aop, bop[mt], acc[j][mt], 0, 0, 0);
        }
      }
    }
    if (GF && closes_group(k0)) {
      asm volatile("");
#pragma unroll
      for (int j = 0; j < NV; ++j)
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          const float sv = SCALE_BF16 ? ((j & 1) ? bf16hi_to_f32(graw[t][j / 2]) : bf16lo_to_f32(graw[t][j / 2]))
                                      : bits_to_f32(graw[t][SCALE_BF16 ? 0 : j]);
#pragma unroll
          for (int mt = 0; mt < MT; ++mt) {
            tot[j][mt][t] = __builtin_fmaf(acc[j][mt][t], sv, tot[j][mt][t]);
            acc[j][mt][t] = 0.0f;
          }
        }
    }
  };

  if (k_begin < p.K) {
    load_step(0, k_begin);
    for (int k0 = k_begin; k0 < k_stop; k0 += 64) {
      load_step(1, k0 + 32);
      compute(0, k0);
      load_step(0, k0 + 64);
      compute(1, k0 + 32);
    }
  }

  // ---- add the waves' tiles through LDS; in each pass wave w finishes registers
  // [w*RPW, (w+1)*RPW) of the chunk.  Register index r = (mt*4 + t)*NV + j; in the accumulator
  // tile, lane (li, kb) register t of instruction j is channel strip*TN + (4*kb + t)*NV + j,
  // token 16*mt + li.
  constexpr int RPW = kChunk / WAVES;
  constexpr int PASSES = R / kChunk;
  static_assert(R % kChunk == 0 && kChunk % WAVES == 0 && NV % RPW == 0, "reduction split");
  // bias and per-channel scales of every pass are requested now, in one batch, so that no pass
  // waits for memory between its barriers
  float bq[PASSES * RPW], fq[PASSES * RPW], res[PASSES * RPW];
#pragma unroll
  for (int pass = 0; pass < PASSES; ++pass) {
    const int r0 = pass * kChunk + wave * RPW;
    const int n0 = strip * TN + (4 * kb + (r0 / NV) % 4) * NV + r0 % NV;
    const bool live = p.slices == 1 && n0 < p.N;
#pragma unroll
    for (int u = 0; u < RPW; ++u) {
      bq[pass * RPW + u] = live && p.bias ? load_scale(p.bias, n0 + u, p.bias_is_bf16) : 0.0f;
      fq[pass * RPW + u] =
          MODE == kFactored && live
              ? load_scale(p.scales, (size_t)(p.scale_batched ? batch : 0) * p.N + n0 + u, p.scale_is_bf16)
              : 1.0f;
    }
  }
#pragma unroll
  for (int pass = 0; pass < PASSES; ++pass) {
#pragma unroll
    for (int c = 0; c < kChunk; ++c) {
      const int r = pass * kChunk + c;
      const int j = r % NV, mt = (r / NV) / 4, t = (r / NV) % 4;
      float v = GF ? tot[j][mt][t] : acc[j][mt][t];
      lds[(wave * kChunk + c) * 64 + lane] = v;
    }
    __syncthreads();
#pragma unroll
    for (int u = 0; u < RPW; ++u) {
      float s = 0.0f;
#pragma unroll
      for (int w2 = 0; w2 < WAVES; ++w2) s = s + lds[(w2 * kChunk + wave * RPW + u) * 64 + lane];
      res[pass * RPW + u] = MODE == kFactored ? s * fq[pass * RPW + u] : s;
    }
    if (pass + 1 < PASSES) __syncthreads();
  }
  // the epilogue is chosen once for all of the lane's outputs
  if (p.slices == 1) epilogue_all_dispatch<PASSES * RPW>(res, bq, p.epilogue, p.bf16_dot, p.bf16_ops);
#pragma unroll
  for (int pass = 0; pass < PASSES; ++pass) {
    const int r0 = pass * kChunk + wave * RPW;  // first register this wave finished in the pass
    const int j0 = r0 % NV, mt = (r0 / NV) / 4, t = (r0 / NV) % 4;
    const int m = mt * 16 + li;
    const int n0 = strip * TN + (4 * kb + t) * NV + j0;
    if (m >= m_rows || n0 >= p.N) continue;
    if (p.slices > 1) {
      float* dst = p.workspace + (((size_t)batch * p.slices + slice) * p.M + m) * p.N + n0;
#pragma unroll
      for (int u = 0; u < RPW; ++u) dst[u] = res[pass * RPW + u];
    } else {
      if (p.out_f32 | p.out_transposed | p.out_f8) {
#pragma unroll
        for (int u = 0; u < RPW; ++u) StoreResult(p, p.group_sizes ? 0 : batch, p.group_sizes ? m_begin + m : m, n0 + u, res[pass * RPW + u]);
        continue;
      }
      uint16_t* dst = p.out + ((size_t)m_begin + m) * p.N + n0;
#pragma unroll
      for (int u = 0; u < RPW; ++u) dst[u] = f32_to_bf16(res[pass * RPW + u]);
    }
  }
  // ragged dot: rows past the last group are a dot of nothing -- epilogue(0) in this strip's channels
  if (tail_begin >= 0 && tail_begin < p.M) {
    const int tail_rows = p.M - tail_begin;
    for (int idx = threadIdx.x; idx < tail_rows * TN; idx += WAVES * 64) {
      const int n = strip * TN + idx % TN, m = tail_begin + idx / TN;
      if (n >= p.N) continue;
      const float b = p.bias ? load_scale(p.bias, n, p.bias_is_bf16) : 0.0f;
      p.out[(size_t)m * p.N + n] = f32_to_bf16(epilogue_dispatch(0.0f, b, p.epilogue, p.bf16_dot, p.bf16_ops));
    }
  }
}

// Sums the K-slices of the workspace in slice order and applies scale/bias/activation.
__global__ __launch_bounds__(256) void dequant_dot_finalize_kernel(DecodeParams p, int mode) {
  const size_t total = (size_t)p.M * p.N;
  const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
  const int batch = blockIdx.y;
  if (idx >= total) return;
  const int n = (int)(idx % p.N);
  const float* ws = p.workspace + (size_t)batch * p.slices * total + idx;
  float v = 0.0f;
  for (int s = 0; s < p.slices; ++s) v = v + ws[(size_t)s * total];
  if (mode == kFactored)
    v = v * load_scale(p.scales, (size_t)(p.scale_batched ? batch : 0) * p.N + n, p.scale_is_bf16);
  const float b = p.bias ? load_scale(p.bias, n, p.bias_is_bf16) : 0.0f;
  StoreResult(p, batch, (int)(idx / p.N), n, epilogue_dispatch(v, b, p.epilogue, p.bf16_dot, p.bf16_ops));
}

// Any shape, any alignment: one thread per output, k in increasing order.  Correct for every
// case the handlers accept; used when the streaming kernels' divisibility rules do not hold
// and for grouped scales with an f32-typed multiply.
__global__ __launch_bounds__(256) void dequant_dot_generic_kernel(DecodeParams p, int wbits, int mode) {
  const size_t total = (size_t)p.M * p.N;
  const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
  const int batch = blockIdx.y;
  if (idx >= total) return;
  const int n = (int)(idx % p.N), m = (int)(idx / p.N);
  // ragged dot (launched with one batch): the row's group picks the weights; rows no group owns add nothing
  int wbatch = batch, k_end = p.K;
  if (p.group_sizes) {
    k_end = 0;
    for (int g = 0; g < p.ragged_groups; ++g) {
      int b0, rows;
      ragged_rows(p, g, &b0, &rows);
      if (m >= b0 && m < b0 + rows) { wbatch = g; k_end = p.K; break; }
    }
  }
  // activations [batch,M,K], or [batch,K,M] when the dot contracts their major dimension
  const uint16_t* a = p.lhs + (p.lhs_k_major ? (size_t)batch * p.M * p.K + m : ((size_t)batch * p.M + m) * p.K);
  const size_t a_step = p.lhs_k_major ? (size_t)p.M : 1;
  const size_t wbase = (size_t)wbatch * p.K * p.N;
  const size_t sbase = (size_t)(p.scale_batched ? wbatch : 0) * (p.K / p.group) * p.N;
  float acc = 0.0f;
  for (int k = 0; k < k_end; ++k) {
    const size_t e = wbase + (size_t)k * p.N + n;
    int wi;
    if (wbits == 8) {
      wi = (int8_t)p.w[e];
    } else {
      const uint32_t nib = (p.w[e >> 1] >> (4 * (e & 1))) & 0xfu;
      wi = p.w_unsigned ? (int)nib : (int)(nib ^ 8u) - 8;
      if (p.zero_points) {
        const size_t ze = sbase + (size_t)(k / p.group) * p.N + n;
        wi -= (int)((p.zero_points[ze >> 1] >> (4 * (ze & 1))) & 0xfu);
      }
    }
    float s = load_scale(p.scales, sbase + (size_t)(k / p.group) * p.N + n, p.scale_is_bf16);
    float wv = (float)wi * s;
    if (mode == kRounded) wv = round_bf16(wv);
    acc = acc + bf16_to_f32(a[(size_t)k * a_step]) * wv;
  }
  const float b = p.bias ? load_scale(p.bias, n, p.bias_is_bf16) : 0.0f;
  StoreResult(p, batch, m, n, epilogue_dispatch(acc, b, p.epilogue, p.bf16_dot, p.bf16_ops));
}

template <int WBITS, int VEC, int MT, int WAVES, int MODE>
int launch_decode(const DecodeParams& dp, int batch, hipStream_t stream, const char* name) {
  void (*kern)(DecodeParams) = nullptr;
  const bool g32 = dp.group % 32 == 0;
  if constexpr (MODE == kFactored)  // the main loop never touches the scales
    kern = dequant_dot_decode_kernel<WBITS, VEC, MT, WAVES, MODE, true, true>;
  else if constexpr (MODE == kGroupFactored)  // groups of whole steps only
    kern = dp.scale_is_bf16 ? dequant_dot_decode_kernel<WBITS, VEC, MT, WAVES, MODE, true, true>
                            : dequant_dot_decode_kernel<WBITS, VEC, MT, WAVES, MODE, false, true>;
  else if (dp.scale_is_bf16)
    kern = g32 ? dequant_dot_decode_kernel<WBITS, VEC, MT, WAVES, MODE, true, true>
               : dequant_dot_decode_kernel<WBITS, VEC, MT, WAVES, MODE, true, false>;
  else
    kern = g32 ? dequant_dot_decode_kernel<WBITS, VEC, MT, WAVES, MODE, false, true>
               : dequant_dot_decode_kernel<WBITS, VEC, MT, WAVES, MODE, false, false>;
  // (a ragged dot: one grid row per chunk of 16 * MT rows any group can have, and one for the rows nobody owns)
  const unsigned rows_y = dp.group_sizes ? (unsigned)(batch + (dp.M + 16 * MT - 1) / (16 * MT)) : (unsigned)batch;
  dim3 grid((unsigned)(dp.strips * dp.slices), rows_y, 1u);
  hipLaunchKernelGGL(kern, grid, dim3(WAVES * 64), 0, stream, dp);
  int rc = CheckLaunch(name);
  if (rc) return rc;
  if (dp.slices > 1) {
    dim3 fgrid((unsigned)(((size_t)dp.M * dp.N + 255) / 256), (unsigned)batch);
    hipLaunchKernelGGL(dequant_dot_finalize_kernel, fgrid, dim3(256), 0, stream, dp, MODE);
    rc = CheckLaunch("dequant_dot_finalize");
  }
  SetLastKernel(name);
  return rc;
}

}  // namespace

int LaunchDecodeFinalize(const DecodeParams& dp, int batch, hipStream_t stream, int mode) {
  dim3 fgrid((unsigned)(((size_t)dp.M * dp.N + 255) / 256), (unsigned)batch);
  hipLaunchKernelGGL(dequant_dot_finalize_kernel, fgrid, dim3(256), 0, stream, dp, mode);
  return CheckLaunch("dequant_dot_finalize");
}

int LaunchDequantDotPrefill(const XlaAmdDequantDot& p, hipStream_t stream);  // tiled_dot_mfma.hip

// Rows of K each workgroup takes so that `slices` workgroups cover K; multiple of 64*waves.
static int RowsPerSlice(int K, int slices, int waves) {
  const int unit = 64 * waves;
  const int per = (K + slices - 1) / slices;
  return (per + unit - 1) / unit * unit;
}

// Splits a SIMD's quarter of a slice between its waves' age classes in proportion to weights
// (option "dequant_dot_skew": four decimal digits, oldest class first; 0 = the default), in units
// of 64 rows; the youngest class takes what rounding leaves.
static void ClassRows(int rows_per_slice, int waves, int* out) {
  const int classes = waves / 4;
  const int units = rows_per_slice / 4 / 64;  // 64-row units per SIMD block, a multiple of `classes`
  // Defaults from a sweep on 8192 x 28672 s4: with equal shares the four waves of a SIMD left the
  // main loop at 11.7, 15.8, 20.2 and 24.5 us (in-kernel clock), the last one running alone at a
  // little over half the SIMD's rate; 4:3:2:1 brings 1 token from 28.3 to 25.9 us, 3:2 for two
  // classes 32 tokens from 38.0 to 36.8 (64 tokens: no change, one wave already fills the SIMD).
  int w[4] = {1, 1, 1, 1};
  if (classes == 4) { w[0] = 4; w[1] = 3; w[2] = 2; w[3] = 1; }
  if (classes == 2) { w[0] = 3; w[1] = 2; }
  if (int v = GetOption("dequant_dot_skew")) {
    w[0] = v / 1000 % 10; w[1] = v / 100 % 10; w[2] = v / 10 % 10; w[3] = v % 10;
    if (classes == 2) { w[0] = v / 10 % 10; w[1] = v % 10; }
  }
  int total = 0;
  for (int c = 0; c < classes; ++c) total += w[c] > 0 ? w[c] : (w[c] = 1);
  int left = units;
  for (int c = 0; c < 4; ++c) out[c] = 0;
  for (int c = 0; c < classes; ++c) {
    int u = c + 1 == classes ? left : (units * w[c] + total / 2) / total;
    if (u > left) u = left;
    out[c] = u * 64;
    left -= u;
  }
}

size_t DequantDotWorkspaceBytes(int64_t batch, int64_t M, int64_t N, int slices) {
  return slices > 1 ? (size_t)batch * slices * M * N * sizeof(float) : 0;
}

// K-slices for a decode launch.  One workgroup per CU is enough once the strips alone give about
// that many (the kernel is bound by its own arithmetic, and every extra slice costs partial sums
// and a second launch).  Fewer strips are split
// until there are, as long as a wave keeps at least four 32-row steps and the partial sums
// (slices*M*N*4 bytes written and read again) stay small: at most 32 rows of them, or half a byte
// per weight whatever the weights' width -- above 16 tokens the kernels are bound by their arithmetic,
// which 4-bit weights do not halve (s8 [64,8192] x [8192,8192]: 44 us in one slice, 30 in two;
// s4 [64,14336] x [14336,4096]: 36 us in two slices, 24 in eight; [64,4096] x [4096,4096]: 23 -> 17).
int DecodeSlices(int64_t batch, int64_t M, int64_t K, int64_t N, int strips, int64_t row_bytes, int waves) {
  if (int s = GetOption("dequant_dot_slices")) return s;
  // (two workgroups per CU up to four tokens, the rule of an earlier kernel generation, costs the
  // current ones 15-30 % on mid-sized matrices: s4 8192 x 8192 at one token 16.6 us in 8 slices, 12.5 in 4)
  const int64_t want = 192;
  (void)row_bytes;
  const double budget = 0.5 * (double)K * (double)N;
  int slices = 1;
  while (strips * slices * batch < want && K / (slices * 2) >= 128 * waves &&
         (slices * 2 * M <= 32 || 2.0 * (slices * 2) * M * N * 4.0 <= budget))
    slices *= 2;
  // a few workgroups more than CUs are worse than half as many: a second round for a quarter of the work
  if (slices > 1 && strips * batch * slices > 256 && strips * batch * slices < 400) slices /= 2;
  return slices;
}

// What xla_amd_dequant_dot_workspace_bytes reports: the scratch the launch below will use for
// this shape (the narrowest strips give the most slices), or what a forced slice count needs.
static size_t DecodeWorkspaceBytesUpTo64(int64_t batch, int64_t M, int64_t K, int64_t N, bool s4) {
  if (M <= 0 || M > 64 || K < 32 || N <= 0 || batch <= 0) return 0;
  const int mt = M <= 16 ? 1 : M <= 32 ? 2 : M <= 48 ? 3 : 4;
  int vec = s4 ? 4 : (mt >= 3 ? 4 : 8);
  if (int v = GetOption("dequant_dot_vec")) vec = v;
  const int nv = vec * (s4 ? 2 : 1);
  const int64_t row_bytes = N * (s4 ? 1 : 2) / 2;
  const int strips = (int)((N + 16 * nv - 1) / (16 * nv));
  size_t bytes = DequantDotWorkspaceBytes(batch, M, N, DecodeSlices(batch, M, K, N, strips, row_bytes, 8));
  // (s8 from 33 tokens on: per-channel scales under an f32 multiply take 128-channel strips, whose
  // fewer workgroups may be split further; the mode is not known here, the larger need decides)
  if (!s4 && mt >= 3 && !GetOption("dequant_dot_vec")) {
    const size_t wide = DequantDotWorkspaceBytes(batch, M, N, DecodeSlices(batch, M, K, N, (int)((N + 127) / 128), row_bytes, 8));
    if (wide > bytes) bytes = wide;
  }
  // s4 up to 16 tokens may run as two workgroups per 256-channel strip that hand over through the
  // workspace (the group size is not known here: the smallest one that path takes decides)
  if (s4 && S4xPairShape(batch, M, K, N, 64)) bytes = bytes > S4xPairWorkspaceBytes(batch, M, N) ? bytes : S4xPairWorkspaceBytes(batch, M, N);
  // small s8 matrices up to 16 tokens: the slices of a strip hand over inside the kernel
  if (!s4 && S8xWorkspaceBytes(batch, M, K, N) > bytes) bytes = S8xWorkspaceBytes(batch, M, K, N);
  return bytes;
}

size_t DequantDotDecodeWorkspaceBytes(int64_t batch, int64_t M, int64_t K, int64_t N, bool s4) {
  if (M <= 64) return DecodeWorkspaceBytesUpTo64(batch, M, K, N, s4);
  // More than 64 tokens on the decode kernels: per batch, all whole chunks of 64 tokens (32 for
  // 4-bit weights under group-factored sums: the mode is not known here, the larger need decides)
  // as one launch with the chunk index as its batch, then the remaining tokens as a second launch;
  // the launches follow each other on the stream and share the scratch.
  size_t bytes = 0;
  for (int64_t chunk = 64; chunk >= (s4 ? 32 : 64); chunk /= 2) {
    const size_t whole = DecodeWorkspaceBytesUpTo64(M / chunk, chunk, K, N, s4);
    const size_t rest = DecodeWorkspaceBytesUpTo64(1, M % chunk, K, N, s4);
    bytes = bytes > whole ? bytes : whole;
    bytes = bytes > rest ? bytes : rest;
  }
  return bytes;
}

// Ragged dot without a single group: every row is a dot of nothing, epilogue(0 [+ bias]).
__global__ __launch_bounds__(256) void ragged_no_groups_kernel(DecodeParams p) {
  const int n = blockIdx.x * 256 + threadIdx.x;
  if (n >= p.N) return;
  const float bias = p.bias ? load_scale(p.bias, n, p.bias_is_bf16) : 0.0f;
  const uint16_t v = f32_to_bf16(epilogue_dispatch(0.0f, bias, p.epilogue, p.bf16_dot, p.bf16_ops));
  for (int m = blockIdx.y; m < p.M; m += gridDim.y) p.out[(size_t)m * p.N + n] = v;
}

// weights_shared: `batch` counts 64-token chunks of one [batch * M, K] activation matrix that all
// use the same weights and scales (only the decode kernels take it).
static int LaunchDequantDotImpl(const XlaAmdDequantDot& p, hipStream_t stream, bool weights_shared) {
  const bool u4 = p.weight_dtype == XLA_FFI_DataType_U4;
  const bool s4 = p.weight_dtype == XLA_FFI_DataType_S4 || u4;  // 4-bit weights, two per byte
  if (!s4 && p.weight_dtype != XLA_FFI_DataType_S8)
    return Fail(XLA_FFI_Error_Code_INVALID_ARGUMENT, "dequant_dot: weights must be S4, U4 or S8");
  if (p.zero_points && !u4)
    return Fail(XLA_FFI_Error_Code_INVALID_ARGUMENT, "dequant_dot: zero points come with U4 weights only");
  if (!IsF32OrBf16(p.scale_dtype) || !IsF32OrBf16(p.dequant_type) || !IsF32OrBf16(p.dot_type) ||
      !IsF32OrBf16(p.epilogue_type) || (p.bias && !IsF32OrBf16(p.bias_dtype)))
    return Fail(XLA_FFI_Error_Code_INVALID_ARGUMENT, "dequant_dot: types must be F32 or BF16");
  if (p.batch < 0 || p.M < 0 || p.K < 0 || p.N < 0 || p.M > 0x7fffffff || p.K > 0x7fffffff ||
      p.N > 0x7fffffff || p.batch > 65535)
    return Fail(XLA_FFI_Error_Code_INVALID_ARGUMENT, "dequant_dot: bad shape");
  if (p.K > 0 && (p.group <= 0 || p.K % p.group != 0))
    return Fail(XLA_FFI_Error_Code_INVALID_ARGUMENT,
                "dequant_dot: group size %lld does not divide K=%lld", (long long)p.group,
                (long long)p.K);
  if (p.epilogue < 0 || p.epilogue > XLA_AMD_EPI_BIAS_SILU)
    return Fail(XLA_FFI_Error_Code_INVALID_ARGUMENT, "dequant_dot: unknown epilogue %d", p.epilogue);
  if ((p.epilogue & 1) && !p.bias)
    return Fail(XLA_FFI_Error_Code_INVALID_ARGUMENT, "dequant_dot: BIAS epilogue without a bias");
  if (p.scale_batch != 1 && p.scale_batch != p.batch)
    return Fail(XLA_FFI_Error_Code_INVALID_ARGUMENT, "dequant_dot: scale batch must be 1 or batch");
  if (p.dequant_type == XLA_FFI_DataType_BF16 && p.scale_dtype != XLA_FFI_DataType_BF16)
    return Fail(XLA_FFI_Error_Code_INVALID_ARGUMENT,
                "dequant_dot: a bf16-typed dequantise multiply needs bf16 scales");
  if (p.batch == 0 && (p.group_sizes || p.group_sizes_dtype != 0) && p.M > 0 && p.N > 0) {
    // a ragged dot over no groups: no row has a group, so every row is epilogue(0 [+ bias])
    if (!p.out || ((p.epilogue & 1) && !p.bias))
      return Fail(XLA_FFI_Error_Code_INVALID_ARGUMENT, "dequant_dot: null buffer");
    if (p.out_dtype != 0 && p.out_dtype != XLA_FFI_DataType_BF16)
      return Fail(XLA_FFI_Error_Code_UNIMPLEMENTED, "dequant_dot: a ragged dot writes bf16 [M,N] from lhs [M,K]");
    DecodeParams fp = {};
    fp.out = (uint16_t*)p.out;
    fp.bias = (p.epilogue & 1) ? p.bias : nullptr;
    fp.bias_is_bf16 = p.bias_dtype == XLA_FFI_DataType_BF16;
    fp.bf16_dot = p.dot_type == XLA_FFI_DataType_BF16;
    fp.bf16_ops = p.epilogue_type == XLA_FFI_DataType_BF16;
    fp.epilogue = p.epilogue;
    fp.M = (int)p.M; fp.N = (int)p.N;
    const unsigned rows = (unsigned)(p.M < 64 ? p.M : 64);
    hipLaunchKernelGGL(ragged_no_groups_kernel, dim3((unsigned)((p.N + 255) / 256), rows), dim3(256), 0, stream, fp);
    SetLastKernel("dequant_dot:ragged_no_groups");
    return CheckLaunch("dequant_dot_ragged_no_groups");
  }
  if (p.batch == 0 || p.M == 0 || p.N == 0) {
    SetLastKernel("dequant_dot:empty");
    return 0;
  }
  if (!p.lhs || !p.weights || !p.scales || !p.out)
    return Fail(XLA_FFI_Error_Code_INVALID_ARGUMENT, "dequant_dot: null buffer");

  DecodeParams dp;
  dp.lhs = (const uint16_t*)p.lhs;
  dp.w = (const uint8_t*)p.weights;
  dp.scales = p.scales;
  dp.bias = (p.epilogue & 1) ? p.bias : nullptr;
  dp.out = (uint16_t*)p.out;
  dp.workspace = (float*)p.workspace;
  dp.M = (int)p.M; dp.K = (int)p.K; dp.N = (int)p.N;
  dp.group = p.K > 0 ? (int)p.group : 1;
  dp.scale_is_bf16 = p.scale_dtype == XLA_FFI_DataType_BF16;
  dp.bias_is_bf16 = p.bias_dtype == XLA_FFI_DataType_BF16;
  dp.scale_batched = p.scale_batch == p.batch && p.batch > 1;
  dp.bf16_dot = p.dot_type == XLA_FFI_DataType_BF16;
  dp.bf16_ops = p.epilogue_type == XLA_FFI_DataType_BF16;
  dp.epilogue = p.epilogue;
  dp.strips = 1; dp.slices = 1; dp.rows_per_slice = 0;
  dp.weights_shared = weights_shared;
  dp.handover_test = GetOption("handover_test");
  if (p.out_dtype != 0 && p.out_dtype != XLA_FFI_DataType_BF16 && p.out_dtype != XLA_FFI_DataType_F32 &&
      p.out_dtype != XLA_FFI_DataType_F8E4M3FN)
    return Fail(XLA_FFI_Error_Code_INVALID_ARGUMENT, "dequant_dot: out must be BF16, F32 or F8E4M3FN");
  dp.out_f32 = p.out_dtype == XLA_FFI_DataType_F32;
  dp.out_f8 = p.out_dtype == XLA_FFI_DataType_F8E4M3FN;
  dp.d_scale = p.d_scale;
  dp.d_multiplies = p.d_scale_multiplies != 0;
  if (dp.out_f8 && !p.d_scale)
    return Fail(XLA_FFI_Error_Code_INVALID_ARGUMENT, "dequant_dot: an F8E4M3FN result needs d_scale");
  dp.out_transposed = p.out_transposed != 0;
  dp.lhs_k_major = p.lhs_k_major != 0;
  // A result other than bf16 [batch,M,N], or activations stored [batch,K,M], keep the call on the
  // kernels that store through StoreResult / read lhs with a stride: the first-generation decode
  // kernel (and its token chunks), the [N,K] streaming kernel and the one-thread-per-output kernels.
  const bool plain = !dp.out_f32 && !dp.out_f8 && !dp.out_transposed && !dp.lhs_k_major;
  if (!plain && p.group_sizes)
    return Fail(XLA_FFI_Error_Code_UNIMPLEMENTED, "dequant_dot: a ragged dot writes bf16 [M,N] from lhs [M,K]");
  dp.w_unsigned = u4;
  dp.zero_points = (const uint8_t*)p.zero_points;
  const bool ragged = p.group_sizes != nullptr;
  if (ragged && p.group_sizes_dtype != XLA_FFI_DataType_S32 && p.group_sizes_dtype != XLA_FFI_DataType_S64)
    return Fail(XLA_FFI_Error_Code_INVALID_ARGUMENT, "dequant_dot: group sizes must be S32 or S64");
  if (ragged && weights_shared) return Fail(XLA_FFI_Error_Code_INTERNAL, "dequant_dot: ragged token chunks");
  dp.group_sizes = p.group_sizes;
  dp.group_sizes_64 = p.group_sizes_dtype == XLA_FFI_DataType_S64;
  dp.ragged_groups = ragged ? (int)p.batch : 0;
  dp.ragged_chunks = 1;
  if (ragged && p.batch + (p.M + 15) / 16 > 65535)
    return Fail(XLA_FFI_Error_Code_UNIMPLEMENTED, "dequant_dot: a ragged dot takes at most 65535 groups plus 16-row chunks");
  if (p.rhs_contracting_dim != 0 && p.rhs_contracting_dim != 1)
    return Fail(XLA_FFI_Error_Code_INVALID_ARGUMENT, "dequant_dot: rhs_contracting_dim must be 0 or 1");
  if (p.rhs_contracting_dim == 1) {  // weights [N,K]
    if (ragged) dp.scale_batched = p.scale_batch == p.batch;  // one set of scales per group, also for a single group
    return LaunchDequantDotNk(dp, p, stream);
  }
  const bool per_channel = p.group == p.K;
  // f32-typed multiply: one scale per channel factors out of the whole sum, scales per group of whole
  // 32-row steps out of each group's sum; anything else under an f32 multiply takes the generic kernel
  const int mode = p.dequant_type == XLA_FFI_DataType_BF16 ? kRounded
                   : per_channel || p.group % 32 != 0     ? kFactored
                                                          : kGroupFactored;

  const int force = GetOption("dequant_dot_kernel");  // 0 auto, 1 generic, 2 decode, 3 prefill
  const bool aligned = p.K % 8 == 0 && p.group % 8 == 0 && ((uintptr_t)p.lhs % 16 == 0) &&
                       ((uintptr_t)p.weights % 16 == 0);
  const bool mode_ok = mode == kRounded || mode == kGroupFactored || per_channel;

  // A ragged dot takes the tiled kernel (a grouped GEMM: 256-row tiles per group) where its tiles cost
  // less than the 64-row chunks of the decode kernel.  The sizes themselves are only known on the
  // device, so both sides are priced on the average group: a group of r rows has r / 64 + 0.5 chunks
  // and max(1, r / 256 + 0.5) tiles on average.  A chunk streams one expert matrix (2.4e-7 us per s8
  // weight, 2.0e-7 per 4-bit one, 0.25-0.3 us per work item); 256 tiles run at a time and take
  // 25 + 0.025 K us.  Measured on MI355X, 96 rows per expert, chunks against tiles: 8 experts of
  // 14336 x 4096 s8 218 us / 327, s4 160 / 343; 16 of 4096 x 14336 s8 457 / 471, s4 386 / 503; 128 of
  // 2048 x 1536 s8 269 / 227.  Below 64 rows per expert most of a tile would be empty.
  bool ragged_tiles = ragged && force == 3;
  if (ragged && force == 0 && p.batch > 0 && p.M / p.batch >= 64) {
    const double rows = (double)p.M / (double)p.batch, kn = (double)p.K * (double)p.N;
    const double chunks_us = (double)p.batch * (rows / 64.0 + 0.5) * (s4 ? 2.0e-7 * kn + 0.3 : 2.4e-7 * kn + 0.25);
    const double tiles = (double)p.batch * std::max(1.0, rows / 256.0 + 0.5) * (double)((p.N + 255) / 256);
    const double tiles_us = std::max(1.0, tiles / 256.0) * (25.0 + 0.025 * (double)p.K) * (s4 ? 1.05 : 1.0);
    ragged_tiles = tiles_us < chunks_us;
  }
  if (plain && force != 1 && force != 2 && aligned && mode_ok && p.M > 64 && !weights_shared && (!ragged || ragged_tiles)) {
    int rc = LaunchDequantDotPrefill(p, stream);
    if (rc >= 0) return rc;  // -1: shape not covered by the tiled kernel, fall through
  }

  // Strip layout of the decode kernels for M tokens, and whether this shape fits them.
  // VEC bytes per lane per row -> NV channels per lane; needs N % NV == 0 and 16-byte rows
  auto decode_shape = [&](int64_t M, int* mt_out, int* vec_out, int* nv_out) {
    const int mt = M <= 16 ? 1 : M <= 32 ? 2 : M <= 48 ? 3 : 4;  // 16-token tiles
    // Narrow strips (4 bytes of s4 = 8 channels, 8 bytes of s8 per lane) measured fastest on
    // MI355X: the loop is bound by the dequantising VALU work, not by load width, and narrow
    // strips give more workgroups to spread over the 256 CUs.  s8 from 33 tokens on took 4 bytes
    // per lane (64-byte pieces of every row) until the factored and rounded modes got their 8-byte forms:
    // [64,8192] x [8192,28672] 87.5 -> 58.5 us, 48 tokens 76 -> 49.
    // (fewer than 64 such strips leave the narrow ones ahead: more workgroups; 4096 x 4096 at 64 tokens
    // 17.5 us against 22.6)
    // (the group-factored form of 8 bytes per lane at three or four token tiles spills 61-329 registers)
    int vec = s4 ? 4 : (mt >= 3 && (mode == kGroupFactored || p.N % 8 != 0 || (p.N + 127) / 128 * p.batch < 64) ? 4 : 8);
    if (int v = GetOption("dequant_dot_vec")) vec = v;
    const int nv = vec * (s4 ? 2 : 1);
    const int64_t row_bytes = p.N * (s4 ? 1 : 2) / 2;
    // buffer offsets are 32-bit: keep every operand (plus one loop overrun) below 2 GiB
    const bool fits32 = (double)p.K * row_bytes + 1024.0 * row_bytes < 2147483648.0 &&
                        (double)M * p.K * 2 < 2147483648.0 &&
                        (double)(p.K / p.group) * p.N * 4 < 2147483648.0;
    *mt_out = mt; *vec_out = vec; *nv_out = nv;
    return p.N % nv == 0 && row_bytes % vec == 0 && nv * mt <= 32 && (vec == 4 || vec == 8 || vec == 16) && fits32;
  };

  // More than 64 tokens on weights the tiled kernel does not take (s4, grouped scales): the
  // decode kernel runs once per 64 tokens (and per batch).  Every token row is computed exactly as
  // in a call of its own, so the chunks compose bit for bit; each pass streams the weights again,
  // which at 8192 x 28672 s4 still reaches 0.55 PFLOP/s against 2-3 TFLOP/s of the generic kernel.
  int mt64, vec64, nv64;
  // (4-bit weights with group-factored sums hold two sets of accumulators per tile: chunks of 32 tokens)
  const int64_t chunk = mode == kGroupFactored && s4 ? 32 : 64;
  if (force != 1 && force != 3 && aligned && mode_ok && p.M > chunk && p.K >= 32 && p.N % 2 == 0 && !ragged &&
      !dp.out_transposed && !dp.lhs_k_major && decode_shape(chunk, &mt64, &vec64, &nv64)) {
    const size_t wbytes = (size_t)p.K * p.N * (s4 ? 1 : 2) / 2;
    const size_t ssz = p.scale_dtype == XLA_FFI_DataType_BF16 ? 2 : 4;
    const size_t sbytes = p.scale_batch == p.batch && p.batch > 1 ? (size_t)(p.K / p.group) * p.N * ssz : 0;
    XlaAmdDequantDot sub = p;
    sub.batch = 1;
    sub.scale_batch = 1;
    char name[128] = "";
    for (int64_t b = 0; b < p.batch; ++b) {
      sub.weights = (const char*)p.weights + b * wbytes;
      sub.scales = (const char*)p.scales + b * sbytes;
      if (p.zero_points)  // one nibble per scale
        sub.zero_points = (const char*)p.zero_points + (sbytes ? b * ((size_t)(p.K / p.group) * p.N / 2) : 0);
      // the whole 64-token chunks go out as one launch with the chunk index in the grid (the
      // workgroups of all chunks then pack onto the CUs together), the remainder as a second one
      const int64_t whole = p.M / chunk;
      for (int part = 0; part < 2; ++part) {
        const int64_t m0 = part == 0 ? 0 : whole * chunk;
        sub.M = part == 0 ? chunk : p.M - m0;
        sub.batch = part == 0 ? whole : 1;
        if (sub.M == 0 || sub.batch == 0) continue;
        sub.lhs = (const uint16_t*)p.lhs + ((size_t)b * p.M + m0) * p.K;
        sub.out = (char*)p.out + ((size_t)b * p.M + m0) * p.N * (dp.out_f32 ? 4 : dp.out_f8 ? 1 : 2);
        const int rc = LaunchDequantDotImpl(sub, stream, true);
        if (rc) return rc;
        if (!name[0]) snprintf(name, sizeof(name), "%s:x%d", xla_amd_last_kernel(), (int)chunk);
      }
    }
    SetLastKernel(name);
    return 0;
  }

  if (force != 1 && force != 3 && aligned && mode_ok && (p.M <= chunk || ragged) && p.K >= 32 && !dp.lhs_k_major) {
    int mt, vec, nv;
    // A ragged dot works in chunks of 16 * mt rows of one group: sized for twice the average group, so
    // that few groups need a second chunk (every chunk streams its group's weights) and the many small
    // ones do not pay for empty token tiles (64 experts, 128 rows: 175 us with 64-row chunks, 37-50 with 16).
    int64_t tile_rows = p.M > 64 ? 64 : p.M;
    if (ragged && p.batch > 0) {
      const int64_t twice = 2 * ((p.M + p.batch - 1) / p.batch);
      tile_rows = twice < tile_rows ? twice : tile_rows;
      if (tile_rows < 1) tile_rows = 1;
      // (three token tiles lose to two with a second chunk for the larger groups: 64 experts [4096,2816],
      // 24 rows each, 174 us against 160)
      if (tile_rows > 32 && tile_rows <= 48) tile_rows = 32;
      if (int v = GetOption("dequant_dot_ragged_tile")) tile_rows = v < tile_rows ? v : tile_rows;
    }
    const bool shape_ok = decode_shape(tile_rows, &mt, &vec, &nv);
    const int64_t row_bytes = p.N * (s4 ? 1 : 2) / 2;
    // s4 with bf16 group scales and a bf16-typed multiply: the kernels that dequantise through the
    // 4x4x4 matrix instruction
    if (shape_ok && plain && s4 && mode == kRounded && GetOption("dequant_dot_x") != 1 && !ragged) {
      const int rc = LaunchDequantDotDecodeS4x(dp, p, stream);
      if (rc >= 0) return rc;
    }
    // small s8 matrices with per-channel scales under an f32-typed multiply: one launch
    if (shape_ok && plain && !s4 && mode == kFactored && per_channel && !weights_shared && !ragged) {
      const int rc = LaunchDequantDotDecodeS8x(dp, p, stream);
      if (rc >= 0) return rc;
    }
    if (shape_ok) {
      dp.strips = (int)((p.N + 16 * nv - 1) / (16 * nv));
      // Up to 16 tokens, when the strips alone give (nearly) a workgroup per CU, the workgroup is
      // the whole CU: 16 waves split K instead of two 8-wave workgroups, and no partial sums
      // leave it (measured 6-7 % faster than the best 8-wave split on C2 up to 8 tokens).
      const bool has_w16 = mt == 1 && nv == 8 && ((s4 && mode == kRounded) || (!s4 && mode == kFactored));
      int waves = 8;
      if (has_w16 && dp.strips * p.batch >= 192 && p.K >= 2048 && !GetOption("dequant_dot_slices") && !ragged) waves = 16;
      if (int wv = GetOption("dequant_dot_waves")) waves = wv == 4 ? 4 : (wv == 16 && has_w16) ? 16 : 8;
      int slices = waves == 16 && !GetOption("dequant_dot_slices")
                       ? 1 : DecodeSlices(p.batch, p.M, p.K, p.N, dp.strips, row_bytes, waves);
      if (slices > 1 && (!p.workspace ||
                         p.workspace_bytes < DequantDotWorkspaceBytes(p.batch, p.M, p.N, slices)))
        slices = 1;
      if (ragged) slices = 1;  // every group is one workgroup per strip: its rows are only known on the device
      dp.slices = slices;
      dp.rows_per_slice = RowsPerSlice(dp.K, slices, waves);
      ClassRows(dp.rows_per_slice, waves, dp.class_rows);
      if (waves == 16) {  // one 16-token tile, 8 channels per lane: the whole CU as one workgroup
        if (s4 && mode == kRounded)
          return launch_decode<4, 4, 1, 16, kRounded>(dp, (int)p.batch, stream, "dequant_dot_decode_s4_v4_m16_w16_rounded");
        if (!s4 && mode == kFactored)
          return launch_decode<8, 8, 1, 16, kFactored>(dp, (int)p.batch, stream, "dequant_dot_decode_s8_v8_m16_w16_factored");
      }
#define XLA_AMD_DECODE(WB, V, MT_, MODE_, NAME)                                       \
  if ((s4 ? 4 : 8) == WB && vec == V && mt == MT_ && mode == MODE_)                   \
    return waves == 4 ? launch_decode<WB, V, MT_, 4, MODE_>(dp, (int)p.batch, stream, NAME) \
                      : launch_decode<WB, V, MT_, 8, MODE_>(dp, (int)p.batch, stream, NAME);
      XLA_AMD_DECODE(4, 16, 1, kRounded, "dequant_dot_decode_s4_v16_m16_rounded")
      XLA_AMD_DECODE(4, 8, 1, kRounded, "dequant_dot_decode_s4_v8_m16_rounded")
      XLA_AMD_DECODE(4, 4, 1, kRounded, "dequant_dot_decode_s4_v4_m16_rounded")
      XLA_AMD_DECODE(4, 8, 2, kRounded, "dequant_dot_decode_s4_v8_m32_rounded")
      XLA_AMD_DECODE(4, 4, 2, kRounded, "dequant_dot_decode_s4_v4_m32_rounded")
      XLA_AMD_DECODE(4, 4, 3, kRounded, "dequant_dot_decode_s4_v4_m48_rounded")
      XLA_AMD_DECODE(4, 4, 4, kRounded, "dequant_dot_decode_s4_v4_m64_rounded")
      XLA_AMD_DECODE(4, 8, 1, kFactored, "dequant_dot_decode_s4_v8_m16_factored")
      XLA_AMD_DECODE(4, 4, 1, kFactored, "dequant_dot_decode_s4_v4_m16_factored")
      XLA_AMD_DECODE(4, 4, 2, kFactored, "dequant_dot_decode_s4_v4_m32_factored")
      XLA_AMD_DECODE(4, 4, 3, kFactored, "dequant_dot_decode_s4_v4_m48_factored")
      XLA_AMD_DECODE(4, 4, 4, kFactored, "dequant_dot_decode_s4_v4_m64_factored")
      XLA_AMD_DECODE(4, 4, 1, kGroupFactored, "dequant_dot_decode_s4_v4_m16_group_factored")
      XLA_AMD_DECODE(4, 4, 2, kGroupFactored, "dequant_dot_decode_s4_v4_m32_group_factored")
      XLA_AMD_DECODE(8, 8, 1, kGroupFactored, "dequant_dot_decode_s8_v8_m16_group_factored")
      XLA_AMD_DECODE(8, 8, 2, kGroupFactored, "dequant_dot_decode_s8_v8_m32_group_factored")
      XLA_AMD_DECODE(8, 4, 3, kGroupFactored, "dequant_dot_decode_s8_v4_m48_group_factored")
      XLA_AMD_DECODE(8, 4, 4, kGroupFactored, "dequant_dot_decode_s8_v4_m64_group_factored")
      XLA_AMD_DECODE(8, 16, 1, kRounded, "dequant_dot_decode_s8_v16_m16_rounded")
      XLA_AMD_DECODE(8, 8, 1, kRounded, "dequant_dot_decode_s8_v8_m16_rounded")
      XLA_AMD_DECODE(8, 8, 2, kRounded, "dequant_dot_decode_s8_v8_m32_rounded")
      XLA_AMD_DECODE(8, 8, 3, kRounded, "dequant_dot_decode_s8_v8_m48_rounded")
      XLA_AMD_DECODE(8, 8, 4, kRounded, "dequant_dot_decode_s8_v8_m64_rounded")
      XLA_AMD_DECODE(8, 4, 3, kRounded, "dequant_dot_decode_s8_v4_m48_rounded")
      XLA_AMD_DECODE(8, 4, 4, kRounded, "dequant_dot_decode_s8_v4_m64_rounded")
      XLA_AMD_DECODE(8, 16, 1, kFactored, "dequant_dot_decode_s8_v16_m16_factored")
      XLA_AMD_DECODE(8, 8, 1, kFactored, "dequant_dot_decode_s8_v8_m16_factored")
      XLA_AMD_DECODE(8, 8, 2, kFactored, "dequant_dot_decode_s8_v8_m32_factored")
      XLA_AMD_DECODE(8, 8, 3, kFactored, "dequant_dot_decode_s8_v8_m48_factored")
      XLA_AMD_DECODE(8, 8, 4, kFactored, "dequant_dot_decode_s8_v8_m64_factored")
      XLA_AMD_DECODE(8, 4, 3, kFactored, "dequant_dot_decode_s8_v4_m48_factored")
      XLA_AMD_DECODE(8, 4, 4, kFactored, "dequant_dot_decode_s8_v4_m64_factored")
#undef XLA_AMD_DECODE
      dp.strips = 1; dp.slices = 1;
    }
  }
  if (weights_shared)
    return Fail(XLA_FFI_Error_Code_INTERNAL, "dequant_dot: a token chunk did not fit the decode kernel");
  if (force == 2 || force == 3)
    return Fail(XLA_FFI_Error_Code_FAILED_PRECONDITION,
                "dequant_dot: the requested kernel does not cover this shape");
  // fallback: any shape
  {
    dp.slices = 1;
    dim3 grid((unsigned)(((size_t)p.M * p.N + 255) / 256), (unsigned)(ragged ? 1 : p.batch));
    hipLaunchKernelGGL(dequant_dot_generic_kernel, grid, dim3(256), 0, stream, dp, s4 ? 4 : 8, mode);
    SetLastKernel("dequant_dot_generic");
    return CheckLaunch("dequant_dot_generic");
  }
}

int LaunchDequantDot(const XlaAmdDequantDot& p, hipStream_t stream) { return LaunchDequantDotImpl(p, stream, false); }

// ---- the same launch for callers that cannot allocate: the split-K partial sums go into a
// fixed array in device memory that comes with the code object instead of a workspace argument.
// Every GPU the library runs on holds its own copy of the array until the process ends.
constexpr size_t kStaticScratchBytes = 8u << 20;
constexpr int kMaxDevices = 64;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

// Device address of `scratch` on the current device.  The array's name is only a host-side handle;
// the address is looked up once per device (with that device current) and kept.
static int StaticScratchPointer(void** out) {
  static std::mutex mu;
  static void* ptrs[kMaxDevices] = {};
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess)
    return Fail(XLA_FFI_Error_Code_INTERNAL, "dequant_dot_static_scratch: hipGetDevice: %s", hipGetErrorString(e));
  if (dev < 0 || dev >= kMaxDevices)
    return Fail(XLA_FFI_Error_Code_INTERNAL, "dequant_dot_static_scratch: device ordinal %d out of range", dev);
  std::lock_guard<std::mutex> lock(mu);
  if (!ptrs[dev]) {
    void* ptr = nullptr;
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !ptr)
      return Fail(XLA_FFI_Error_Code_INTERNAL, "dequant_dot_static_scratch: hipGetSymbolAddress: %s",
                  hipGetErrorString(e));
    ptrs[dev] = ptr;
  }
  *out = ptrs[dev];
  return 0;
}

int LaunchDequantDotStaticScratch(const XlaAmdDequantDot& p, hipStream_t stream) {
  const bool four_bit = p.weight_dtype == XLA_FFI_DataType_S4 || p.weight_dtype == XLA_FFI_DataType_U4;
  // exactly what the public sizers report: the decode kernels' partial sums, or the split last round
  // of the tiled kernel when more than 64 tokens go there (it adds the halves of a tile in a fixed
  // order only when the whole of that scratch is there, so a shape needing more is refused as well)
  size_t need = 0;
  if (p.batch > 0 && p.M > 0 && p.K > 0 && p.N > 0) {
    if (p.rhs_contracting_dim == 1) {
      need = DequantDotNkWorkspaceBytes(p.batch, p.M, p.K, p.N, four_bit);
    } else {
      need = DequantDotDecodeWorkspaceBytes(p.batch, p.M, p.K, p.N, four_bit);
      const size_t tail = TiledTailWorkspaceBytes(p.batch, p.M, p.K, p.N);
      if (tail > need) need = tail;
    }
  }
  if (need > kStaticScratchBytes)
    return Fail(XLA_FFI_Error_Code_RESOURCE_EXHAUSTED,
                "dequant_dot_static_scratch: this shape splits K through %zu bytes of partial sums, the static "
                "scratch holds %zu; use xla_amd_launch_dequant_dot with a workspace",
                need, kStaticScratchBytes);
  void* ptr = nullptr;
  if (int rc = StaticScratchPointer(&ptr)) return rc;
  XlaAmdDequantDot q = p;
  q.workspace = ptr;
  q.workspace_bytes = kStaticScratchBytes;
  return LaunchDequantDotImpl(q, stream, false);
}

}  // namespace xla_amd
