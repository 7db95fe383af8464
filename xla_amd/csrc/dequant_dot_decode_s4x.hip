// Weight-streaming dequantize-dot for s4 weights with bf16 scales per group of rows under a
// bf16-typed multiply (every dequantised weight is one RNE rounding of the exact product w * s:
// fusion_emitter_int4_device_test.cc:93-104 pattern, FloatNormalization of
// xla/service/cpu/cpu_compiler.cc:804-817) -- the "s4x" kernels, for up to 64 tokens.
//
// On this chip a SIMD issues one VALU or MFMA instruction about every four cycles whatever the
// instruction does, so the loop is priced in instructions per weight.  Widening and scaling a
// nibble with v_fma_mix_f32 costs one instruction per weight.  Here v_mfma_f32_4x4x4_16B_f16 does it
// for four weights per lane at once.  In each block of four lanes it computes
//   D[i][j] = sum_k A[i][k] * B[k][j] + C[i][j];
// lane i supplies row i of A (four f16), lane j column j of B and of C and receives column j of D
// (four f32).  With A[i][k] = 1024 + u (nibble k of lane i in offset binary, straight from one
// v_bitop3_b32), B[k][j] = s_j where k = j and 0 elsewhere, and C[i][j] = -1032 s_j, lane j ends up
// with (u - 8) * s_j for slot j of all four lanes: the exact products w * s of ONE channel at FOUR
// rows -- scaled and transposed by one instruction, exact because every product has at most 19
// significant bits.  Two v_cvt_pk_bf16_f32 round the four to bf16, and two such quads are the
// 8-row operand of v_mfma_f32_16x16x32_bf16 (16 channels x 32 rows against 16 tokens).
// Per 4096 weights: 32 v_bitop3 + 8 shifts + 16 small MFMAs + 32 v_cvt_pk + 8 MFMAs per 16 tokens,
// against 32 + 8 + 64 v_fma_mix + 32 + 8 of the v_fma_mix formulation.
//
// Scales enter B as f16, multiplied by 2^12 (2^8 for the nibbles that arrive as 1024 + 16u):
// exact for 2^-22 <= |s| < 8; the factor leaves with the final sums.  A group whose scales
// are all in that window takes a short integer conversion; otherwise the wave converts them one
// by one, takes zeros as they are, and flags channels with any other scale (huge, tiny, subnormal,
// inf, NaN), which are recomputed at the end by a plain loop: every input gets the reference's
// result.
//
// Consuming side: lane (kb, q, i) = (lane >> 4, (lane >> 2) & 3, lane & 3) takes rows 8 kb + i and
// 8 kb + i + 4 of a 32-row step, 16 bytes (32 channels) of each.  Loading side: weights and
// activations go global -> LDS by direct loads whose lanes are laid out for the memory system, not
// for the arithmetic: consecutive lanes read consecutive 16-byte pieces of one row.  With COLS = 2 a
// wave covers 256 channels, so every load instruction takes whole 128-byte lines (measured on
// MI355X for this matrix: 64-byte pieces per workgroup stream at 5.4 TB/s at best, whole lines
// at 6.8 TB/s); the rows are then split over two workgroups per strip, and the second adds the
// first one's partial sums, handed over through the workspace, before the epilogue.
//
// Bound: HBM.  Algorithmic bytes: K*N/2 (weights) + scales, bias, lhs and out once each.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

#include "decode_common.h"
#include "device_numerics.h"
#include "launch.h"

namespace xla_amd {
namespace {

typedef _Float16 halfx4 __attribute__((ext_vector_type(4)));
typedef uint16_t ushortx2 __attribute__((ext_vector_type(2)));
typedef __attribute__((address_space(3))) void* lds_ptr_t;

// MT: 16-token tiles.  WAVES: waves per workgroup (they split the rows).  COLS: 128-channel columns
// a wave covers (1 or 2).  DEPTH: steps whose loads are in flight or in use (>= 2).
// U4: the nibbles are unsigned (0..15) and every scale may come with a zero point (one u4 value per
// scale, packed like the weights; none: zero).  The zero point takes the place of the 8 that is
// subtracted from a biased s4 nibble: it goes into operand C of the scaling MFMA, per channel.
template <int MT, int WAVES, int COLS, int DEPTH, bool U4 = false>
__global__ __launch_bounds__(WAVES * 64) void dequant_dot_decode_s4x_kernel(DecodeParams p) {
  constexpr int R = 32 * MT * COLS;  // accumulator registers per lane: 32 channels x MT token tiles per column
  constexpr int kChunk = (WAVES <= 8) ? 32 : 16;
  constexpr int TN = 128 * COLS;     // channels per strip
  constexpr int WROW = 64 * COLS;    // bytes of a weight row a wave covers
  constexpr float kUnscale = 0x1p-12f;
  // Per wave DEPTH slots of one step's data, [32 rows][WROW bytes] of weights and MT tiles of
  // [16 tokens][64 bytes] of activations.  The same memory later carries the waves' partial tiles.
  constexpr int kWBytes = 32 * WROW;
  constexpr int kSlot = kWBytes + MT * 1024;
  constexpr int kRingBytes = WAVES * DEPTH * kSlot, kSumBytes = 2 * WAVES * kChunk * 64 * 4;
  __shared__ __attribute__((aligned(16))) uint8_t smem[kRingBytes > kSumBytes ? kRingBytes : kSumBytes];
  float* const lds = (float*)smem;
  __shared__ uint32_t lds_bad[4 * COLS];
  __shared__ int lds_partner;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int li = lane & 15, kb = lane >> 4, q = (lane >> 2) & 3, i = lane & 3;
  if (threadIdx.x < 4 * COLS) lds_bad[threadIdx.x] = 0;
  // Consecutive workgroup ids land on different XCDs (round robin over 8): 128-channel strips are
  // renumbered so that neighbours, which share cache lines, share an L2.  The two workgroups of a
  // 256-channel strip keep consecutive ids (they share no lines, and the one that waits must be
  // dispatched after the one it waits for).
  int bid = blockIdx.x;
  if (!p.pair) {
    const int total = gridDim.x;
    if (total % 8 == 0) bid = (bid % 8) * (total / 8) + bid / 8;
  }
  const int slice = bid % p.slices;
  const int strip = bid / p.slices;
  const int batch = blockIdx.y;
  const int group = p.group;
  const int groups = p.K / group;
  // two workgroups per strip that hand over inside the kernel: slice 0 produces, slice 1 finishes
  const bool producer = p.pair && slice == 0, finisher = p.pair && slice == 1;
  unsigned long long* const flag = p.flags + 2 * ((size_t)blockIdx.y * p.strips + strip);  // then the generation
  unsigned long long target = 0;  // what the raised flag holds in this run (thread 0 raises or polls)
  if (p.pair && threadIdx.x == 0) target = HandOverTarget(p.epoch, flag + 1);

  const uint32_t pitch = (uint32_t)p.N >> 1;
  const __amdgpu_buffer_rsrc_t rw =
      make_rsrc(p.w + (p.weights_shared ? (size_t)0 : (size_t)batch * p.K * pitch), (uint32_t)p.K * pitch);
  // one descriptor over this batch's activations: tokens >= M lie past its end and read as zeros
  const __amdgpu_buffer_rsrc_t ra = make_rsrc(p.lhs + (size_t)batch * p.M * p.K, (uint32_t)p.M * p.K * 2u);
  const __amdgpu_buffer_rsrc_t rs = make_rsrc(
      (const char*)p.scales + (size_t)(p.scale_batched ? batch : 0) * groups * p.N * 2, (uint32_t)groups * p.N * 2u);
  // zero points [groups, N / 2]; without them the descriptor is empty and every load returns zero
  const bool has_zp = U4 && p.zero_points != nullptr;
  const __amdgpu_buffer_rsrc_t rz =
      make_rsrc(has_zp ? p.zero_points + (size_t)(p.scale_batched ? batch : 0) * groups * pitch : p.w,
                has_zp ? (uint32_t)groups * pitch : 0u);

  constexpr uint32_t kNowhere = 0x80000000u;
  // Loading side: LPR lanes cover one row (16 bytes each), so a load instruction takes 64 / LPR whole
  // rows of WROW contiguous bytes; lane l deposits at slot + 16 * l: the slot is a row-major
  // [32 rows][WROW bytes] tile.  32-channel pieces beyond N (N % 32 == 0) read as zeros.
  constexpr int LPR = 4 * COLS, RPI = 64 / LPR, NLD = 32 / RPI;
  // LDS serves a 16-byte read 16 lanes at a time, and those 16 pieces must fall into 16 different
  // 16-byte bank groups (address / 16 mod 16).  The loads deposit lane l's piece at 16 * l whatever it
  // fetched, so the layout is swizzled by choosing WHICH piece of its row (weights) or token
  // (activations) a lane fetches -- the lanes of a row still cover the same contiguous bytes.
  // Weights, two columns: rows i and i + 2 of a lane group would meet in the same bank groups (rows
  // are 128 bytes apart); rows with bit 1 set keep their two 64-byte halves exchanged.
  const int wpiece = COLS == 2 ? (lane % LPR) ^ ((((lane / LPR) >> 1) & 1) << 2) : lane % LPR;
  const uint32_t voff_w = strip * TN + 32 * wpiece < p.N
                              ? (uint32_t)(lane / LPR) * pitch + (uint32_t)((strip * TN + 32 * wpiece) >> 1)
                              : kNowhere;
  uint8_t* const my_ring = smem + wave * (DEPTH * kSlot);
  // Consuming side: rows 8 * kb + i and 8 * kb + i + 4, column c, piece q
  uint32_t rd_off[COLS];
#pragma unroll
  for (int c = 0; c < COLS; ++c)
    rd_off[c] = (uint32_t)(WROW * (8 * kb + i) + 16 * q + 64 * (COLS == 2 ? c ^ ((i >> 1) & 1) : c));
  // activations, loading side: lane l fetches 16 bytes (8 rows) of token l >> 2 and deposits them at
  // 16 * l; consuming side: token li, block kb.  Tokens are 64 bytes apart, so tokens t, t + 4, t + 8,
  // t + 12 would meet: token t keeps its four blocks in the order block ^ ((t >> 2) & 3).
  const uint32_t voff_a = ((uint32_t)(lane >> 2) * p.K + (uint32_t)(((lane & 3) ^ ((lane >> 4) & 3)) * 8)) * 2u;
  const uint32_t rd_off_a = (uint32_t)(64 * li + 16 * (kb ^ ((li >> 2) & 3)));
  // as column j = i of B and D the lane stands for channels 128c + 32q + 8d + sm + h of the strip,
  // sm = (0,4,2,6)[i]; one dword of a scales row holds the pair h = 0, 1
  const int sm = (i & 1) * 4 + (i >> 1) * 2;
  uint32_t voff_s[COLS], voff_z[COLS];
#pragma unroll
  for (int c = 0; c < COLS; ++c) {
    const int n = strip * TN + 128 * c + 32 * q;
    voff_s[c] = n < p.N ? (uint32_t)(n + sm) * 2u : kNowhere;
    voff_z[c] = n < p.N ? (uint32_t)n >> 1 : kNowhere;  // 4 bytes per d: the 8 channels of one weight dword
  }
  // byte selectors that put a 16-bit scale where s_j sits in column j = i of B (0x0c selects zero):
  // sel[h][r]: register r of the column, taking the low (h = 0) or high (h = 1) half of the source
  const uint32_t pos = (i & 1) ? 0x01000c0cu : 0x0c0c0100u;   // value in the high / low half
  const uint32_t sel00 = i < 2 ? pos : 0x0c0c0c0cu, sel01 = i < 2 ? 0x0c0c0c0cu : pos;
  const uint32_t sel10 = sel00 == 0x0c0c0c0cu ? sel00 : sel00 + ((i & 1) ? 0x02020000u : 0x00000202u);
  const uint32_t sel11 = sel01 == 0x0c0c0c0cu ? sel01 : sel01 + ((i & 1) ? 0x02020000u : 0x00000202u);

  floatx4 acc[COLS][4][2][MT];
#pragma unroll
  for (int c = 0; c < COLS; ++c)
#pragma unroll
    for (int d = 0; d < 4; ++d)
#pragma unroll
      for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) acc[c][d][h][mt] = floatx4{0.f, 0.f, 0.f, 0.f};

  // this wave's units (one scale group of rows each).  The producer of a pair takes fewer rows than
  // the finisher (rows_first against the rest), so that its sums are on their way while the finisher
  // still streams; class_units[2..3] and units_per_simd2 describe the finisher's split then.
  const int spg = group >> 5;  // steps per unit, a multiple of DEPTH
  const int slice_begin = finisher ? p.rows_first : slice * p.rows_per_slice;
  const int slice_rows = producer ? p.rows_first : p.rows_per_slice;
  const int units = slice_rows / group;
  const int cls = wave >> 2;
  const int ups = finisher ? p.units_per_simd2 : p.units_per_simd;
  const int cu0 = finisher ? p.class_units[2] : p.class_units[0];
  const int cu1 = finisher ? p.class_units[3] : p.class_units[1];
  const int first = (wave & 3) * ups + (cls ? cu0 : 0);
  int cnt = min(first + (cls ? cu1 : cu0), units) - first;
  const int k_begin = slice_begin + first * group;
  if (k_begin >= p.K) cnt = 0;

  uint32_t sraw[COLS][4];
  uint32_t zraw[COLS][4];  // U4: the zero points of the dword's 8 channels, one nibble each
  halfx4 Bm[COLS][4][2];
  floatx4 Cm[COLS][4][2];
  uint32_t bad = 0;

  auto load_scales = [&](int km) {  // group km / group of the lane's channel pairs
    const uint32_t vs = (uint32_t)(km / group) * (uint32_t)p.N * 2u;
#pragma unroll
    for (int c = 0; c < COLS; ++c)
#pragma unroll
      for (int d = 0; d < 4; ++d) sraw[c][d] = __builtin_amdgcn_raw_buffer_load_b32(rs, voff_s[c] + vs + 16u * d, 0, 0);
    if constexpr (U4) {
      const uint32_t vz = (uint32_t)(km / group) * pitch;  // a row of zero points is as long as a row of weights
#pragma unroll
      for (int c = 0; c < COLS; ++c)
#pragma unroll
        for (int d = 0; d < 4; ++d) zraw[c][d] = __builtin_amdgcn_raw_buffer_load_b32(rz, voff_z[c] + vz + 4u * d, 0, 0);
    }
  };
  auto load_step = [&](int buf, int row) {  // row: first row of the step
    uint8_t* const slot = my_ring + buf * kSlot;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, (lds_ptr_t)(uintptr_t)(slot + kWBytes + mt * 1024), 16,
                                               voff_a + (uint32_t)(row + 16 * mt * p.K) * 2u, 0, 0, 0);
    // (the offsets are spelled out rather than kept in an array indexed by j: with such an argument
    // to this builtin inside a lambda the compiler's host pass drops the kernel's launch stub)
    const uint32_t rp = (uint32_t)row * pitch;
#pragma unroll
    for (int j = 0; j < NLD; ++j)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rw, (lds_ptr_t)(uintptr_t)(slot + 1024 * j), 16,
                                               voff_w + rp + (uint32_t)(RPI * j) * pitch, 0, 0, 0);
  };
  // B and C of the channels the lane stands for, from sraw
  auto prepare = [&]() {
    const halfx4 off0 = {(_Float16)-1032.0f, (_Float16)-1032.0f, (_Float16)-1032.0f, (_Float16)-1032.0f};
    const halfx4 off1 = {(_Float16)-1152.0f, (_Float16)-1152.0f, (_Float16)-1152.0f, (_Float16)-1152.0f};
    // all exponents in [105, 129] (2^-22 <= |s| < 8)?  Both halves of a dword at once, in
    // unsigned 16-bit lanes: |bits| - (105 << 7) wraps below the window and exceeds 25 << 7 above it
    ushortx2 worst = {0, 0};
#pragma unroll
    for (int c = 0; c < COLS; ++c)
#pragma unroll
      for (int d = 0; d < 4; ++d) {
        const ushortx2 ax = __builtin_bit_cast(ushortx2, sraw[c][d] & 0x7fff7fffu);
        worst = __builtin_elementwise_max(worst, (ushortx2)(ax - (ushortx2){105u << 7, 105u << 7}));
      }
    const bool fast = __builtin_amdgcn_ballot_w64(max(worst[0], worst[1]) >= (25u << 7)) == 0;  // wave-uniform
    if (fast) {
#pragma unroll
      for (int c = 0; c < COLS; ++c)
#pragma unroll
        for (int d = 0; d < 4; ++d) {
          // bf16 (8 exponent, 7 mantissa bits) -> f16 (5, 10) times 2^12 (low half) | 2^8 (high half):
          // shift the fields up by three and re-bias the exponent by 100 | 104, in 16-bit lanes (the six
          // exponent bits that survive the shift are enough inside the window)
          const uint32_t x = sraw[c][d];
          const ushortx2 ax = __builtin_bit_cast(ushortx2, x & 0x7fff7fffu);
          const ushortx2 t = (ushortx2)((ushortx2)(ax << (ushortx2){3, 3}) - (ushortx2){(uint16_t)(100u << 10), (uint16_t)(104u << 10)});
          const uint32_t pair = __builtin_bit_cast(uint32_t, t) | (x & 0x80008000u);
          Bm[c][d][0] = __builtin_bit_cast(halfx4, uintx2{__builtin_amdgcn_perm(pair, pair, sel00), __builtin_amdgcn_perm(pair, pair, sel01)});
          Bm[c][d][1] = __builtin_bit_cast(halfx4, uintx2{__builtin_amdgcn_perm(pair, pair, sel10), __builtin_amdgcn_perm(pair, pair, sel11)});
        }
    } else {
      asm volatile("");
#pragma unroll
      for (int c = 0; c < COLS; ++c)
#pragma unroll
        for (int d = 0; d < 4; ++d)
#pragma unroll
          for (int h = 0; h < 2; ++h) {
            const float s = h ? bf16hi_to_f32(sraw[c][d]) : bf16lo_to_f32(sraw[c][d]);
            const float a = __builtin_fabsf(s);
            const bool ok = (a >= 0x1p-22f && a < 8.0f) || a == 0.0f;
            if (!ok) bad |= 1u << (8 * c + 2 * d + h);
            const float sv = ok ? s * (h ? 256.0f : 4096.0f) : 0.0f;
            const uint32_t pair = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(sv, sv));
            Bm[c][d][h] = __builtin_bit_cast(halfx4, uintx2{__builtin_amdgcn_perm(pair, pair, sel00), __builtin_amdgcn_perm(pair, pair, sel01)});
          }
    }
#pragma unroll
    for (int c = 0; c < COLS; ++c)
#pragma unroll
      for (int d = 0; d < 4; ++d)
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          halfx4 off = h ? off1 : off0;
          if constexpr (U4) {
            // -(1024 + z) | -(1024 + 16 z) of the four channels the block's columns stand for, in the
            // order the nibbles of a weight dword are unpacked in: f16 bits 0xe400 | z, 0xe400 | z << 4
            const uint32_t z = zraw[c][d], m = h ? 0x00f000f0u : 0x000f000fu;
            off = __builtin_bit_cast(halfx4, uintx2{(uint32_t)__builtin_amdgcn_bitop3_b32(z, m, 0xe400e400u, 0x6a),
                                                    (uint32_t)__builtin_amdgcn_bitop3_b32(z >> 8, m, 0xe400e400u, 0x6a)});
          }
          Cm[c][d][h] = __builtin_amdgcn_mfma_f32_4x4x4f16(off, Bm[c][d][h], floatx4{0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
        }
  };
  // One 32-row step.  The work of consecutive operands (16 channels x 32 rows each: 2 small MFMAs,
  // 4 conversions, MT large MFMAs) is overlapped by hand: while operand o goes through the large
  // MFMAs, operand o + 1 is in the small ones and the nibbles of operand o + 2 are being unpacked,
  // so that no instruction waits for the one just before it.  A SIMD issues one VALU or matrix
  // instruction per four cycles and a matrix instruction then occupies the matrix pipe for 8 (small)
  // or 16 (large) cycles: VALU instructions placed between them ride along for free, instructions
  // that wait for a result do not.  sched_barrier pins the order; the compiler still places waits.
  auto compute = [&](int buf, int row) {
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"((DEPTH - 1) * (MT + NLD)) : "memory");
    const uint8_t* const slot = my_ring + buf * kSlot;
    uintx4 av[MT];
    uintx4 wq[COLS][2];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) av[mt] = *(const uintx4*)(slot + kWBytes + mt * 1024 + rd_off_a);
#pragma unroll
    for (int c = 0; c < COLS; ++c) {
      wq[c][0] = *(const uintx4*)(slot + rd_off[c]);
      wq[c][1] = *(const uintx4*)(slot + rd_off[c] + 4 * WROW);
    }
    if (row + 32 > p.K) {  // scalar: only a step that reaches the end of K
      asm volatile("");
      const bool ok = row + 8 * kb < p.K;
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
        av[mt] = uintx4{ok ? av[mt][0] : 0u, ok ? av[mt][1] : 0u, ok ? av[mt][2] : 0u, ok ? av[mt][3] : 0u};
    }
    bf16x8 bop[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) bop[mt] = __builtin_bit_cast(bf16x8, av[mt]);
    constexpr int NO = COLS * 8;   // operands of the step: o = (c, d, h)
    uint32_t ysh[2] = {0u, 0u};    // x >> 8 of the two rows of the current (c, d)
    halfx4 A[3][2];                // unpacked nibbles of operand o % 3, rows rho = 0, 1
    floatx4 Dq[2][2];              // scaled products of operand o % 2
    auto unpack = [&](int o, int rho) {
      const int c = o / 8, d = (o / 2) % 4, h = o % 2;
      const uint32_t x = wq[c][rho][d];
      if (h == 0) ysh[rho] = x >> 8;
      // f16 1024 + u | 1024 + 16 u; an s4 nibble is biased on the way (u = w + 8: its top bit flipped)
      const uint32_t m = h ? 0x00f000f0u : 0x000f000fu, k = U4 ? 0x64006400u : h ? 0x64806480u : 0x64086408u;
      A[o % 3][rho] = __builtin_bit_cast(halfx4, uintx2{(uint32_t)__builtin_amdgcn_bitop3_b32(x, m, k, 0x6a),
                                                        (uint32_t)__builtin_amdgcn_bitop3_b32(ysh[rho], m, k, 0x6a)});
    };
    auto small = [&](int o, int rho) {
      const int c = o / 8, d = (o / 2) % 4, h = o % 2;
      Dq[o % 2][rho] = __builtin_amdgcn_mfma_f32_4x4x4f16(A[o % 3][rho], Bm[c][d][h], Cm[c][d][h], 0, 0, 0);
    };
    uintx4 aw;
    auto convert = [&](int o, int rho) {
      aw[2 * rho] = pack_bf16x2(Dq[o % 2][rho][0], Dq[o % 2][rho][1]);
      aw[2 * rho + 1] = pack_bf16x2(Dq[o % 2][rho][2], Dq[o % 2][rho][3]);
    };
    auto large = [&](int o, int mt) {
      const int c = o / 8, d = (o / 2) % 4, h = o % 2;
      acc[c][d][h][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, aw), bop[mt], acc[c][d][h][mt], 0, 0, 0);
    };
    // fill: operands 0 and 1 unpacked, operand 0 through the small MFMAs
    unpack(0, 0); unpack(0, 1);
    __builtin_amdgcn_sched_barrier(0);
    small(0, 0); unpack(1, 0);
    __builtin_amdgcn_sched_barrier(0);
    small(0, 1); unpack(1, 1);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int o = 0; o < NO; ++o) {
      if (o + 1 < NO) small(o + 1, 0);
      convert(o, 0);
      __builtin_amdgcn_sched_barrier(0);
      if (o + 1 < NO) small(o + 1, 1);
      convert(o, 1);
      __builtin_amdgcn_sched_barrier(0);
      if (o + 2 < NO) unpack(o + 2, 0);
      __builtin_amdgcn_sched_barrier(0);
      large(o, 0);
      if (o + 2 < NO) unpack(o + 2, 1);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int mt = 1; mt < MT; ++mt) large(o, mt);
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  if (cnt > 0) {
    load_scales(k_begin);
#pragma unroll
    for (int j = 0; j < DEPTH - 1; ++j) load_step(j, k_begin + 32 * j);
    for (int u = 0; u < cnt; ++u) {
      const int km = k_begin + u * group;
      prepare();
      load_scales(km + group);  // past the last group the loads return zeros
      // at least one round: the scale loads just issued are then known to be DEPTH steps of
      // loads old when the next unit waits for them, and that wait leaves the steps in flight alone
      int t = 0;
      do {
#pragma unroll
        for (int j = 0; j < DEPTH; ++j) {
          load_step((j + DEPTH - 1) % DEPTH, km + 32 * (t + j + DEPTH - 1));
          compute(j, km + 32 * (t + j));
        }
        t += DEPTH;
      } while (t < spg);
    }
  }
  if (bad) {  // rare: channels whose scale does not fit the f16 operand
#pragma unroll
    for (int c = 0; c < COLS; ++c)
#pragma unroll
      for (int d = 0; d < 4; ++d)
#pragma unroll
        for (int h = 0; h < 2; ++h)
          if (bad & (1u << (8 * c + 2 * d + h))) {
            const int ch = 128 * c + 32 * q + 8 * d + sm + h;
            atomicOr(&lds_bad[ch >> 5], 1u << (ch & 31));
          }
  }
  // loads for steps past the wave's last may still be on their way into the ring
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();  // every wave is done with its ring: the memory now carries the partial tiles
  // ---- add the waves' tiles through LDS.  Register r = (c * MT + mt) * 32 + e32 holds channel
  // strip * TN + 128 * c + 32 * (lane >> 4) + e32, token 16 * mt + (lane & 15): a lane owns 32
  // consecutive channels per column.  In the MFMA tiles e32 = 8d + e sits in
  // acc[c][d][e & 1][mt][v], v = 2 * ((e >> 1) & 1) + (e >> 2).
  constexpr int RPW = kChunk / WAVES;
  constexpr int PASSES = R / kChunk;
  static_assert(R % kChunk == 0 && kChunk % WAVES == 0 && 32 % RPW == 0, "reduction split");
  const bool finishes = p.slices == 1 || finisher;  // this workgroup applies the epilogue and writes the result
  float bq[PASSES * RPW], res[PASSES * RPW];
#pragma unroll
  for (int pass = 0; pass < PASSES; ++pass) {
    const int r0 = pass * kChunk + wave * RPW;
    const int n0 = strip * TN + 128 * (r0 / (32 * MT)) + 32 * kb + r0 % 32;
    const bool live = finishes && n0 < p.N;
#pragma unroll
    for (int u = 0; u < RPW; ++u)
      bq[pass * RPW + u] = live && p.bias ? load_scale(p.bias, n0 + u, p.bias_is_bf16) : 0.0f;
  }
  // Two buffers of kChunk registers per wave: a wave deposits pass + 1 (16 bytes per lane and
  // instruction) before it collects pass, so the passes overlap and need one barrier each.  The sums
  // over the waves run in wave order.
  static_assert(RPW == 4, "a lane collects one 16-byte piece per wave and pass");
  floatx4* const lds4 = (floatx4*)smem;
  auto deposit = [&](int pass) {
#pragma unroll
    for (int q4 = 0; q4 < kChunk / 4; ++q4) {
      floatx4 v;
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int r = pass * kChunk + 4 * q4 + u;
        const int c = r / (32 * MT), mt = (r / 32) % MT, ch = r % 32, d = ch / 8, e = ch % 8;
        v[u] = acc[c][d][e & 1][mt][2 * ((e >> 1) & 1) + (e >> 2)];
      }
      lds4[(((pass & 1) * WAVES + wave) * (kChunk / 4) + q4) * 64 + lane] = v;
    }
  };
  deposit(0);
  __syncthreads();
#pragma unroll
  for (int pass = 0; pass < PASSES; ++pass) {
    if (pass + 1 < PASSES) deposit(pass + 1);
    floatx4 s = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int w2 = 0; w2 < WAVES; ++w2) {
      const floatx4 v = lds4[(((pass & 1) * WAVES + w2) * (kChunk / 4) + wave) * 64 + lane];
#pragma unroll
      for (int u = 0; u < 4; ++u) s[u] = s[u] + v[u];
    }
#pragma unroll
    for (int u = 0; u < RPW; ++u) res[pass * RPW + u] = s[u] * kUnscale;
    if (pass + 1 < PASSES) __syncthreads();
  }

  // ---- hand-over between the two workgroups of a strip.  The producer's sums and the flag go out
  // as device-scope stores, the finisher reads them with device-scope loads: no cache maintenance.
  // The producer has the lower workgroup id of the two, so it was dispatched first and never waits
  // for anything; should the flag still not show after a long bounded wait, the finisher computes
  // the whole strip by the plain loop below instead.
  // The sums travel in the threads' own order -- [pass][wave][lane][RPW floats], 64 KiB... per strip
  // R * 64 floats -- so that every wave stores and loads 64 x 16 contiguous bytes.
  static_assert(RPW == 4 || COLS == 1, "the hand-over moves 16 bytes per lane and pass");
  const __amdgpu_buffer_rsrc_t rh = make_rsrc(p.workspace + ((size_t)batch * p.strips + strip) * (R * 64), R * 64 * 4);
  constexpr int kDeviceScope = 16;  // sc1: the access is performed where every XCD sees it
  bool partner_ok = true;
  if (finisher) {
    if (threadIdx.x == 0) {
      int ok = 0;
      const int spins = p.handover_test ? kHandOverTestSpins : kHandOverSpins;
      for (int spin = 0; spin < spins; ++spin) {
        if (__hip_atomic_load(flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == target) { ok = 1; break; }
        __builtin_amdgcn_s_sleep(8);
      }
      lds_partner = ok;
    }
    __syncthreads();
    partner_ok = lds_partner != 0;
    if (partner_ok) {
      uintx4 other[PASSES];
#pragma unroll
      for (int pass = 0; pass < PASSES; ++pass)
        other[pass] = __builtin_amdgcn_raw_buffer_load_b128(rh, (uint32_t)(((pass * WAVES + wave) * 64 + lane) * 16), 0, kDeviceScope);
#pragma unroll
      for (int pass = 0; pass < PASSES; ++pass)
#pragma unroll
        for (int u = 0; u < RPW; ++u) res[pass * RPW + u] = bits_to_f32(other[pass][u]) + res[pass * RPW + u];
    }
  }
  if (finishes) epilogue_all_dispatch<PASSES * RPW>(res, bq, p.epilogue, p.bf16_dot, p.bf16_ops);
#pragma unroll
  for (int pass = 0; pass < PASSES; ++pass) {
    const int r0 = pass * kChunk + wave * RPW;
    const int m = ((r0 / 32) % MT) * 16 + li;
    const int n0 = strip * TN + 128 * (r0 / (32 * MT)) + 32 * kb + r0 % 32;
    if (m >= p.M || n0 >= p.N) continue;
    if (producer) {
      if constexpr (RPW == 4)
        __builtin_amdgcn_raw_buffer_store_b128(uintx4{f32_to_bits(res[pass * RPW]), f32_to_bits(res[pass * RPW + 1]),
                                                      f32_to_bits(res[pass * RPW + 2]), f32_to_bits(res[pass * RPW + 3])},
                                               rh, (uint32_t)(((pass * WAVES + wave) * 64 + lane) * 16), 0, kDeviceScope);
    } else if (!finishes) {
      float* dst = p.workspace + (((size_t)batch * p.slices + slice) * p.M + m) * p.N + n0;
#pragma unroll
      for (int u = 0; u < RPW; ++u) dst[u] = res[pass * RPW + u];
    } else {
      uint16_t* dst = p.out + ((size_t)batch * p.M + m) * p.N + n0;
#pragma unroll
      for (int u = 0; u < RPW; ++u) dst[u] = f32_to_bf16(res[pass * RPW + u]);
    }
  }

  // ---- flagged channels (or, after a failed hand-over, every channel): the whole wave recomputes
  // each (token, channel) over the rows with ordinary arithmetic, in a fixed order, and overwrites
  // what the loop above produced for it.  The stores above must have landed first.
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  uint32_t any_bad = partner_ok ? 0u : 1u;
#pragma unroll
  for (int c = 0; c < 4 * COLS; ++c) any_bad |= lds_bad[c];
  if (any_bad) {
    const int ks = partner_ok ? slice_begin : 0;
    const int ke = partner_ok ? min(ks + slice_rows, p.K) : p.K;
    const uint16_t* sc16 = (const uint16_t*)p.scales + (size_t)(p.scale_batched ? batch : 0) * groups * p.N;
    const uint8_t* wb = p.w + (p.weights_shared ? (size_t)0 : (size_t)batch * p.K * pitch);
    const uint8_t* zb = p.zero_points ? p.zero_points + (size_t)(p.scale_batched ? batch : 0) * groups * pitch : nullptr;
    for (int ch = wave; ch < TN; ch += WAVES) {
      const int n = strip * TN + ch;
      if ((partner_ok && !((lds_bad[ch >> 5] >> (ch & 31)) & 1u)) || n >= p.N) continue;
      for (int m = 0; m < p.M; ++m) {
        const uint16_t* arow = p.lhs + ((size_t)batch * p.M + m) * p.K;
        float v = 0.0f;
        for (int k = ks + lane; k < ke; k += 64) {
          const uint32_t nib = (wb[(size_t)k * pitch + (n >> 1)] >> (4 * (n & 1))) & 0xfu;
          int wi = (int)(nib ^ 8u) - 8;
          if constexpr (U4) {
            wi = (int)nib;
            if (p.zero_points) wi -= (int)((zb[(size_t)(k / group) * pitch + (n >> 1)] >> (4 * (n & 1))) & 0xfu);
          }
          const float wv = round_bf16((float)wi * bf16_to_f32(sc16[(size_t)(k / group) * p.N + n]));
          v = v + bf16_to_f32(arow[k]) * wv;
        }
#pragma unroll
        for (int sh = 32; sh >= 1; sh >>= 1) v = v + __shfl_xor(v, sh);
        if (lane != 0) continue;
        // where the thread that owns (m, n) keeps it in the hand-over buffer
        const int hr = ((ch >> 7) * MT + (m >> 4)) * 32 + (ch & 31);
        float* const hslot = p.workspace + ((size_t)batch * p.strips + strip) * (R * 64) +
                             (((hr / kChunk) * WAVES + (hr % kChunk) / RPW) * 64 + 16 * ((ch & 127) >> 5) + (m & 15)) * RPW +
                             (hr % kChunk) % RPW;
        if (producer) {
          __hip_atomic_store(hslot, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        } else if (!finishes) {
          p.workspace[(((size_t)batch * p.slices + slice) * p.M + m) * p.N + n] = v;
        } else {
          if (finisher && partner_ok) v = __hip_atomic_load(hslot, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) + v;
          const float b = p.bias ? load_scale(p.bias, n, p.bias_is_bf16) : 0.0f;
          p.out[((size_t)batch * p.M + m) * p.N + n] = f32_to_bf16(epilogue_dispatch(v, b, p.epilogue, p.bf16_dot, p.bf16_ops));
        }
      }
    }
  }
  if (p.pair) {
    // the producer raises the flag once all its sums have landed; the finisher, done with the slot
    // whether the flag showed or not, moves the strip on to its next generation so that the next
    // run (also a replay of this same launch from a captured graph) waits for new sums
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (threadIdx.x == 0) {
      if (finisher) HandOverNextGeneration(flag + 1, target);
      else if (!p.handover_test) __hip_atomic_store(flag, target, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  }
}

template <int MT, int WAVES, int COLS, int DEPTH, bool U4 = false>
int launch_s4x(const DecodeParams& dp, int batch, hipStream_t stream, const char* name) {
  dim3 grid((unsigned)(dp.strips * dp.slices), (unsigned)batch);
  hipLaunchKernelGGL((dequant_dot_decode_s4x_kernel<MT, WAVES, COLS, DEPTH, U4>), grid, dim3(WAVES * 64), 0, stream, dp);
  int rc = CheckLaunch(name);
  if (rc) return rc;
  if (dp.slices > 1 && !dp.pair) rc = LaunchDecodeFinalize(dp, batch, stream, kRounded);
  SetLastKernel(name);
  return rc;
}

}  // namespace

// Bytes of workspace the in-kernel hand-over between the two workgroups of a 256-channel strip
// needs: the producer's f32 sums, 16 KiB per (batch, strip), and an 8-byte flag and generation each.
size_t S4xPairWorkspaceBytes(int64_t batch, int64_t M, int64_t N) {
  (void)M;  // the producer's sums travel as whole 16-token tiles: 16 x 256 floats per strip
  return (size_t)batch * ((N + 255) / 256) * (16 * 256 * 4 + 16);  // sums, flag, generation
}

// Whole 128-byte lines per load and two workgroups per 256-channel strip: up to 16 tokens (the
// accumulators and scale operands of two columns fill the registers).  Chosen by itself when those
// workgroups fill most of the machine and every wave gets at least one group of rows; option
// "dequant_dot_pair" = 1 takes it wherever the shape allows, 2 never.
bool S4xPairShape(int64_t batch, int64_t M, int64_t K, int64_t N, int64_t group) {
  const int mode = GetOption("dequant_dot_pair");
  if (mode == 2 || M < 1 || M > 16 || N % 32 != 0 || group % 64 != 0 || K < 2 * group) return false;
  if (mode == 1) return true;
  const int64_t wgs = batch * ((N + 255) / 256) * 2;
  return K / 2 >= 8 * group && wgs >= 128 && wgs <= 1024;
}

int LaunchDequantDotDecodeS4x(DecodeParams dp, const XlaAmdDequantDot& p, hipStream_t stream) {
  const bool u4 = p.weight_dtype == XLA_FFI_DataType_U4;
  if ((p.weight_dtype != XLA_FFI_DataType_S4 && !u4) || !dp.scale_is_bf16 || p.M > 64 || p.N % 32 != 0 || p.group % 64 != 0)
    return -1;
  if (u4 && p.zero_points && ((uintptr_t)p.zero_points % 4) != 0) return -1;  // read a dword (8 channels) at a time
  const int mt = p.M <= 16 ? 1 : p.M <= 32 ? 2 : p.M <= 48 ? 3 : 4;
  const int group = (int)p.group;
  const int spg = group / 32;   // steps per unit
  int depth = 2;  // two steps in the ring measured faster than four at every token count
  if (int v = GetOption("dequant_dot_depth")) depth = v;
  if (mt > 2 && depth > 2) depth = 2;  // 48 and 64 tokens: the ring leaves room for two steps
  if ((depth != 2 && depth != 4) || p.K < group || spg % depth != 0) return -1;
  const int64_t row_bytes = p.N / 2;
  if ((double)p.K * row_bytes + 1024.0 * row_bytes >= 2147483648.0 || (double)p.M * p.K * 2 >= 2147483648.0 ||
      (double)(p.K / p.group + 8) * p.N * 2 >= 2147483648.0)
    return -1;
  const int waves = 8;
  const int b = (int)p.batch;
  // a SIMD serves its older wave first: the older class takes the larger share of the rows
  // (7:5 measured best up to 32 tokens, 5:3 from there on, where the matrix pipe is the busier one)
  int w0 = mt <= 2 ? 7 : 5, w1 = mt <= 2 ? 5 : 3;
  if (int v = GetOption("dequant_dot_skew")) { w0 = v / 10 % 10; w1 = v % 10; }
  if (w0 + w1 <= 0) { w0 = 1; w1 = 1; }
  auto split_rows = [&](int slices) {
    dp.slices = slices;
    const int per = (int)((p.K + slices - 1) / slices);
    dp.rows_per_slice = (per + group - 1) / group * group;
    const int units = dp.rows_per_slice / group;
    dp.units_per_simd = (units + 3) / 4;
    int u0 = (dp.units_per_simd * w0 + (w0 + w1) / 2) / (w0 + w1);
    if (u0 > dp.units_per_simd) u0 = dp.units_per_simd;
    dp.class_units[0] = u0;
    dp.class_units[1] = dp.units_per_simd - u0;
    dp.class_units[2] = dp.class_units[3] = 0;
  };
  dp.pair = 0;
  dp.flags = nullptr;
  dp.epoch = 0;
  dp.rows_first = 0;
  dp.units_per_simd2 = 0;
  const bool forced_slices = GetOption("dequant_dot_slices") != 0;
  if (mt == 1 && depth == 2 && !forced_slices && S4xPairShape(p.batch, p.M, p.K, p.N, p.group) && p.workspace &&
      ((uintptr_t)p.workspace % 8) == 0 && p.workspace_bytes >= S4xPairWorkspaceBytes(p.batch, p.M, p.N)) {
    dp.strips = (int)((p.N + 255) / 256);
    dp.pair = 1;
    dp.flags = (unsigned long long*)((char*)p.workspace + (size_t)p.batch * dp.strips * (16 * 256 * 4));
    dp.epoch = NextHandOverEpoch();
    // Rows are split evenly ("dequant_dot_share" sets the producer's sixteenths): giving the producer
    // less, so that its sums are in memory before the finisher asks, measured slower at every token
    // count -- the finisher's own loop is what the kernel waits for.
    int share = 8;
    if (int v = GetOption("dequant_dot_share")) share = v;
    const int groups_total = (int)((p.K + group - 1) / group);
    int g0 = (groups_total * share + 8) / 16;
    if (g0 < 1) g0 = 1;
    if (g0 > groups_total - 1) g0 = groups_total - 1;
    auto class_split = [&](int units, int* ups, int* c0, int* c1) {
      *ups = (units + 3) / 4;
      int u0 = (*ups * w0 + (w0 + w1) / 2) / (w0 + w1);
      if (u0 > *ups) u0 = *ups;
      *c0 = u0;
      *c1 = *ups - u0;
    };
    dp.slices = 2;
    dp.rows_first = g0 * group;
    dp.rows_per_slice = (groups_total - g0) * group;   // the finisher's rows (to the end of K, rounded up to a group)
    class_split(g0, &dp.units_per_simd, &dp.class_units[0], &dp.class_units[1]);
    class_split(groups_total - g0, &dp.units_per_simd2, &dp.class_units[2], &dp.class_units[3]);
    if (u4) return launch_s4x<1, 8, 2, 2, true>(dp, b, stream, "dequant_dot_decode_u4x_m16_pair");
    return launch_s4x<1, 8, 2, 2>(dp, b, stream, "dequant_dot_decode_s4x_m16_pair");
  }
  dp.strips = (int)((p.N + 127) / 128);
  // once the strips alone (nearly) fill the CUs, K-slices only add a second launch
  int slices = dp.strips * p.batch >= 192 && !forced_slices
                   ? 1 : DecodeSlices(p.batch, p.M, p.K, p.N, dp.strips, row_bytes, waves);
  if (slices > 1 && (!p.workspace || p.workspace_bytes < DequantDotWorkspaceBytes(p.batch, p.M, p.N, slices)))
    slices = 1;
  while (slices > 1 && p.K / slices < group) slices /= 2;
  split_rows(slices);
  if (u4) {
    if (depth != 2) return -1;
    if (mt == 1) return launch_s4x<1, 8, 1, 2, true>(dp, b, stream, "dequant_dot_decode_u4x_m16_d2");
    if (mt == 2) return launch_s4x<2, 8, 1, 2, true>(dp, b, stream, "dequant_dot_decode_u4x_m32_d2");
    if (mt == 3) return launch_s4x<3, 8, 1, 2, true>(dp, b, stream, "dequant_dot_decode_u4x_m48_d2");
    return launch_s4x<4, 8, 1, 2, true>(dp, b, stream, "dequant_dot_decode_u4x_m64_d2");
  }
#define XLA_AMD_S4X(MT_, DEPTH_, NAME) \
  if (mt == MT_ && depth == DEPTH_) return launch_s4x<MT_, 8, 1, DEPTH_>(dp, b, stream, NAME);
  XLA_AMD_S4X(1, 2, "dequant_dot_decode_s4x_m16_d2")
  XLA_AMD_S4X(1, 4, "dequant_dot_decode_s4x_m16_d4")
  XLA_AMD_S4X(2, 2, "dequant_dot_decode_s4x_m32_d2")
  XLA_AMD_S4X(2, 4, "dequant_dot_decode_s4x_m32_d4")
  XLA_AMD_S4X(3, 2, "dequant_dot_decode_s4x_m48_d2")
  XLA_AMD_S4X(4, 2, "dequant_dot_decode_s4x_m64_d2")
#undef XLA_AMD_S4X
  return -1;
}

}  // namespace xla_amd
