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
// Lane (kb, q, i) = (lane >> 4, (lane >> 2) & 3, lane & 3) loads rows i and i + 4 of an 8-row
// block, 16 bytes (32 channels) of each.  SIDE scale groups are walked side by side: the four
// kb sit in SIDE different groups, 4 / SIDE consecutive 8-row blocks in each.  SIDE = 4 rebuilds
// the scale operands once per group / 8 steps, but spreads a step's activations over four cache
// lines per token (fine for a few tokens); SIDE = 1 reads 64 contiguous bytes per token and step.
//
// Bound: HBM.  Algorithmic bytes: K*N/2 (weights) + scales, bias, lhs and out once each.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "decode_common.h"
#include "device_numerics.h"
#include "launch.h"

namespace xla_amd {
namespace {

typedef _Float16 halfx4 __attribute__((ext_vector_type(4)));
typedef uint16_t ushortx2 __attribute__((ext_vector_type(2)));
typedef __attribute__((address_space(3))) void* lds_ptr_t;

// MT: 16-token tiles.  WAVES: waves per workgroup (they split the rows).  SIDE: scale groups side
// by side (1, 2 or 4).  DEPTH: steps whose loads are in flight or in use (>= 2).
template <int MT, int WAVES, int SIDE, int DEPTH>
__global__ __launch_bounds__(WAVES * 64) void dequant_dot_decode_s4x_kernel(DecodeParams p) {
  constexpr int R = 32 * MT;      // accumulator registers per lane: 32 channels x MT token tiles
  constexpr int KBG = 4 / SIDE;   // 8-row blocks of one group in a step
  constexpr int kChunk = (WAVES <= 8) ? 32 : 16;
  constexpr float kUnscale = 0x1p-12f;
  // Weights and activations travel global -> LDS without passing registers: per wave DEPTH slots of
  // one step's data, [32 rows][64 bytes] of weights and MT tiles of [16 tokens][64 bytes] of
  // activations.  The same memory later carries the waves' partial tiles to be added.
  constexpr int kSlot = 2048 + MT * 1024;
  constexpr int kRingBytes = WAVES * DEPTH * kSlot, kSumBytes = WAVES * kChunk * 64 * 4;
  __shared__ __attribute__((aligned(16))) uint8_t smem[kRingBytes > kSumBytes ? kRingBytes : kSumBytes];
  float* const lds = (float*)smem;
  __shared__ uint32_t lds_bad[4];

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int li = lane & 15, kb = lane >> 4, q = (lane >> 2) & 3, i = lane & 3;
  if (threadIdx.x < 4) lds_bad[threadIdx.x] = 0;
  int bid = blockIdx.x;
  {
    const int total = gridDim.x;
    if (total % 8 == 0) bid = (bid % 8) * (total / 8) + bid / 8;
  }
  const int slice = bid % p.slices;
  const int strip = bid / p.slices;
  const int batch = blockIdx.y;
  const int group = p.group;
  const int groups = p.K / group;

  const uint32_t pitch = (uint32_t)p.N >> 1;
  const __amdgpu_buffer_rsrc_t rw =
      make_rsrc(p.w + (p.weights_shared ? (size_t)0 : (size_t)batch * p.K * pitch), (uint32_t)p.K * pitch);
  // one descriptor over this batch's activations: tokens >= M lie past its end and read as zeros
  const __amdgpu_buffer_rsrc_t ra = make_rsrc(p.lhs + (size_t)batch * p.M * p.K, (uint32_t)p.M * p.K * 2u);
  const __amdgpu_buffer_rsrc_t rs = make_rsrc(
      (const char*)p.scales + (size_t)(p.scale_batched ? batch : 0) * groups * p.N * 2, (uint32_t)groups * p.N * 2u);

  constexpr uint32_t kNowhere = 0x80000000u;
  const int n_chunk = strip * 128 + 32 * q;  // the lane's 32 channels (N % 32 == 0: all inside or none)
  const bool lane_live = n_chunk < p.N;
  const int side = kb / KBG;                                   // which of the SIDE groups
  const int lane_row = side * group + (kb % KBG) * 8;          // first row of the lane's block in a step
  // Loading side: lane l fetches 16 bytes of row (l >> 2) of a 16-row half step, chunk l & 3, so four
  // neighbouring lanes read 64 contiguous bytes; row R = 8 * kb' + r of a step is row r of block kb'.
  // The data of lane l lands at slot + 16 * l: the slot is a row-major [32 rows][64 bytes] tile.
  uint32_t voff_w[2];
#pragma unroll
  for (int half = 0; half < 2; ++half) {
    const int Rr = 16 * half + (lane >> 2), kbl = Rr >> 3;
    const int row = (kbl / KBG) * group + (kbl % KBG) * 8 + (Rr & 7);
    const int nl = strip * 128 + 32 * (lane & 3);
    voff_w[half] = nl < p.N ? (uint32_t)row * pitch + (uint32_t)(nl >> 1) : kNowhere;
  }
  uint8_t* const my_ring = smem + wave * (DEPTH * kSlot);
  // Reading side: rows 8 * kb + i and 8 * kb + i + 4, chunk q
  const uint32_t rd_off = (uint32_t)(64 * (8 * kb + i) + 16 * q);
  // activations, loading side: lane l fetches 16 bytes (8 rows) of token l >> 2 for the block kb' = l & 3
  // and deposits them at 16 * l; reading side: token li, block kb
  const uint32_t voff_a =
      ((uint32_t)(lane >> 2) * p.K + (uint32_t)(((lane & 3) / KBG) * group + ((lane & 3) % KBG) * 8)) * 2u;
  const uint32_t rd_off_a = (uint32_t)(64 * li + 16 * kb);
  // as column j = i of B and D the lane stands for channels n_chunk + 8d + sm + h, sm = (0,4,2,6)[i];
  // one dword of a scales row holds the pair h = 0, 1
  const int sm = (i & 1) * 4 + (i >> 1) * 2;
  const uint32_t voff_s = lane_live ? ((uint32_t)side * p.N + (uint32_t)(n_chunk + sm)) * 2u : kNowhere;
  // byte selectors that put a 16-bit scale where s_j sits in column j = i of B (0x0c selects zero):
  // sel[h][r]: register r of the column, taking the low (h = 0) or high (h = 1) half of the source
  const uint32_t pos = (i & 1) ? 0x01000c0cu : 0x0c0c0100u;   // value in the high / low half
  const uint32_t sel00 = i < 2 ? pos : 0x0c0c0c0cu, sel01 = i < 2 ? 0x0c0c0c0cu : pos;
  const uint32_t sel10 = sel00 == 0x0c0c0c0cu ? sel00 : sel00 + ((i & 1) ? 0x02020000u : 0x00000202u);
  const uint32_t sel11 = sel01 == 0x0c0c0c0cu ? sel01 : sel01 + ((i & 1) ? 0x02020000u : 0x00000202u);

  floatx4 acc[4][2][MT];
#pragma unroll
  for (int d = 0; d < 4; ++d)
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) acc[d][h][mt] = floatx4{0.f, 0.f, 0.f, 0.f};

  // this wave's units (SIDE groups of rows each)
  const int macro = SIDE * group;
  const int spg = group / (8 * KBG);  // steps per unit, a multiple of DEPTH
  const int units = p.rows_per_slice / macro;
  const int cls = wave >> 2;
  int first = (wave & 3) * p.units_per_simd;
#pragma unroll
  for (int c = 0; c < (WAVES + 3) / 4; ++c)
    if (c < cls) first += p.class_units[c];
  int cnt = min(first + p.class_units[cls], units) - first;
  const int k_begin = slice * p.rows_per_slice + first * macro;
  if (k_begin >= p.K) cnt = 0;

  uint32_t sraw[4];
  halfx4 Bm[4][2];
  floatx4 Cm[4][2];
  uint32_t bad = 0;

  auto load_scales = [&](int km) {  // groups km / group + side of the lane's four channel pairs
    const uint32_t vs = voff_s + (uint32_t)(km / group) * (uint32_t)p.N * 2u;
#pragma unroll
    for (int d = 0; d < 4; ++d) sraw[d] = __builtin_amdgcn_raw_buffer_load_b32(rs, vs + 16u * d, 0, 0);
  };
  auto load_step = [&](int buf, int row) {  // row: first row of the step in the first of the SIDE groups
    uint8_t* const slot = my_ring + buf * kSlot;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, (lds_ptr_t)(uintptr_t)(slot + 2048 + mt * 1024), 16,
                                               voff_a + (uint32_t)(row + 16 * mt * p.K) * 2u, 0, 0, 0);
    const uint32_t rp = (uint32_t)row * pitch;
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rw, (lds_ptr_t)(uintptr_t)slot, 16, voff_w[0] + rp, 0, 0, 0);
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rw, (lds_ptr_t)(uintptr_t)(slot + 1024), 16, voff_w[1] + rp, 0, 0, 0);
  };
  // B and C of the eight channels the lane stands for, from sraw
  auto prepare = [&]() {
    const halfx4 off0 = {(_Float16)-1032.0f, (_Float16)-1032.0f, (_Float16)-1032.0f, (_Float16)-1032.0f};
    const halfx4 off1 = {(_Float16)-1152.0f, (_Float16)-1152.0f, (_Float16)-1152.0f, (_Float16)-1152.0f};
    // all eight exponents in [105, 129] (2^-22 <= |s| < 8)?  Both halves of a dword at once, in
    // unsigned 16-bit lanes: |bits| - (105 << 7) wraps below the window and exceeds 25 << 7 above it
    ushortx2 worst = {0, 0};
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      const ushortx2 ax = __builtin_bit_cast(ushortx2, sraw[d] & 0x7fff7fffu);
      worst = __builtin_elementwise_max(worst, (ushortx2)(ax - (ushortx2){105u << 7, 105u << 7}));
    }
    const bool fast = __builtin_amdgcn_ballot_w64(max(worst[0], worst[1]) >= (25u << 7)) == 0;  // wave-uniform
    if (fast) {
#pragma unroll
      for (int d = 0; d < 4; ++d) {
        // bf16 (8 exponent, 7 mantissa bits) -> f16 (5, 10) times 2^12 (low half) | 2^8 (high half):
        // shift the fields up by three and re-bias the exponent by 100 | 104, in 16-bit lanes (the six
        // exponent bits that survive the shift are enough inside the window)
        const uint32_t x = sraw[d];
        const ushortx2 ax = __builtin_bit_cast(ushortx2, x & 0x7fff7fffu);
        const ushortx2 t = (ushortx2)((ushortx2)(ax << (ushortx2){3, 3}) - (ushortx2){(uint16_t)(100u << 10), (uint16_t)(104u << 10)});
        const uint32_t pair = __builtin_bit_cast(uint32_t, t) | (x & 0x80008000u);
        Bm[d][0] = __builtin_bit_cast(halfx4, uintx2{__builtin_amdgcn_perm(pair, pair, sel00), __builtin_amdgcn_perm(pair, pair, sel01)});
        Bm[d][1] = __builtin_bit_cast(halfx4, uintx2{__builtin_amdgcn_perm(pair, pair, sel10), __builtin_amdgcn_perm(pair, pair, sel11)});
      }
    } else {
      asm volatile("");
#pragma unroll
      for (int d = 0; d < 4; ++d)
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          const float s = h ? bf16hi_to_f32(sraw[d]) : bf16lo_to_f32(sraw[d]);
          const float a = __builtin_fabsf(s);
          const bool ok = (a >= 0x1p-22f && a < 8.0f) || a == 0.0f;
          if (!ok) bad |= 1u << (2 * d + h);
          const float sv = ok ? s * (h ? 256.0f : 4096.0f) : 0.0f;
          const uint32_t pair = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(sv, sv));
          Bm[d][h] = __builtin_bit_cast(halfx4, uintx2{__builtin_amdgcn_perm(pair, pair, sel00), __builtin_amdgcn_perm(pair, pair, sel01)});
        }
    }
#pragma unroll
    for (int d = 0; d < 4; ++d)
#pragma unroll
      for (int h = 0; h < 2; ++h)
        Cm[d][h] = __builtin_amdgcn_mfma_f32_4x4x4f16(h ? off1 : off0, Bm[d][h], floatx4{0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
  };
  auto compute = [&](int buf, int row) {
    // the step's data has landed once at most the loads of the DEPTH - 1 later steps are outstanding
    // (loads complete in order; the scale loads in between only make this wait longer)
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"((DEPTH - 1) * (MT + 2)) : "memory");
    const uint8_t* const slot = my_ring + buf * kSlot;
    uintx4 av[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) av[mt] = *(const uintx4*)(slot + 2048 + mt * 1024 + rd_off_a);
    uintx4 wq[2];
    wq[0] = *(const uintx4*)(slot + rd_off);
    wq[1] = *(const uintx4*)(slot + rd_off + 256);
    if (row + (SIDE - 1) * group + 8 * KBG > p.K) {  // scalar: only a step that reaches the end of K
      asm volatile("");
      const bool ok = row + lane_row < p.K;
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
        av[mt] = uintx4{ok ? av[mt][0] : 0u, ok ? av[mt][1] : 0u, ok ? av[mt][2] : 0u, ok ? av[mt][3] : 0u};
    }
    bf16x8 bop[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) bop[mt] = __builtin_bit_cast(bf16x8, av[mt]);
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      floatx4 D[2][2];
#pragma unroll
      for (int rho = 0; rho < 2; ++rho) {
        const uint32_t x = wq[rho][d];
        const uint32_t y = x >> 8;
        // nibbles (0,4), (2,6) as 1024 + u; (1,5), (3,7) as 1024 + 16u
        const uint32_t p0 = __builtin_amdgcn_bitop3_b32(x, 0x000f000fu, 0x64086408u, 0x6a);
        const uint32_t p1 = __builtin_amdgcn_bitop3_b32(x, 0x00f000f0u, 0x64806480u, 0x6a);
        const uint32_t p2 = __builtin_amdgcn_bitop3_b32(y, 0x000f000fu, 0x64086408u, 0x6a);
        const uint32_t p3 = __builtin_amdgcn_bitop3_b32(y, 0x00f000f0u, 0x64806480u, 0x6a);
        D[0][rho] = __builtin_amdgcn_mfma_f32_4x4x4f16(__builtin_bit_cast(halfx4, uintx2{p0, p2}), Bm[d][0], Cm[d][0], 0, 0, 0);
        D[1][rho] = __builtin_amdgcn_mfma_f32_4x4x4f16(__builtin_bit_cast(halfx4, uintx2{p1, p3}), Bm[d][1], Cm[d][1], 0, 0, 0);
      }
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const uintx4 a = {pack_bf16x2(D[h][0][0], D[h][0][1]), pack_bf16x2(D[h][0][2], D[h][0][3]),
                          pack_bf16x2(D[h][1][0], D[h][1][1]), pack_bf16x2(D[h][1][2], D[h][1][3])};
        const bf16x8 aop = __builtin_bit_cast(bf16x8, a);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
          acc[d][h][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(aop, bop[mt], acc[d][h][mt], 0, 0, 0);
      }
    }
  };

  if (cnt > 0) {
    // first row of step t of the unit at km; steps past the unit's last run on into the next unit
    auto step_row = [&](int km, int t) { return t < spg ? km + 8 * KBG * t : km + macro + 8 * KBG * (t - spg); };
    load_scales(k_begin);
#pragma unroll
    for (int j = 0; j < DEPTH - 1; ++j) load_step(j, step_row(k_begin, j));
    for (int u = 0; u < cnt; ++u) {
      const int km = k_begin + u * macro;
      prepare();
      load_scales(km + macro);  // past the last group the loads return zeros
      // at least one round: the scale loads just issued are then known to be DEPTH steps of
      // loads old when the next unit waits for them, and that wait leaves the steps in flight alone
      int t = 0;
      do {
#pragma unroll
        for (int j = 0; j < DEPTH; ++j) {
          load_step((j + DEPTH - 1) % DEPTH, step_row(km, t + j + DEPTH - 1));
          compute(j, km + 8 * KBG * (t + j));
        }
        t += DEPTH;
      } while (t < spg);
    }
  }
  if (bad) {  // rare: channels whose scale does not fit the f16 operand
#pragma unroll
    for (int d = 0; d < 4; ++d)
#pragma unroll
      for (int h = 0; h < 2; ++h)
        if (bad & (1u << (2 * d + h))) {
          const int ch = 32 * q + 8 * d + sm + h;
          atomicOr(&lds_bad[ch >> 5], 1u << (ch & 31));
        }
  }

  // loads for steps past the wave's last may still be on their way into the ring
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();  // every wave is done with its ring: the memory now carries the partial tiles
  // ---- add the waves' tiles through LDS.  Register r = mt * 32 + c holds channel
  // strip * 128 + 32 * (lane >> 4) + c, token 16 * mt + (lane & 15): a lane owns 32 consecutive
  // channels.  In the MFMA tiles c = 8d + e sits in acc[d][e & 1][mt][v], v = 2 * ((e >> 1) & 1) + (e >> 2).
  constexpr int RPW = kChunk / WAVES;
  constexpr int PASSES = R / kChunk;
  static_assert(R % kChunk == 0 && kChunk % WAVES == 0 && 32 % RPW == 0, "reduction split");
  float bq[PASSES * RPW], res[PASSES * RPW];
#pragma unroll
  for (int pass = 0; pass < PASSES; ++pass) {
    const int r0 = pass * kChunk + wave * RPW;
    const int n0 = strip * 128 + 32 * kb + r0 % 32;
    const bool live = p.slices == 1 && n0 < p.N;
#pragma unroll
    for (int u = 0; u < RPW; ++u)
      bq[pass * RPW + u] = live && p.bias ? load_scale(p.bias, n0 + u, p.bias_is_bf16) : 0.0f;
  }
#pragma unroll
  for (int pass = 0; pass < PASSES; ++pass) {
#pragma unroll
    for (int c = 0; c < kChunk; ++c) {
      const int r = pass * kChunk + c;
      const int mt = r / 32, ch = r % 32, d = ch / 8, e = ch % 8;
      lds[(wave * kChunk + c) * 64 + lane] = acc[d][e & 1][mt][2 * ((e >> 1) & 1) + (e >> 2)];
    }
    __syncthreads();
#pragma unroll
    for (int u = 0; u < RPW; ++u) {
      float s = 0.0f;
#pragma unroll
      for (int w2 = 0; w2 < WAVES; ++w2) s = s + lds[(w2 * kChunk + wave * RPW + u) * 64 + lane];
      res[pass * RPW + u] = s * kUnscale;
    }
    if (pass + 1 < PASSES) __syncthreads();
  }
  if (p.slices == 1) epilogue_all_dispatch<PASSES * RPW>(res, bq, p.epilogue, p.bf16_dot, p.bf16_ops);
#pragma unroll
  for (int pass = 0; pass < PASSES; ++pass) {
    const int r0 = pass * kChunk + wave * RPW;
    const int m = (r0 / 32) * 16 + li;
    const int n0 = strip * 128 + 32 * kb + r0 % 32;
    if (m >= p.M || n0 >= p.N) continue;
    if (p.slices > 1) {
      float* dst = p.workspace + (((size_t)batch * p.slices + slice) * p.M + m) * p.N + n0;
#pragma unroll
      for (int u = 0; u < RPW; ++u) dst[u] = res[pass * RPW + u];
    } else {
      uint16_t* dst = p.out + ((size_t)batch * p.M + m) * p.N + n0;
#pragma unroll
      for (int u = 0; u < RPW; ++u) dst[u] = f32_to_bf16(res[pass * RPW + u]);
    }
  }

  // ---- flagged channels: the whole wave recomputes each (token, channel) over the slice's rows with
  // ordinary arithmetic, in a fixed order, and overwrites what the loop above produced for it
  __syncthreads();
  if ((lds_bad[0] | lds_bad[1] | lds_bad[2] | lds_bad[3]) == 0) return;
  const int ks = slice * p.rows_per_slice, ke = min(ks + p.rows_per_slice, p.K);
  const uint16_t* sc16 = (const uint16_t*)p.scales + (size_t)(p.scale_batched ? batch : 0) * groups * p.N;
  const uint8_t* wb = p.w + (p.weights_shared ? (size_t)0 : (size_t)batch * p.K * pitch);
  for (int ch = wave; ch < 128; ch += WAVES) {
    const int n = strip * 128 + ch;
    if (!((lds_bad[ch >> 5] >> (ch & 31)) & 1u) || n >= p.N) continue;
    for (int m = 0; m < p.M; ++m) {
      const uint16_t* arow = p.lhs + ((size_t)batch * p.M + m) * p.K;
      float v = 0.0f;
      for (int k = ks + lane; k < ke; k += 64) {
        const uint32_t nib = (wb[(size_t)k * pitch + (n >> 1)] >> (4 * (n & 1))) & 0xfu;
        const float wv = round_bf16((float)((int)(nib ^ 8u) - 8) * bf16_to_f32(sc16[(size_t)(k / group) * p.N + n]));
        v = v + bf16_to_f32(arow[k]) * wv;
      }
#pragma unroll
      for (int sh = 32; sh >= 1; sh >>= 1) v = v + __shfl_xor(v, sh);
      if (lane != 0) continue;
      if (p.slices > 1) {
        p.workspace[(((size_t)batch * p.slices + slice) * p.M + m) * p.N + n] = v;
      } else {
        const float b = p.bias ? load_scale(p.bias, n, p.bias_is_bf16) : 0.0f;
        p.out[((size_t)batch * p.M + m) * p.N + n] = f32_to_bf16(epilogue_dispatch(v, b, p.epilogue, p.bf16_dot, p.bf16_ops));
      }
    }
  }
}

template <int MT, int WAVES, int SIDE, int DEPTH>
int launch_s4x(const DecodeParams& dp, int batch, hipStream_t stream, const char* name) {
  dim3 grid((unsigned)(dp.strips * dp.slices), (unsigned)batch);
  hipLaunchKernelGGL((dequant_dot_decode_s4x_kernel<MT, WAVES, SIDE, DEPTH>), grid, dim3(WAVES * 64), 0, stream, dp);
  int rc = CheckLaunch(name);
  if (rc) return rc;
  if (dp.slices > 1) rc = LaunchDecodeFinalize(dp, batch, stream, kRounded);
  SetLastKernel(name);
  return rc;
}

}  // namespace

int LaunchDequantDotDecodeS4x(DecodeParams dp, const XlaAmdDequantDot& p, hipStream_t stream) {
  if (p.weight_dtype != XLA_FFI_DataType_S4 || !dp.scale_is_bf16 || p.M > 64 || p.N % 32 != 0 || p.group % 32 != 0)
    return -1;
  const int mt = p.M <= 16 ? 1 : p.M <= 32 ? 2 : p.M <= 48 ? 3 : 4;
  int side = 1;  // groups side by side cost more in scattered activation reads than they save in scale set-up
  if (int v = GetOption("dequant_dot_side")) side = v;
  if (side != 1 && side != 2 && side != 4) return -1;
  while (side < 4 && p.group / (8 * (4 / side)) < 2) side *= 2;  // at least two steps per unit
  const int macro = side * (int)p.group;
  const int spg = (int)p.group / (8 * (4 / side));   // steps per unit
  int depth = 2;  // two steps in the ring measured faster than four at every token count
  if (int v = GetOption("dequant_dot_depth")) depth = v;
  while (depth > 2 && spg % depth != 0) --depth;
  if (p.K < macro || spg % depth != 0) return -1;
  const int64_t row_bytes = p.N / 2;
  if ((double)p.K * row_bytes + 1024.0 * row_bytes >= 2147483648.0 || (double)p.M * p.K * 2 >= 2147483648.0 ||
      (double)(p.K / p.group + 8) * p.N * 2 >= 2147483648.0)
    return -1;
  const int waves = 8;
  dp.strips = (int)((p.N + 127) / 128);
  // once the strips alone (nearly) fill the CUs, K-slices only add a second launch
  int slices = dp.strips * p.batch >= 192 && !GetOption("dequant_dot_slices")
                   ? 1 : DecodeSlices(p.batch, p.M, p.K, p.N, dp.strips, row_bytes, waves);
  if (slices > 1 && (!p.workspace || p.workspace_bytes < DequantDotWorkspaceBytes(p.batch, p.M, p.N, slices)))
    slices = 1;
  while (slices > 1 && p.K / slices < macro) slices /= 2;
  dp.slices = slices;
  const int per = (int)((p.K + slices - 1) / slices);
  dp.rows_per_slice = (per + macro - 1) / macro * macro;
  const int units = dp.rows_per_slice / macro;
  dp.units_per_simd = (units + 3) / 4;
  // a SIMD serves its older wave first: the older class may take the larger share
  int w0 = 7, w1 = 5;
  if (int v = GetOption("dequant_dot_skew")) { w0 = v / 10 % 10; w1 = v % 10; }
  if (w0 + w1 <= 0) { w0 = 1; w1 = 1; }
  int u0 = (dp.units_per_simd * w0 + (w0 + w1) / 2) / (w0 + w1);
  if (u0 > dp.units_per_simd) u0 = dp.units_per_simd;
  dp.class_units[0] = u0;
  dp.class_units[1] = dp.units_per_simd - u0;
  dp.class_units[2] = dp.class_units[3] = 0;
  const int b = (int)p.batch;
#define XLA_AMD_S4X(MT_, SIDE_, DEPTH_, NAME) \
  if (mt == MT_ && side == SIDE_ && depth == DEPTH_) return launch_s4x<MT_, 8, SIDE_, DEPTH_>(dp, b, stream, NAME);
#define XLA_AMD_S4X_SIDES(MT_, DEPTH_, TOKENS)                                        \
  XLA_AMD_S4X(MT_, 1, DEPTH_, "dequant_dot_decode_s4x_" TOKENS "_side1_d" #DEPTH_)   \
  XLA_AMD_S4X(MT_, 2, DEPTH_, "dequant_dot_decode_s4x_" TOKENS "_side2_d" #DEPTH_)   \
  XLA_AMD_S4X(MT_, 4, DEPTH_, "dequant_dot_decode_s4x_" TOKENS "_side4_d" #DEPTH_)
  if (mt > 2 && depth > 2) depth = 2;  // 48 and 64 tokens: the accumulators leave room for two steps
  if (spg % depth != 0) return -1;
  XLA_AMD_S4X_SIDES(1, 4, "m16")
  XLA_AMD_S4X_SIDES(1, 2, "m16")
  XLA_AMD_S4X_SIDES(2, 4, "m32")
  XLA_AMD_S4X_SIDES(2, 2, "m32")
  XLA_AMD_S4X_SIDES(3, 2, "m48")
  XLA_AMD_S4X_SIDES(4, 2, "m64")
#undef XLA_AMD_S4X_SIDES
#undef XLA_AMD_S4X
  return -1;
}

}  // namespace xla_amd
