// Dequantize-dot over weights stored [N,K] -- the contracting dimension minor, as
// `dot(lhs, convert(s4[N,K])), rhs_contracting_dims={1}` spells it
// (xla/backends/gpu/codegen/triton/tests/fusion_emitter_int4_device_test.cc:867-892) and as a
// checkpoint written for `y = x W^T` stores its matrices.  4-bit weights are packed two per byte
// along K (low nibble = the even k, xla/packing.cc:142-170), scales are [N] or [N, K/group].
//
// K-minor rows are already the matrix instruction's operand: for v_mfma_f32_16x16x32_bf16 lane
// (c, q) = (lane % 16, lane / 16) holds 8 consecutive k of row c, so a lane that fetches 16
// contiguous bytes of channel c owns two (s8) or four (s4) operands with no transposition.
// (The bytes are fetched quad-wise, 64 contiguous bytes per four lanes, and re-dealt to those
// lanes through a small wave-private LDS buffer: see NkStage::VIA_LDS.)
// A wave walks K for CT tiles of 16 channels and MT tiles of 16 tokens; the waves of a workgroup
// take neighbouring channels over the same k and share the activations through LDS.  Few
// channels: K is cut into slices (grid.z) whose f32 partial sums the finalize kernel adds in
// slice order.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <atomic>

#include "decode_common.h"

namespace xla_amd {
namespace {

constexpr uint32_t kPastEnd = 0x80000000u;  // every buffer here is smaller than 2 GiB
constexpr int kNkWaves = 4;

struct NkParams {
  DecodeParams d;        // operands, shapes, types, slices (strips: channel strips of kNkWaves*CT*16)
  int k_per_slice;       // multiple of the step (and of the group for group-factored sums)
  int group_shift;       // log2(group); 31 for one scale per channel
  int m_chunks;          // grid.y = batch * m_chunks, chunk c takes tokens [c*16*MT, +16*MT)
  int scale_batches;     // sets of scales (and zero points): the batch count, or 1 when all batches share one
};

// (scale groups are powers of two, or one per channel: shift 31)
static __device__ __forceinline__ uint32_t group_of(const NkParams& p, uint32_t k) { return k >> p.group_shift; }

// Stage geometry shared by the kernel and its launch.
template <int WBITS, int MT>
struct NkStage {
  static constexpr int KP = 128 / WBITS;                      // k per lane and step: 16 bytes of weights
  static constexpr int STEP = 4 * KP;                         // k per step (one b128 load per lane and tile)
  static constexpr int SPS = (WBITS == 4 && MT == 4) ? 2 : 4; // steps per stage
  static constexpr int KS = SPS * STEP;                       // k per stage
  static constexpr int ROWB = KS * 2 + 16;                    // LDS pitch of a token row: 16 tokens x 16 bytes
                                                              // then cover all 64 banks once
  static constexpr int TOK = 16 * MT;
  static constexpr int STAGE_BYTES = TOK * ROWB;
  static constexpr int CHUNKS = TOK * (KS / 8) / (kNkWaves * 64);  // 16-byte pieces a thread moves per stage
  // Whether a lane fetches the very bytes it multiplies (the four lanes of a quad then read four different
  // 64-byte segments, which the address unit serves at a quarter of its rate: its FIFO was full 59 % of
  // the time) or the wave fetches whole segments per quad and re-deals them through 1 KiB of LDS per
  // channel tile.  Measured on 8192 x 28672 s4: 41 -> 35 us up to 8 tokens, 41 -> 38 at 16, 52 -> 50 at
  // 32, but 58 -> 61 at 64, where the activation reads already keep LDS busy; s8 gains at every size.
  static constexpr bool VIA_LDS = !(WBITS == 4 && MT == 4);
};

// WBITS 8 | 4; MT token tiles; CT channel tiles per wave; MODE as in the [K,N] kernels:
// kRounded   bf16(w * s) per weight (bf16-typed multiply; group % KP == 0 or one scale per channel)
// kFactored  integers through the matrix cores, one scale per channel applied to the sum
// kGroupFactored  the same per scale group (group % (4*KP) == 0), folded with fma(sum, scale, total)
//
// K goes by in stages of SPS steps.  The workgroup's activations of a stage ([16 MT tokens][KS k])
// are fetched once, cooperatively, into one of two LDS buffers, from where every wave reads its
// matrix operands; a wave's weights (and scales) of the next stage are requested, all of them,
// before it starts on the current one, so a whole stage of loads is in flight per wave.  One
// barrier per stage.
// ZP: u4 weights with zero points.  The main loop has no branch: the scales of a bf16-typed multiply
// are bf16, and scales and zero points come through buffer descriptors with 32-bit offsets.
template <int WBITS, int MT, int CT, int MODE, bool ZP>
__global__ __launch_bounds__(kNkWaves * 64) void dequant_dot_nk_kernel(NkParams q) {
  const DecodeParams& p = q.d;
  using S = NkStage<WBITS, MT>;
  constexpr int KP = S::KP, NJ = KP / 8, STEP = S::STEP, SPS = S::SPS, KS = S::KS, ROWB = S::ROWB, CHUNKS = S::CHUNKS;
  constexpr bool GF = MODE == kGroupFactored;
  constexpr bool VIA_LDS = S::VIA_LDS;
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];  // [2][STAGE_BYTES], then [waves][CT][1024]
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int c = lane & 15, kq = lane >> 4;
  const int strip = blockIdx.x, slice = blockIdx.z;
  int batch = blockIdx.y / q.m_chunks, chunk = blockIdx.y % q.m_chunks;
  // ragged dot: grid.y walks work items, the chunks of 16 * MT rows of every group in group order
  // (groups + m_chunks of them at most; the sizes are read on the device); `batch` becomes the item's
  // group, [m_first, m_first + rows) its rows of the one [M,K] activation matrix; an item past the last
  // chunk has nothing to do
  int m_first = 0, m_rows = p.M;
  if (p.group_sizes) {
    int g_sel, begin_sel, rows_sel, last_end;
    ragged_item<16 * MT>(p, (int)blockIdx.y, lane, &g_sel, &begin_sel, &rows_sel, &last_end);
    if (g_sel < 0) return;  // (the whole workgroup, before any barrier)
    batch = g_sel;
    chunk = 0;
    m_first = begin_sel;
    m_rows = rows_sel;
  }
  const int a_batch = p.group_sizes ? 0 : batch;
  const int m0 = chunk * 16 * MT;
  const int rows_here = min(16 * MT, m_rows - m0);
  if (rows_here <= 0) return;  // (the whole workgroup, before any barrier)
  const int n_wave = (strip * kNkWaves + wave) * CT * 16;  // (a wave past N loads nothing and stores nothing)
  const int G = p.K / p.group;  // scales per channel
  const uint32_t row_bytes = (uint32_t)p.K * WBITS / 8;
  const size_t sbatch = p.scale_batched ? batch : 0;

  const __amdgpu_buffer_rsrc_t rw =
      make_rsrc(p.w + (size_t)batch * p.N * row_bytes, (uint32_t)p.N * row_bytes);
  const __amdgpu_buffer_rsrc_t ra =
      make_rsrc(p.lhs + ((size_t)a_batch * p.M + m_first + m0) * p.K, (uint32_t)rows_here * (uint32_t)p.K * 2u);
  // scales of a bf16-typed multiply: bf16 [N,G]; zero points: one nibble each, same shape
  const uint32_t sc_elems = (uint32_t)p.N * (uint32_t)G;
  const __amdgpu_buffer_rsrc_t rs = make_rsrc((const uint16_t*)p.scales + sbatch * sc_elems, sc_elems * 2u);
  const uint32_t zp_first = (uint32_t)(sbatch * sc_elems);  // element index of this batch's first zero point
  const __amdgpu_buffer_rsrc_t rz =
      make_rsrc(ZP ? p.zero_points : p.w, ZP ? (uint32_t)(((size_t)q.scale_batches * sc_elems + 1) >> 1) : 0u);
  uint32_t voff_w[CT], elem_s[CT];
#pragma unroll
  for (int t = 0; t < CT; ++t) {
    const int n = n_wave + t * 16 + c;
    // VIA_LDS: fetched by lane (channel lane / 4, piece lane % 4), a quad reading 64 contiguous bytes
    const int nf = VIA_LDS ? n_wave + t * 16 + (lane >> 2) : n;
    voff_w[t] = nf < p.N ? (uint32_t)nf * row_bytes + (VIA_LDS ? lane & 3 : kq) * 16 : kPastEnd;
    elem_s[t] = (uint32_t)max(0, min(n, p.N - 1)) * (uint32_t)G;
  }

  const int k_begin = slice * q.k_per_slice;
  const int k_end = min(p.K, k_begin + q.k_per_slice);

  floatx4 acc[CT][MT], tot[GF ? CT : 1][GF ? MT : 1];
#pragma unroll
  for (int t = 0; t < CT; ++t)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      acc[t][mt] = floatx4{0.f, 0.f, 0.f, 0.f};
      if (GF) tot[t][mt] = floatx4{0.f, 0.f, 0.f, 0.f};
    }

  uintx4 wq[2][SPS][CT], areg[CHUNKS];
  uint32_t sraw[2][SPS][CT], zraw[2][SPS][CT];  // kRounded / ZP: the lane's scale (bf16 bits) / zero point of the step
  const float z_default = WBITS == 4 ? (p.w_unsigned ? 0.0f : 8.0f) : 0.0f;

  // ---- the stage's activations: piece id = i * 256 + tid -> token row id / (KS/8), 8 k at (id % (KS/8)) * 8
  auto load_acts = [&](int ks) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < CHUNKS; ++i) {
      const int id = i * (kNkWaves * 64) + tid;
      const int row = id / (KS / 8), col = id % (KS / 8);
      const uint32_t k = (uint32_t)(ks + col * 8);
      // (K % 8 == 0: a piece lies inside its row or past it)
      areg[i] = __builtin_amdgcn_raw_buffer_load_b128(
          ra, row < rows_here && k < (uint32_t)k_end ? (uint32_t)row * (uint32_t)p.K * 2u + k * 2u : kPastEnd, 0, 0);
    }
  };
  auto store_acts = [&](int buf) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < CHUNKS; ++i) {
      const int id = i * (kNkWaves * 64) + tid;
      const int row = id / (KS / 8), col = id % (KS / 8);
      *reinterpret_cast<uintx4*>(lds + buf * S::STAGE_BYTES + row * ROWB + col * 16) = areg[i];
    }
  };
  auto load_weights = [&](int set, int ks) __attribute__((always_inline)) {
#pragma unroll
    for (int st = 0; st < SPS; ++st) {
      // a 16-byte piece lies inside its row or past it (the row pitch is a multiple of 16 bytes):
      // past it the lane must not read on into the next row
      const uint32_t kl = (uint32_t)(ks + st * STEP + kq * KP);
      const bool live = kl < (uint32_t)k_end;
      const bool live_f = (uint32_t)(ks + st * STEP + (VIA_LDS ? lane & 3 : kq) * KP) < (uint32_t)k_end;  // the piece this lane fetches
      const uint32_t wb = (uint32_t)(ks + st * STEP) * WBITS / 8;
#pragma unroll
      for (int t = 0; t < CT; ++t)
        wq[set][st][t] = __builtin_amdgcn_raw_buffer_load_b128(rw, live_f ? voff_w[t] + wb : kPastEnd, 0, 0);
      if constexpr (MODE == kRounded || ZP) {
        const uint32_t g = group_of(q, live ? kl : 0u);
#pragma unroll
        for (int t = 0; t < CT; ++t) {
          const uint32_t e = elem_s[t] + g;
          if constexpr (MODE == kRounded)
            sraw[set][st][t] = (uint32_t)(uint16_t)__builtin_amdgcn_raw_buffer_load_b16(rs, e * 2u, 0, 0);
          if constexpr (ZP) {
            const uint32_t ez = zp_first + e;  // nibble ez & 1 of byte ez >> 1
            zraw[set][st][t] = ((uint32_t)(uint8_t)__builtin_amdgcn_raw_buffer_load_b8(rz, ez >> 1, 0, 0)) | ((ez & 1u) << 8);
          }
        }
      }
    }
  };

  // whether the scale group ends with the step that starts at k0 (groups are whole steps)
  // ---- fetched pieces -> matrix operands, through 1 KiB of LDS that only this wave touches (LDS serves a
  // wave's instructions in order: no wait between the write and the read).  Lane (r, p) = (lane / 4,
  // lane % 4) holds piece p of channel r and writes it to slot p ^ (r / 4) of row r; lane (c, kq) reads
  // slot kq ^ (c / 4) of row c.  Both ways 16 lanes cover all 64 banks once.
  uint8_t* stage_w = lds + 2 * S::STAGE_BYTES + wave * (CT * 1024);
  const uint32_t st_wr = (uint32_t)(lane >> 2) * 64u + (uint32_t)(((lane & 3) ^ (lane >> 4)) << 4);
  const uint32_t st_rd = (uint32_t)c * 64u + (uint32_t)((kq ^ (c >> 2)) << 4);
  auto transpose = [&](int set, int st, uintx4* x) __attribute__((always_inline)) {
#pragma unroll
    for (int t = 0; t < CT; ++t) {
      if constexpr (VIA_LDS) {
        uint8_t* b = stage_w + t * 1024;  // (one buffer: the read of the step before was issued first)
        *reinterpret_cast<uintx4*>(b + st_wr) = wq[set][st][t];
        __builtin_amdgcn_wave_barrier();  // (no instruction: keeps the compiler from moving the read up)
        x[t] = *reinterpret_cast<const uintx4*>(b + st_rd);
      } else {
        x[t] = wq[set][st][t];
      }
    }
  };

  auto closes_group = [&](int k0) __attribute__((always_inline)) {
    return ((uint32_t)(k0 + STEP) & ((uint32_t)p.group - 1u)) == 0u;
  };

  auto compute = [&](int set, int st, int buf, int k0, const uintx4* xw) __attribute__((always_inline)) {
    float gs[CT][4] = {};
    const bool closing = GF && k0 < k_end && closes_group(k0);
    if (closing) {  // its scales, by output register
      const uint32_t g = group_of(q, (uint32_t)k0);
#pragma unroll
      for (int t = 0; t < CT; ++t)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int n = n_wave + t * 16 + 4 * kq + i;
          gs[t][i] = load_scale(p.scales, (sbatch * p.N + (size_t)max(0, min(n, p.N - 1))) * G + g, p.scale_is_bf16);
        }
    }
    // the lane's operands of the step: token 16 mt + c, k = st * STEP + kq * KP + 8 j ...
    uintx4 av[MT][NJ];
    const uint8_t* abase = lds + buf * S::STAGE_BYTES + c * ROWB + (st * STEP + kq * KP) * 2;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int j = 0; j < NJ; ++j)
        av[mt][j] = *reinterpret_cast<const uintx4*>(abase + mt * 16 * ROWB + j * 16);
#pragma unroll
    for (int t = 0; t < CT; ++t) {
      // 4-bit: nibble e of a dword arrives as the f16 value 1024 + u (even e) or 1024 + 16 u (odd e);
      // (u - z) * s = (1024 + u) * s - (1024 + z) * s = (1024 + 16 u) * (s / 16) - (64 + z) * s:
      // one fma each, exact for a scale of 8 significant bits with |1040 s| finite (an infinite scale
      // gives NaN where the product would be an infinity)
      float s = 1.0f, z = z_default;
      if constexpr (MODE == kRounded) s = bf16lo_to_f32(sraw[set][st][t]);
      if constexpr (ZP) z = (float)((zraw[set][st][t] >> ((zraw[set][st][t] >> 6) & 4u)) & 0xfu);  // bit 8: the high nibble
      const float s_even = s, c_even = s * -(1024.0f + z), s_odd = s * 0.0625f, c_odd = s * -(64.0f + z);
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        float f[8];
        if constexpr (WBITS == 4) {
          typedef _Float16 halfx2 __attribute__((ext_vector_type(2)));
          const uint32_t x = xw[t][j];
          // nibble pairs (0,4), (1,5) of x and (2,6), (3,7) of x >> 8, offset binary for s4 (the
          // sign bit flipped: u = w + 8), as they are for u4
          const uint32_t ce = p.w_unsigned ? 0x64006400u : 0x64086408u, co = p.w_unsigned ? 0x64006400u : 0x64806480u;
          const halfx2 p04 = __builtin_bit_cast(halfx2, __builtin_amdgcn_bitop3_b32(x, 0x000f000fu, ce, 0x6a));
          const halfx2 p15 = __builtin_bit_cast(halfx2, __builtin_amdgcn_bitop3_b32(x, 0x00f000f0u, co, 0x6a));
          const halfx2 p26 = __builtin_bit_cast(halfx2, __builtin_amdgcn_bitop3_b32(x >> 8, 0x000f000fu, ce, 0x6a));
          const halfx2 p37 = __builtin_bit_cast(halfx2, __builtin_amdgcn_bitop3_b32(x >> 8, 0x00f000f0u, co, 0x6a));
          f[0] = __builtin_fmaf((float)p04[0], s_even, c_even);
          f[1] = __builtin_fmaf((float)p15[0], s_odd, c_odd);
          f[2] = __builtin_fmaf((float)p26[0], s_even, c_even);
          f[3] = __builtin_fmaf((float)p37[0], s_odd, c_odd);
          f[4] = __builtin_fmaf((float)p04[1], s_even, c_even);
          f[5] = __builtin_fmaf((float)p15[1], s_odd, c_odd);
          f[6] = __builtin_fmaf((float)p26[1], s_even, c_even);
          f[7] = __builtin_fmaf((float)p37[1], s_odd, c_odd);
        } else {
          // 16 bytes are two operands: dwords (2j, 2j + 1)
          const uint32_t x0 = xw[t][j * 2], x1 = xw[t][j * 2 + 1];
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            f[e] = (float)(int8_t)((x0 >> (8 * e)) & 0xffu);
            f[4 + e] = (float)(int8_t)((x1 >> (8 * e)) & 0xffu);
          }
          if (MODE == kRounded) {
#pragma unroll
            for (int e = 0; e < 8; ++e) f[e] = f[e] * s;
          }
        }
        const uintx4 a = {pack_bf16x2(f[0], f[1]), pack_bf16x2(f[2], f[3]), pack_bf16x2(f[4], f[5]),
                          pack_bf16x2(f[6], f[7])};
        const bf16x8 aop = __builtin_bit_cast(bf16x8, a);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
          acc[t][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(aop, __builtin_bit_cast(bf16x8, av[mt][j]),
                                                               acc[t][mt], 0, 0, 0);
      }
    }
    if (closing) {
#pragma unroll
      for (int t = 0; t < CT; ++t)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            tot[t][mt][i] = __builtin_fmaf(acc[t][mt][i], gs[t][i], tot[t][mt][i]);
            acc[t][mt][i] = 0.0f;
          }
    }
  };
  // Steps past k_end run on zeros (their loads are masked) rather than being branched around: a
  // branch between a stage's loads and their use lets the compiler move the loads down to the use.
  auto compute_stage = [&](int set, int ks) __attribute__((always_inline)) {
    uintx4 xw[2][CT];  // the operands of this step and, requested one step ahead, of the next
    transpose(set, 0, xw[0]);
#pragma unroll
    for (int st = 0; st < SPS; ++st) {
      if (st + 1 < SPS) transpose(set, st + 1, xw[(st + 1) & 1]);
      compute(set, st, set, ks + st * STEP, xw[st & 1]);  // (buffer index = register set)
    }
  };

  load_acts(k_begin);
  load_weights(0, k_begin);
  store_acts(0);
  __syncthreads();
  for (int ks = k_begin; ks < k_end; ks += 2 * KS) {  // two stages a round; the second may lie past k_end
    load_acts(ks + KS);
    load_weights(1, ks + KS);
    __builtin_amdgcn_sched_barrier(0);  // (keeps the next stage's loads above this stage's arithmetic)
    compute_stage(0, ks);
    __builtin_amdgcn_sched_barrier(0);
    store_acts(1);  // nobody reads buffer 1 any more: every wave passed the barrier that ended its stage
    __syncthreads();
    load_acts(ks + 2 * KS);
    load_weights(0, ks + 2 * KS);
    __builtin_amdgcn_sched_barrier(0);
    compute_stage(1, ks + KS);
    __builtin_amdgcn_sched_barrier(0);
    store_acts(0);
    __syncthreads();
  }

  // ---- lane (c, kq), register i of tile (t, mt): channel n_wave + 16 t + 4 kq + i, token m0 + 16 mt + c.
  // One tile at a time (the fences keep the scheduler from interleaving the tiles' activations,
  // which would hold every tile's temporaries in registers at once).
  // (expanded, not unrolled: with the general stores in its body the compiler left the tile loop
  // rolled, and accumulators indexed by a run-time t live in scratch memory -- also in the main loop)
  const bool quads = p.N % 4 == 0;
  static_for<0, CT>([&](auto tile_index) {
    constexpr int t = decltype(tile_index)::value;
    float fq[4], bq[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int n = max(0, min(n_wave + t * 16 + 4 * kq + i, p.N - 1));
      fq[i] = MODE == kFactored && p.slices == 1 ? load_scale(p.scales, sbatch * p.N + n, p.scale_is_bf16) : 1.0f;
      bq[i] = p.bias && p.slices == 1 ? load_scale(p.bias, n, p.bias_is_bf16) : 0.0f;
    }
    static_for<0, MT>([&](auto token_tile) {
      constexpr int mt = decltype(token_tile)::value;
      float v[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        if constexpr (GF) v[i] = tot[t][mt][i] * fq[i];
        else v[i] = acc[t][mt][i] * fq[i];
      }
      if (p.slices == 1) epilogue_all_dispatch<4>(v, bq, p.epilogue, p.bf16_dot, p.bf16_ops);
      const int n = n_wave + t * 16 + 4 * kq, m = mt * 16 + c;
      if (m < rows_here && n < p.N) {
        const size_t o = ((size_t)a_batch * p.M + m_first + m0 + m) * p.N + n;
        if (p.slices > 1) {
          float* dst = p.workspace + ((size_t)batch * p.slices + slice) * ((size_t)p.M * p.N) + (size_t)(m0 + m) * p.N + n;
          if (quads) {
            *reinterpret_cast<floatx4*>(dst) = floatx4{v[0], v[1], v[2], v[3]};
          } else {
#pragma unroll
            for (int i = 0; i < 4; ++i)
              if (n + i < p.N) dst[i] = v[i];
          }
        } else if (p.out_f32 | p.out_transposed | p.out_f8) {
#pragma unroll
          for (int i = 0; i < 4; ++i)
            if (n + i < p.N) StoreResult(p, a_batch, m_first + m0 + m, n + i, v[i]);
        } else if (quads) {
          *reinterpret_cast<uintx2*>(p.out + o) = uintx2{pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3])};
        } else {
#pragma unroll
          for (int i = 0; i < 4; ++i)
            if (n + i < p.N) p.out[o + i] = f32_to_bf16(v[i]);
        }
      }
      __builtin_amdgcn_sched_barrier(0);
    });
  });
}

// Any shape and alignment: one thread per output, k in increasing order.
__global__ __launch_bounds__(256) void dequant_dot_nk_generic_kernel(DecodeParams p, int wbits, int mode) {
  const size_t total = (size_t)p.M * p.N;
  const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
  const int batch = blockIdx.y;
  if (idx >= total) return;
  const int n = (int)(idx % p.N), m = (int)(idx / p.N);
  const int G = p.K / p.group;
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
  const size_t wrow = ((size_t)wbatch * p.N + n) * p.K;                     // in elements
  const size_t srow = ((size_t)(p.scale_batched ? wbatch : 0) * p.N + n) * G;
  float acc = 0.0f;
  for (int k = 0; k < k_end; ++k) {
    const size_t e = wrow + k;
    int wi;
    if (wbits == 8) {
      wi = (int8_t)p.w[e];
    } else {
      const uint32_t nib = (p.w[e >> 1] >> (4 * (e & 1))) & 0xfu;
      wi = p.w_unsigned ? (int)nib : (int)(nib ^ 8u) - 8;
      if (p.zero_points) {
        const size_t ze = srow + k / p.group;
        wi -= (int)((p.zero_points[ze >> 1] >> (4 * (ze & 1))) & 0xfu);
      }
    }
    float wv = (float)wi * load_scale(p.scales, srow + k / p.group, p.scale_is_bf16);
    if (mode == kRounded) wv = round_bf16(wv);
    acc = acc + bf16_to_f32(a[(size_t)k * a_step]) * wv;
  }
  const float b = p.bias ? load_scale(p.bias, n, p.bias_is_bf16) : 0.0f;
  StoreResult(p, batch, m, n, epilogue_dispatch(acc, b, p.epilogue, p.bf16_dot, p.bf16_ops));
}

// Ragged dot: rows past the last group are a dot of nothing, epilogue(0).  Workgroup (x, y) takes 256
// channels and every gridDim.y-th of those rows; usually there are none and it returns at once.
__global__ __launch_bounds__(256) void nk_ragged_tail_rows_kernel(DecodeParams p) {
  int begin, rows;
  ragged_rows(p, p.ragged_groups - 1, &begin, &rows);
  const int n = blockIdx.x * 256 + threadIdx.x;
  if (n >= p.N) return;
  const float bias = p.bias ? load_scale(p.bias, n, p.bias_is_bf16) : 0.0f;
  const uint16_t v = f32_to_bf16(epilogue_dispatch(0.0f, bias, p.epilogue, p.bf16_dot, p.bf16_ops));
  for (int m = begin + rows + blockIdx.y; m < p.M; m += gridDim.y) p.out[(size_t)m * p.N + n] = v;
}

template <int WBITS, int MT, int CT, int MODE, bool ZP>
int launch_nk(const NkParams& q, int batch, hipStream_t stream, const char* name) {
  constexpr size_t kLds = 2 * (size_t)NkStage<WBITS, MT>::STAGE_BYTES +
                          (NkStage<WBITS, MT>::VIA_LDS ? (size_t)kNkWaves * CT * 1024 : 0);
  // per kernel instantiation and device: one bit per device ordinal (two threads that race set the
  // attribute to the same value)
  static std::atomic<unsigned long long> configured{0};
  int device = 0;
  (void)hipGetDevice(&device);
  const unsigned long long bit = 1ull << (device & 63);
  if (kLds > 48 * 1024 && !(configured.load(std::memory_order_acquire) & bit)) {
    hipError_t e = hipFuncSetAttribute((const void*)dequant_dot_nk_kernel<WBITS, MT, CT, MODE, ZP>,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)kLds);
    if (e != hipSuccess)
      return Fail(XLA_FFI_Error_Code_INTERNAL, "%s: cannot reserve %zu bytes of LDS: %s", name, kLds, hipGetErrorString(e));
    configured.fetch_or(bit, std::memory_order_release);
  }
  // (a ragged dot: one grid row per chunk any group can have)
  dim3 grid((unsigned)q.d.strips, (unsigned)(q.d.group_sizes ? batch + q.m_chunks : batch * q.m_chunks), (unsigned)q.d.slices);
  hipLaunchKernelGGL((dequant_dot_nk_kernel<WBITS, MT, CT, MODE, ZP>), grid, dim3(kNkWaves * 64), kLds, stream, q);
  int rc = CheckLaunch(name);
  if (rc) return rc;
  if (q.d.slices > 1) rc = LaunchDecodeFinalize(q.d, batch, stream, MODE);
  if (q.d.group_sizes && rc == 0) {
    hipLaunchKernelGGL(nk_ragged_tail_rows_kernel, dim3((unsigned)((q.d.N + 255) / 256), 16u), dim3(256), 0, stream, q.d);
    rc = CheckLaunch("dequant_dot_nk_ragged_tail_rows");
  }
  SetLastKernel(name);
  return rc;
}

struct NkShape {
  int wbits, kp, step, mt, ct, strips, m_chunks, slices, k_per_slice;
};

// Token tiles, channel tiles and K-slices for a shape the streaming kernel takes.
// tile_rows: the rows that decide the number of token tiles (a ragged dot: about what a group owns), 0 = M.
NkShape PlanNk(int64_t batch, int64_t M, int64_t K, int64_t N, bool four_bit, int64_t slice_unit, bool tuned_ct = true,
               int64_t tile_rows = 0) {
  NkShape s;
  s.wbits = four_bit ? 4 : 8;
  s.kp = 128 / s.wbits;
  s.step = 4 * s.kp;
  if (tile_rows <= 0) tile_rows = M;
  s.mt = tile_rows <= 16 ? 1 : tile_rows <= 32 ? 2 : 4;
  // One token tile: a channel tile per wave and about four workgroups per CU measured fastest on
  // 8192 x 28672 s4 (1 / 2 / 4 slices: 55.6 / 48.3 / 44.1 us with one tile per wave, 78.9 / 55.2 /
  // 57.5 us with two); more token tiles: two channel tiles per wave, two workgroups per CU.
  s.ct = s.mt == 1 ? 1 : 2;
  if (int v = tuned_ct ? GetOption("dequant_dot_nk_ct") : 0) s.ct = s.mt != 1 ? 2 : v == 1 ? 1 : v == 4 ? 4 : 2;  // (one token tile only)
  s.strips = (int)((N + kNkWaves * s.ct * 16 - 1) / (kNkWaves * s.ct * 16));
  s.m_chunks = (int)((M + 16 * s.mt - 1) / (16 * s.mt));
  // few workgroups: cut K while a slice keeps eight steps (or whole groups) and the partial sums
  // (written and read again) stay below half a byte per weight.  One token tile: up to four ways,
  // towards four workgroups per CU; more: up to eight ways, towards two per CU
  // (s4 [64,14336] x [4096,14336]^T: 60 us in two slices, 26 in eight; [64,28672] x [8192,28672]^T 64 -> 54).
  const int64_t unit = slice_unit > s.step ? slice_unit : s.step;
  const int64_t want = s.mt == 1 ? 1024 : 448;
  const int most = s.mt == 1 ? 4 : 8;
  int slices = 1;
  const int64_t wgs = (int64_t)s.strips * batch * s.m_chunks;
  while (slices < most && wgs * slices < want && K / (slices * 2) >= 8 * s.step &&
         (K / (slices * 2)) % unit == 0 && 2.0 * (slices * 2) * M * N * 4.0 <= 0.5 * (double)K * N)
    slices *= 2;
  if (int v = GetOption("dequant_dot_slices")) {
    if (K % (v * unit) == 0) slices = v;
  }
  s.slices = slices;
  s.k_per_slice = (int)((K / slices + unit - 1) / unit * unit);
  return s;
}

}  // namespace

int LaunchDequantDotPrefillNk(const XlaAmdDequantDot& p, hipStream_t stream);  // tiled_dot_mfma.hip

size_t DequantDotNkWorkspaceBytes(int64_t batch, int64_t M, int64_t K, int64_t N, bool four_bit) {
  if (batch <= 0 || M <= 0 || K <= 0 || N <= 0) return 0;
  // more than 64 tokens may run on the tiled kernel, which splits the tiles of a short last round
  if (M > 64) {
    const size_t tail = TiledTailWorkspaceBytes(batch, M, K, N);
    const size_t slices = DequantDotWorkspaceBytes(batch, M, N, PlanNk(batch, M, K, N, four_bit, 0).slices);
    return tail > slices ? tail : slices;
  }
  // (the group is not known here: a slice of whole 128-k steps holds whole groups only when the
  // group divides it, which the launch checks again; sizing assumes the most slices)
  const NkShape s = PlanNk(batch, M, K, N, four_bit, 0);
  return DequantDotWorkspaceBytes(batch, M, N, s.slices);
}

int LaunchDequantDotNk(DecodeParams dp, const XlaAmdDequantDot& p, hipStream_t stream) {
  const bool four_bit = p.weight_dtype != XLA_FFI_DataType_S8;
  const int wbits = four_bit ? 4 : 8;
  const int kp = 128 / wbits;
  const bool per_channel = p.group == p.K;
  // f32-typed multiply: one scale per channel factors out of the whole sum, scales per group of whole
  // steps out of each group's sum; other groups under an f32 multiply take the one-thread-per-output kernel
  const int mode = p.dequant_type == XLA_FFI_DataType_BF16 ? kRounded
                   : per_channel || p.group % (4 * kp) != 0 ? kFactored
                                                            : kGroupFactored;
  const int64_t row_bytes = p.K * wbits / 8;
  int group_shift = per_channel ? 31 : -1;  // (k >> 31 == 0: the one scale of the channel)
  for (int s = 0; s < 31 && !per_channel; ++s)
    if ((int64_t)1 << s == p.group) group_shift = s;
  const bool ragged = p.group_sizes != nullptr;
  // (a ragged dot takes the tiled kernel -- 256-row tiles per group -- once the groups average 96 rows)
  const bool plain = !dp.out_f32 && !dp.out_f8 && !dp.out_transposed && !dp.lhs_k_major;  // else: no tiled kernel
  if (plain && p.M > 64 && (!ragged || GetOption("dequant_dot_kernel") == 3 || p.M / p.batch >= 96) &&
      GetOption("dequant_dot_kernel") != 1 && GetOption("dequant_dot_kernel") != 2) {
    const int rc = LaunchDequantDotPrefillNk(p, stream);
    if (rc >= 0) return rc;  // -1: the tiled kernel does not take it (or token chunks are cheaper)
  }
  bool fast = row_bytes % 16 == 0 && p.K >= 4 * kp && ((uintptr_t)p.lhs % 16 == 0) && ((uintptr_t)p.weights % 16 == 0) &&
              (double)p.N * row_bytes < 2147483648.0 && (double)p.M * p.K * 2 < 2147483648.0 &&
              p.batch * ((p.M + 15) / 16) <= 65535 && GetOption("dequant_dot_kernel") != 1 &&
              (!ragged || (double)p.M * p.N * 2 < 2147483648.0);
  if (group_shift < 0) fast = false;  // groups are powers of two, or one scale per channel
  if (dp.lhs_k_major) fast = false;   // the streaming kernel reads activations [M,K]
  if ((double)p.scale_batch * p.N * (p.K / p.group) * 4 >= 2147483648.0) fast = false;  // 32-bit offsets into the scales
  if (mode == kRounded && !per_channel && p.group % kp != 0) fast = false;
  if (mode == kFactored && !per_channel) fast = false;  // an f32 multiply by scales that do not cover whole steps
  if (p.zero_points && !per_channel && p.group % kp != 0) fast = false;
  if (!fast) {
    if (GetOption("dequant_dot_kernel") == 2 || GetOption("dequant_dot_kernel") == 3)
      return Fail(XLA_FFI_Error_Code_FAILED_PRECONDITION, "dequant_dot: the requested kernel does not cover this shape");
    dp.slices = 1;
    dim3 grid((unsigned)(((size_t)p.M * p.N + 255) / 256), (unsigned)(ragged ? 1 : p.batch));
    hipLaunchKernelGGL(dequant_dot_nk_generic_kernel, grid, dim3(256), 0, stream, dp, wbits,
                       mode == kGroupFactored ? (int)kFactored : mode);
    SetLastKernel("dequant_dot_nk_generic");
    return CheckLaunch("dequant_dot_nk_generic");
  }
  const bool zp = p.zero_points != nullptr;
  // (a ragged dot: any group may own any number of the rows; token tiles for twice the average)
  const int64_t tile_rows = ragged ? std::min<int64_t>(p.M, 2 * ((p.M + p.batch - 1) / p.batch)) : 0;
  NkShape s = PlanNk(p.batch, p.M, p.K, p.N, four_bit, mode == kGroupFactored ? p.group : 0, /*tuned_ct=*/!zp, tile_rows);
  if (ragged || (s.slices > 1 && (!p.workspace || p.workspace_bytes < DequantDotWorkspaceBytes(p.batch, p.M, p.N, s.slices)))) {
    // (a group's rows are only known on the device: every group is one workgroup per strip and token chunk)
    s.slices = 1;
    s.k_per_slice = (int)p.K;
  }
  NkParams q;
  q.d = dp;
  q.d.strips = s.strips;
  q.d.slices = s.slices;
  q.k_per_slice = s.k_per_slice;
  q.group_shift = group_shift;
  q.m_chunks = s.m_chunks;
  q.scale_batches = dp.scale_batched ? (int)p.batch : 1;
#define XLA_AMD_NK(WB, MT_, CT_, MODE_, NAME)                                             \
  if (wbits == WB && s.mt == MT_ && s.ct == CT_ && mode == MODE_) {                       \
    if constexpr (WB == 4 && CT_ == (MT_ == 1 ? 1 : 2))                                   \
      if (zp) return launch_nk<WB, MT_, CT_, MODE_, true>(q, (int)p.batch, stream, NAME "_zp"); \
    return launch_nk<WB, MT_, CT_, MODE_, false>(q, (int)p.batch, stream, NAME);          \
  }
#define XLA_AMD_NK_MODES(WB, MT_, CT_, TAG)                                         \
  XLA_AMD_NK(WB, MT_, CT_, kRounded, "dequant_dot_nk_" TAG "_rounded")              \
  XLA_AMD_NK(WB, MT_, CT_, kFactored, "dequant_dot_nk_" TAG "_factored")            \
  XLA_AMD_NK(WB, MT_, CT_, kGroupFactored, "dequant_dot_nk_" TAG "_group_factored")
  XLA_AMD_NK_MODES(4, 1, 1, "s4_m16")
  XLA_AMD_NK_MODES(4, 2, 2, "s4_m32")
  XLA_AMD_NK_MODES(4, 4, 2, "s4_m64")
  XLA_AMD_NK_MODES(8, 1, 1, "s8_m16")
  XLA_AMD_NK_MODES(8, 2, 2, "s8_m32")
  XLA_AMD_NK_MODES(8, 4, 2, "s8_m64")
  XLA_AMD_NK_MODES(4, 1, 2, "s4_m16_c2")
  XLA_AMD_NK_MODES(4, 1, 4, "s4_m16_c4")
  XLA_AMD_NK_MODES(8, 1, 2, "s8_m16_c2")
  XLA_AMD_NK_MODES(8, 1, 4, "s8_m16_c4")
#undef XLA_AMD_NK_MODES
#undef XLA_AMD_NK
  return Fail(XLA_FFI_Error_Code_INTERNAL, "dequant_dot: no [N,K] kernel for this shape");
}

}  // namespace xla_amd
