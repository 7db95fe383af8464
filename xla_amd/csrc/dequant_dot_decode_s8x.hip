// Decode dequantize-dot for small matrices: s8 weights [K,N] with one scale per output channel under
// an f32-typed multiply, up to 16 tokens, in ONE launch.
//
//   out[b,m,n] = epilogue( scale[n] * sum_k lhs[b,m,k] * w[b,k,n] )
//
// A matrix of a few MB is over in a couple of microseconds of HBM time, so the kernel is all
// latency: nothing may wait for anything it could have asked for earlier.  A workgroup of 8 waves
// owns 128 channels (one 128-byte line per row of s8) and 256 * STEPS rows -- or 64 channels where
// the wide strips would be fewer workgroups than the chip has CUs: half the bytes per workgroup
// for the same number of slices to wait for ([16,4096]x[4096,4096]: 8.2 -> 7.1 us).  Every wave
// requests ALL its weights (STEPS steps of 32 rows, 8 or 4 bytes per lane and row) and activations
// before it touches the first, so one round trip to memory covers the whole matrix.  The integers go through
// v_mfma_f32_16x16x32_bf16 exactly (an s8 value is a bf16 value), the waves add their tiles
// through LDS, and the K-slices of a strip add up inside the kernel: every slice but the last
// stores its f32 sums with device-scope stores and raises a flag; the last slice -- dispatched
// after the others, so what it waits for is already running -- adds them in slice order, applies
// scale, bias and activation and writes the bf16 result.  The order of every addition is fixed, so
// results do not depend on scheduling.
//
// Bound: HBM.  Algorithmic bytes: K*N (weights) + scale, bias, lhs and out once each.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "decode_common.h"
#include "device_numerics.h"
#include "launch.h"

namespace xla_amd {
namespace {

constexpr int kWaves = 8;

// NV: channels per lane, 8 (strips of 128 channels, one 128-byte line per row) or 4 (strips of 64:
// half the bytes per workgroup, for matrices whose wide strips would leave CUs without one)
template <int STEPS, int NV>
__global__ __launch_bounds__(kWaves * 64) void dequant_dot_decode_s8x_kernel(DecodeParams p) {
  constexpr int kStripChannels = 16 * NV;
  constexpr int kSumsPerStrip = 16 * kStripChannels;  // f32 sums of one 16-token tile
  constexpr int R = 4 * NV;   // accumulator registers per lane
  constexpr int RPW = R / kWaves;
  __shared__ float lds[kWaves * R * 64];  // 64 or 32 KiB
  __shared__ int lds_all_here;

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int li = lane & 15, kb = lane >> 4;
  // workgroup ids in dispatch order: the slices of a strip follow each other, the finisher last
  int slice = blockIdx.x % p.slices;
  int strip = blockIdx.x / p.slices;
  if (NV == 4 && p.pairs_per_group) {
    const int low = blockIdx.x & 7;
    slice = low % p.slices;
    strip = 2 * ((blockIdx.x >> 4) * p.pairs_per_group + low / p.slices) + ((blockIdx.x >> 3) & 1);
    if (strip >= p.strips) return;  // the grid is padded to whole groups of 16
  }
  const int batch = blockIdx.y;
  const bool finisher = slice == p.slices - 1;

  const int n_lane = strip * kStripChannels + li * NV;
  const uint32_t pitch = (uint32_t)p.N;
  const __amdgpu_buffer_rsrc_t rw = make_rsrc(p.w + (size_t)batch * p.K * pitch, (uint32_t)p.K * pitch);
  // token li of the one 16-token tile; tokens >= M lie past the end and read as zeros
  const __amdgpu_buffer_rsrc_t ra = make_rsrc(p.lhs + (size_t)batch * p.M * p.K, (uint32_t)p.M * p.K * 2u);
  constexpr uint32_t kNowhere = 0x80000000u;
  const uint32_t voff_w = n_lane < p.N ? (uint32_t)(8 * kb) * pitch + (uint32_t)n_lane : kNowhere;
  const uint32_t voff_a = ((uint32_t)li * p.K + 8 * kb) * 2u;
  const int k_begin = slice * p.rows_per_slice + wave * (32 * STEPS);  // rows_per_slice = 256 * STEPS

  // ---- every load of this wave, at once
  uint32_t wq[STEPS][8][NV / 4];
  uintx4 aq[STEPS];
#pragma unroll
  for (int s = 0; s < STEPS; ++s) {
    const int k0 = k_begin + 32 * s;
    aq[s] = __builtin_amdgcn_raw_buffer_load_b128(ra, voff_a + (uint32_t)k0 * 2u, 0, 0);
#pragma unroll
    for (int r = 0; r < 8; ++r) buffer_load_words<NV / 4>(rw, voff_w + (uint32_t)k0 * pitch, (uint32_t)r * pitch, wq[s][r]);
  }
  // what the finisher's epilogue needs, requested now as well: the lane ends up with channels
  // n0 .. n0+RPW-1 of token li (see the reduction below)
  const int n0 = strip * kStripChannels + (4 * kb + (wave >> 1)) * NV + (wave & 1) * RPW;
  // (raw bits now, converted after the arithmetic: a conversion here would wait for every load above)
  const int bias_esz = p.bias_is_bf16 ? 2 : 4, scale_esz = p.scale_is_bf16 ? 2 : 4;
  const __amdgpu_buffer_rsrc_t rbias = make_rsrc(p.bias, p.bias ? (uint32_t)p.N * bias_esz : 0u);
  const __amdgpu_buffer_rsrc_t rscale = make_rsrc(
      (const char*)p.scales + (size_t)(p.scale_batched ? batch : 0) * p.N * scale_esz, (uint32_t)p.N * scale_esz);
  // N % 8 == 0 and n0 % RPW == 0: the lane's RPW values are inside the vector or not at all (with
  // RPW = 2 the loads reach two values further, past the end at most: those read as zeros)
  const bool ep_live = finisher && n0 < p.N;
  // two 8-byte loads whatever the type (bf16: the second one goes nowhere): no branch for the
  // compiler to put a wait in front of
  auto load_four = [&](__amdgpu_buffer_rsrc_t r, bool is_bf16) -> uintx4 {
    const uint32_t first = ep_live ? (uint32_t)n0 * (is_bf16 ? 2u : 4u) : kNowhere;
    const uintx2 lo = __builtin_amdgcn_raw_buffer_load_b64(r, first, 0, 0);
    const uintx2 hi = __builtin_amdgcn_raw_buffer_load_b64(r, is_bf16 || !ep_live ? kNowhere : first + 8u, 0, 0);
    return uintx4{lo[0], lo[1], hi[0], hi[1]};
  };
  const uintx4 bias_raw = load_four(rbias, p.bias_is_bf16 != 0);
  const uintx4 scale_raw = load_four(rscale, p.scale_is_bf16 != 0);
  __builtin_amdgcn_sched_barrier(0);  // the loads stay up here, ahead of the arithmetic
  auto four_value = [](const uintx4& raw, bool is_bf16, int u) {
    return is_bf16 ? ((u & 1) ? bf16hi_to_f32(raw[u >> 1]) : bf16lo_to_f32(raw[u >> 1])) : bits_to_f32(raw[u]);
  };

  floatx4 acc[NV];
#pragma unroll
  for (int j = 0; j < NV; ++j) acc[j] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int s = 0; s < STEPS; ++s) {
    const bf16x8 bop = __builtin_bit_cast(bf16x8, aq[s]);
#pragma unroll
    for (int q = 0; q < NV / 4; ++q)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        float f[8];
#pragma unroll
        for (int r = 0; r < 8; ++r) f[r] = (float)(int8_t)((wq[s][r][q] >> (8 * e)) & 0xffu);
        const uintx4 a = {pack_bf16x2(f[0], f[1]), pack_bf16x2(f[2], f[3]), pack_bf16x2(f[4], f[5]),
                          pack_bf16x2(f[6], f[7])};
        acc[q * 4 + e] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), bop, acc[q * 4 + e], 0, 0, 0);
      }
  }

  // ---- the waves' tiles added through LDS in wave order.  Register c = t * NV + j of lane (li, kb)
  // is channel (4 * kb + t) * NV + j of the strip, token li; wave w finishes registers 4w .. 4w+3.
#pragma unroll
  for (int c = 0; c < R; ++c) lds[(wave * R + c) * 64 + lane] = acc[c % NV][c / NV];
  __syncthreads();
  float res[RPW];
#pragma unroll
  for (int u = 0; u < RPW; ++u) {
    float s = 0.0f;
#pragma unroll
    for (int w2 = 0; w2 < kWaves; ++w2) s = s + lds[(w2 * R + wave * RPW + u) * 64 + lane];
    res[u] = s;
  }

  // ---- the slices of the strip, added by its last one.  Sums travel in the threads' own order, 16
  // bytes per thread, as device-scope stores and loads: no cache maintenance on either side.
  constexpr int kDeviceScope = 16;  // sc1: the access is performed where every XCD sees it
  const int others = p.slices - 1;
  const size_t strip_index = (size_t)batch * p.strips + strip;
  // per strip: one flag per producing slice, then the strip's generation
  unsigned long long* const flags = p.flags + strip_index * (size_t)(others + 1);
  unsigned long long target = 0;  // only read where it is used: thread 0 of a producer, the watching lanes
  if (others > 0 && (finisher ? (wave == 0 && lane < others) : tid == 0)) target = HandOverTarget(p.epoch, flags + others);
  bool all_here = true;
  if (others > 0) {
    const __amdgpu_buffer_rsrc_t rh =
        make_rsrc(p.workspace + strip_index * (size_t)others * kSumsPerStrip, (uint32_t)others * kSumsPerStrip * 4u);
    if (!finisher) {
      if constexpr (RPW == 4)
        __builtin_amdgcn_raw_buffer_store_b128(
            uintx4{f32_to_bits(res[0]), f32_to_bits(res[1]), f32_to_bits(res[2]), f32_to_bits(res[3])}, rh,
            (uint32_t)((slice * (kWaves * 64) + tid) * 16), 0, kDeviceScope);
      else
        __builtin_amdgcn_raw_buffer_store_b64(uintx2{f32_to_bits(res[0]), f32_to_bits(res[1])}, rh,
                                              (uint32_t)((slice * (kWaves * 64) + tid) * 8), 0, kDeviceScope);
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      __syncthreads();
      if (tid == 0 && !p.handover_test) __hip_atomic_store(flags + slice, target, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      return;
    }
    if (wave == 0) {  // lane s < others watches slice s (at most 15 of them)
      int ok = 1;
      if (lane < others) {
        ok = 0;
        const int spins = p.handover_test ? kHandOverTestSpins : kHandOverSpins;
        for (int spin = 0; spin < spins; ++spin) {
          if (__hip_atomic_load(flags + lane, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == target) { ok = 1; break; }
          __builtin_amdgcn_s_sleep(4);
        }
      }
      const int all_ok = __all(ok);
      if (lane == 0) lds_all_here = all_ok;
    }
    __syncthreads();
    all_here = lds_all_here != 0;
    if (all_here) {
      // slice 0 first, this workgroup's own sums last
      float v[RPW];
#pragma unroll
      for (int u = 0; u < RPW; ++u) v[u] = 0.0f;
      for (int s0 = 0; s0 < others; s0 += 4) {
        uintx4 o[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const uint32_t at = s0 + i < others ? (uint32_t)(((s0 + i) * (kWaves * 64) + tid) * (4 * RPW)) : kNowhere;
          if constexpr (RPW == 4) {
            o[i] = __builtin_amdgcn_raw_buffer_load_b128(rh, at, 0, kDeviceScope);
          } else {
            const uintx2 h = __builtin_amdgcn_raw_buffer_load_b64(rh, at, 0, kDeviceScope);
            o[i] = uintx4{h[0], h[1], 0u, 0u};
          }
        }
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (s0 + i < others) {
#pragma unroll
            for (int u = 0; u < RPW; ++u) v[u] = v[u] + bits_to_f32(o[i][u]);
          }
      }
#pragma unroll
      for (int u = 0; u < RPW; ++u) res[u] = v[u] + res[u];
      // the strip moves on to its next generation: the next run (also a replay of this launch from a
      // captured graph) waits for new sums
      if (tid == 0) HandOverNextGeneration(flags + others, target);
    }
  }
  if (all_here) {
    float bq[RPW];
#pragma unroll
    for (int u = 0; u < RPW; ++u) {
      res[u] = res[u] * four_value(scale_raw, p.scale_is_bf16 != 0, u);
      bq[u] = four_value(bias_raw, p.bias_is_bf16 != 0, u);  // zeros without a bias
    }
    epilogue_all_dispatch<RPW>(res, bq, p.epilogue, p.bf16_dot, p.bf16_ops);
    if (li < p.M && n0 < p.N) {
      uint16_t* dst = p.out + ((size_t)batch * p.M + li) * p.N + n0;
      if (n0 + RPW <= p.N) {  // N % 4 == 0 and n0 % RPW == 0: whole and aligned
        if constexpr (RPW == 4)
          *reinterpret_cast<uintx2*>(dst) = uintx2{pack_bf16x2(res[0], res[1]), pack_bf16x2(res[2], res[3])};
        else
          *reinterpret_cast<uint32_t*>(dst) = pack_bf16x2(res[0], res[1]);
      } else {
#pragma unroll
        for (int u = 0; u < RPW; ++u)
          if (n0 + u < p.N) dst[u] = f32_to_bf16(res[u]);
      }
    }
    return;
  }
  // ---- a flag that never showed (bounded wait above): the strip over all of K by the plain loop
  for (int ch = wave; ch < kStripChannels; ch += kWaves) {
    const int n = strip * kStripChannels + ch;
    if (n >= p.N) continue;
    for (int m = 0; m < p.M; ++m) {
      const uint16_t* arow = p.lhs + ((size_t)batch * p.M + m) * p.K;
      const uint8_t* wb = p.w + (size_t)batch * p.K * pitch;
      float v = 0.0f;
      for (int k = lane; k < p.K; k += 64) v = v + bf16_to_f32(arow[k]) * (float)(int8_t)wb[(size_t)k * pitch + n];
#pragma unroll
      for (int sh = 32; sh >= 1; sh >>= 1) v = v + __shfl_xor(v, sh);
      if (lane != 0) continue;
      v = v * load_scale(p.scales, (size_t)(p.scale_batched ? batch : 0) * p.N + n, p.scale_is_bf16);
      const float b = p.bias ? load_scale(p.bias, n, p.bias_is_bf16) : 0.0f;
      p.out[((size_t)batch * p.M + m) * p.N + n] = f32_to_bf16(epilogue_dispatch(v, b, p.epilogue, p.bf16_dot, p.bf16_ops));
    }
  }
  if (tid == 0) HandOverNextGeneration(flags + others, target);  // a flag raised late belongs to the old generation
}

template <int STEPS, int NV>
int launch_s8x(const DecodeParams& dp, int batch, hipStream_t stream, const char* name) {
  dim3 grid((unsigned)(dp.strips * dp.slices), (unsigned)batch);
  if (NV == 4 && dp.pairs_per_group) {
    const int pairs = (dp.strips + 1) / 2;
    grid.x = (unsigned)((pairs + dp.pairs_per_group - 1) / dp.pairs_per_group * 16);
  }
  hipLaunchKernelGGL((dequant_dot_decode_s8x_kernel<STEPS, NV>), grid, dim3(kWaves * 64), 0, stream, dp);
  const int rc = CheckLaunch(name);
  SetLastKernel(name);
  return rc;
}

struct S8xShape {
  int steps;    // steps of 32 rows per wave; 0: the shape is not one for this kernel
  int channels; // per strip: 128 or 64
  int64_t strips, slices;
  size_t sums_bytes() const { return (size_t)16 * channels * 4; }  // one producer's 16-token tile
};

S8xShape S8xShapeFor(int64_t batch, int64_t M, int64_t K, int64_t N) {
  S8xShape none = {0, 0, 0, 0};
  if (GetOption("dequant_dot_x") == 1) return none;
  if (M < 1 || M > 16 || K < 256 || K % 256 != 0 || N % 8 != 0) return none;
  const int64_t units = K / 256;  // one step of every wave each
  const int64_t wide = (N + 127) / 128;
  int steps = 0;
  if (int v = GetOption("dequant_dot_steps")) {
    steps = v;
  } else {
    // Few slices beat many workgroups: every slice beyond the first costs the strip's last workgroup
    // a device-scope round trip more to wait for (measured on [16,4096]x[4096,4096]: 4 / 8 / 16 slices
    // 8.2 / 9.1 / 10.0 us; the same bytes with no slices at all 4.8 - 6.2 us).  So: the most steps
    // per wave that still leave 64 workgroups.
    for (int s : {4, 2, 1})
      if (units % s == 0 && (steps == 0 || wide * batch * (units / steps) < 64)) steps = s;
  }
  if ((steps != 1 && steps != 2 && steps != 4) || units % steps != 0) return none;
  S8xShape shape = {steps, 128, wide, units / steps};
  // strips of 64 channels where the wide ones would leave CUs without a workgroup: the same number
  // of slices to wait for, half the bytes per workgroup
  const int forced = GetOption("dequant_dot_strip");
  if (forced == 64 || (forced == 0 && shape.strips * batch * shape.slices < 256)) {
    shape.channels = 64;
    shape.strips = (N + 63) / 64;
  }
  if (shape.slices > 16 || shape.strips * batch * shape.slices > 1024) return none;
  return shape;
}

}  // namespace

size_t S8xWorkspaceBytes(int64_t batch, int64_t M, int64_t K, int64_t N) {
  const S8xShape shape = S8xShapeFor(batch, M, K, N);
  if (!shape.steps) return 0;
  const int64_t others = shape.slices - 1;
  // per strip: the producers' sums and flags, and one generation word
  return others > 0 ? (size_t)(batch * shape.strips) * ((size_t)others * (shape.sums_bytes() + 8) + 8) : 0;
}

int LaunchDequantDotDecodeS8x(DecodeParams dp, const XlaAmdDequantDot& p, hipStream_t stream) {
  if (p.weight_dtype != XLA_FFI_DataType_S8 || p.dequant_type == XLA_FFI_DataType_BF16 || p.group != p.K) return -1;
  const S8xShape shape = S8xShapeFor(p.batch, p.M, p.K, p.N);
  const int steps = shape.steps;
  if (!steps) return -1;
  if ((double)p.K * p.N >= 2147483648.0 || (double)p.M * p.K * 2 >= 2147483648.0) return -1;
  dp.strips = (int)shape.strips;
  dp.slices = (int)shape.slices;
  dp.rows_per_slice = 256 * steps;
  dp.flags = nullptr;
  dp.epoch = 0;
  dp.pairs_per_group = shape.channels == 64 && (dp.slices == 1 || dp.slices == 2 || dp.slices == 4) ? 8 / dp.slices : 0;
  if (dp.slices > 1) {
    const size_t need = S8xWorkspaceBytes(p.batch, p.M, p.K, p.N);
    if (!p.workspace || ((uintptr_t)p.workspace % 16) != 0 || p.workspace_bytes < need) return -1;
    const size_t sums = (size_t)p.batch * dp.strips * (dp.slices - 1) * shape.sums_bytes();
    dp.flags = (unsigned long long*)((char*)p.workspace + sums);
    dp.epoch = NextHandOverEpoch();
  }
  const int b = (int)p.batch;
  if (shape.channels == 64) {
    if (steps == 1) return launch_s8x<1, 4>(dp, b, stream, "dequant_dot_decode_s8x_m16_n64_s1");
    if (steps == 2) return launch_s8x<2, 4>(dp, b, stream, "dequant_dot_decode_s8x_m16_n64_s2");
    return launch_s8x<4, 4>(dp, b, stream, "dequant_dot_decode_s8x_m16_n64_s4");
  }
  if (steps == 1) return launch_s8x<1, 8>(dp, b, stream, "dequant_dot_decode_s8x_m16_s1");
  if (steps == 2) return launch_s8x<2, 8>(dp, b, stream, "dequant_dot_decode_s8x_m16_s2");
  return launch_s8x<4, 8>(dp, b, stream, "dequant_dot_decode_s8x_m16_s4");
}

}  // namespace xla_amd
