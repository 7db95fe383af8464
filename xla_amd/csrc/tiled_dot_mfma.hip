// LDS-tiled MFMA dots for prefill shapes.
//
//   kFp8 : out[m,n] = epi( a_scale*b_scale * sum_k A8[m,k] * B8[n,k] )   f8e4m3fn x f8e4m3fn
//   kS8  : out[b,m,n] = epi( scale[b,n] * sum_k A[b,m,k] * W[b,k,n] )    bf16 x s8 (per channel)
//
// A workgroup of 4 waves owns a 128x128 output tile and walks K in stages of
// 128 bytes of the activation row (128 fp8 or 64 bf16 values).  Both operand
// tiles of a stage sit in LDS with the contracting dimension contiguous, so a
// lane fetches its MFMA fragment with 128-bit reads; the next stage's global
// loads are issued before the current stage's MFMAs and written to the other
// LDS buffer afterwards.  The s8 weights are [K,N] with N minor: a lane reads
// 4 channels of 8 consecutive rows, converts (exactly) to bf16 and writes each
// channel's 8 values as one 16-byte LDS row piece -- the transposition costs
// nothing beyond the convert.
//
// The MFMA's 16-row operand is fed with *output channels* and the 16-column
// operand with tokens, so a lane ends up with 4 consecutive channels of one
// token and stores them as one 8-byte piece of the bf16 output row.
//
// Bound: MFMA (fp8: v_mfma_f32_16x16x128_f8f6f4, bf16: v_mfma_f32_16x16x32_bf16).
// Algorithmic flops: 2*M*N*K per batch.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "device_numerics.h"
#include "launch.h"

namespace xla_amd {
namespace {

enum : int { kFp8 = 0, kS8 = 1 };

constexpr int kTM = 128, kTN = 128;  // output tile (tokens x channels)
constexpr int kStageBytes = 128;     // bytes of K per LDS row per stage
constexpr int kPitch = kStageBytes + 16;  // padded LDS row pitch: 128-bit reads stay conflict-free

struct TiledParams {
  const uint8_t* a;     // kFp8: f8 [M,K]; kS8: bf16 [batch,M,K]
  const uint8_t* b;     // kFp8: f8 [N,K]; kS8: s8 [batch,K,N]
  const float* a_scale; // kFp8 device scalars
  const float* b_scale;
  const void* scales;   // kS8: [scale_batch, N]
  const void* bias;
  uint16_t* out;        // [batch, M, N]
  int M, K, N;
  int scale_is_bf16, bias_is_bf16, scale_batched;
  int bf16_dot, bf16_ops, epilogue;
  int tiles_m, tiles_n;
  int require_pow2_scales;  // kFp8 with a bf16-typed dequantise multiply: exact only then
};

__device__ __forceinline__ bool is_pow2_f32(float s) {
  const uint32_t u = f32_to_bits(s);
  const uint32_t e = (u >> 23) & 0xffu;
  // normal power of two whose product with any finite f8 value stays a normal bf16
  return (u & 0x807fffffu) == 0u && e > 24u && e < 230u;
}

template <int KIND>
__global__ __launch_bounds__(256) void tiled_dot_kernel(TiledParams p) {
  constexpr int ESZ = KIND == kFp8 ? 1 : 2;      // bytes per A element
  constexpr int KS = kStageBytes / ESZ;          // K elements per stage
  __shared__ __attribute__((aligned(16))) uint8_t lds_a[2][kTM * kPitch];
  __shared__ __attribute__((aligned(16))) uint8_t lds_b[2][kTN * kPitch];

  if (KIND == kFp8 && p.require_pow2_scales) {
    if (!(is_pow2_f32(*p.a_scale) && is_pow2_f32(*p.b_scale))) return;  // the exact kernel runs
  }

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int li = lane & 15, kb = lane >> 4;
  const int wm = wave >> 1, wn = wave & 1;

  int bid = blockIdx.x;
  {
    const int total = gridDim.x;
    if (total % 8 == 0) bid = (bid % 8) * (total / 8) + bid / 8;  // one XCD: a contiguous run
  }
  const int tm = bid % p.tiles_m, tn = bid / p.tiles_m;
  const int batch = blockIdx.y;
  const int m0 = tm * kTM, n0 = tn * kTN;

  const uint8_t* A = p.a + (size_t)batch * p.M * p.K * ESZ;
  const uint8_t* B = p.b + (size_t)batch * p.K * p.N;  // kS8 only uses the batch offset

  floatx4 acc[4][4];
#pragma unroll
  for (int x = 0; x < 4; ++x)
#pragma unroll
    for (int y = 0; y < 4; ++y) acc[x][y] = floatx4{0.f, 0.f, 0.f, 0.f};

  uintx4 ga[4];
  uintx4 gb[4];      // kFp8: 4 chunks of the B tile; kS8: 8 dwords = rows of 4 channels
  auto gload = [&](int k0) {
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int c = tid + 256 * q, row = c >> 3, col = (c & 7) * 16;  // 8 chunks of 16 B per row
      const int m = m0 + row;
      const int kbyte = k0 * ESZ + col;
      ga[q] = uintx4{0u, 0u, 0u, 0u};
      if (m < p.M && kbyte < p.K * ESZ)
        ga[q] = *reinterpret_cast<const uintx4*>(A + (size_t)m * p.K * ESZ + kbyte);
      if (KIND == kFp8) {
        const int n = n0 + row;
        gb[q] = uintx4{0u, 0u, 0u, 0u};
        if (n < p.N && kbyte < p.K) gb[q] = *reinterpret_cast<const uintx4*>(p.b + (size_t)n * p.K + kbyte);
      }
    }
    if (KIND == kS8) {
      const int kblk = tid >> 5, nq = tid & 31;  // 8 row blocks x 32 channel quads
      const int n = n0 + nq * 4;
#pragma unroll
      for (int r = 0; r < 8; ++r) {
        const int k = k0 + kblk * 8 + r;
        uint32_t v = 0u;
        if (k < p.K && n < p.N) v = *reinterpret_cast<const uint32_t*>(B + (size_t)k * p.N + n);
        gb[r >> 2][r & 3] = v;
      }
    }
  };
  auto lstore = [&](int buf) {
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int c = tid + 256 * q, row = c >> 3, col = (c & 7) * 16;
      *reinterpret_cast<uintx4*>(&lds_a[buf][row * kPitch + col]) = ga[q];
      if (KIND == kFp8) *reinterpret_cast<uintx4*>(&lds_b[buf][row * kPitch + col]) = gb[q];
    }
    if (KIND == kS8) {
      const int kblk = tid >> 5, nq = tid & 31;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        float f[8];
#pragma unroll
        for (int r = 0; r < 8; ++r) f[r] = (float)(int8_t)((gb[r >> 2][r & 3] >> (8 * e)) & 0xffu);
        uintx4 v = {pack_bf16x2(f[0], f[1]), pack_bf16x2(f[2], f[3]), pack_bf16x2(f[4], f[5]),
                    pack_bf16x2(f[6], f[7])};
        *reinterpret_cast<uintx4*>(&lds_b[buf][(nq * 4 + e) * kPitch + kblk * 16]) = v;
      }
    }
  };

  const int stages = (p.K + KS - 1) / KS;
  gload(0);
  lstore(0);
  __syncthreads();
  for (int s = 0; s < stages; ++s) {
    const int buf = s & 1;
    if (s + 1 < stages) gload((s + 1) * KS);
    if (KIND == kFp8) {
      intx8 fa[4], fb[4];
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        const uint8_t* ra = &lds_a[buf][(wm * 64 + t * 16 + li) * kPitch + kb * 32];
        const uint8_t* rb = &lds_b[buf][(wn * 64 + t * 16 + li) * kPitch + kb * 32];
        uintx4 a0 = *reinterpret_cast<const uintx4*>(ra), a1 = *reinterpret_cast<const uintx4*>(ra + 16);
        uintx4 b0 = *reinterpret_cast<const uintx4*>(rb), b1 = *reinterpret_cast<const uintx4*>(rb + 16);
        fa[t] = intx8{(int)a0[0], (int)a0[1], (int)a0[2], (int)a0[3], (int)a1[0], (int)a1[1], (int)a1[2], (int)a1[3]};
        fb[t] = intx8{(int)b0[0], (int)b0[1], (int)b0[2], (int)b0[3], (int)b1[0], (int)b1[1], (int)b1[2], (int)b1[3]};
      }
#pragma unroll
      for (int nt = 0; nt < 4; ++nt)
#pragma unroll
        for (int mt = 0; mt < 4; ++mt)
          acc[nt][mt] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(fb[nt], fa[mt], acc[nt][mt],
                                                                         0, 0, 0, 0, 0, 0);
    } else {
#pragma unroll
      for (int ks = 0; ks < 2; ++ks) {
        bf16x8 fa[4], fb[4];
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          fa[t] = *reinterpret_cast<const bf16x8*>(
              &lds_a[buf][(wm * 64 + t * 16 + li) * kPitch + ks * 64 + kb * 16]);
          fb[t] = *reinterpret_cast<const bf16x8*>(
              &lds_b[buf][(wn * 64 + t * 16 + li) * kPitch + ks * 64 + kb * 16]);
        }
#pragma unroll
        for (int nt = 0; nt < 4; ++nt)
#pragma unroll
          for (int mt = 0; mt < 4; ++mt)
            acc[nt][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fb[nt], fa[mt], acc[nt][mt], 0, 0, 0);
      }
    }
    if (s + 1 < stages) lstore(buf ^ 1);
    __syncthreads();
  }

  // ---- epilogue: lane (li, kb), register t of tile (nt, mt):
  //      token m0 + wm*64 + mt*16 + li, channel n0 + wn*64 + nt*16 + 4*kb + t
  float alpha = 1.0f;
  if (KIND == kFp8) alpha = *p.a_scale * *p.b_scale;
#pragma unroll
  for (int mt = 0; mt < 4; ++mt) {
    const int m = m0 + wm * 64 + mt * 16 + li;
    if (m >= p.M) continue;
#pragma unroll
    for (int nt = 0; nt < 4; ++nt) {
      const int n = n0 + wn * 64 + nt * 16 + 4 * kb;
      if (n >= p.N) continue;
      float v[4];
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        float x = acc[nt][mt][t];
        if (KIND == kFp8) {
          x = x * alpha;
        } else {
          const size_t si = (size_t)(p.scale_batched ? batch : 0) * p.N + n + t;
          x = (n + t < p.N) ? x * (p.scale_is_bf16 ? bf16_to_f32(((const uint16_t*)p.scales)[si])
                                                   : ((const float*)p.scales)[si])
                            : 0.0f;
        }
        float bv = 0.0f;
        if (p.bias && n + t < p.N)
          bv = p.bias_is_bf16 ? bf16_to_f32(((const uint16_t*)p.bias)[n + t]) : ((const float*)p.bias)[n + t];
        v[t] = epilogue_dispatch(x, bv, p.epilogue, p.bf16_dot, p.bf16_ops);
      }
      uint16_t* dst = p.out + ((size_t)batch * p.M + m) * p.N + n;
      if (n + 3 < p.N && (p.N & 3) == 0) {
        uintx2 o = {pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3])};
        *reinterpret_cast<uintx2*>(dst) = o;
      } else {
#pragma unroll
        for (int t = 0; t < 4; ++t)
          if (n + t < p.N) dst[t] = f32_to_bf16(v[t]);
      }
    }
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

// Exact, slow f8 scaled dot for scales that are not powers of two under a bf16-typed
// dequantise multiply: each operand value is rounded to bf16 after its scale, as the HLO does.
__global__ __launch_bounds__(256) void fp8_dot_exact_kernel(TiledParams p, int b_is_nk, int deq_bf16,
                                                            int only_if_not_pow2) {
  if (only_if_not_pow2 && is_pow2_f32(*p.a_scale) && is_pow2_f32(*p.b_scale)) return;
  const size_t total = (size_t)p.M * p.N;
  const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= total) return;
  const int n = (int)(idx % p.N), m = (int)(idx / p.N);
  float sa = *p.a_scale, sb = *p.b_scale;
  if (deq_bf16) { sa = round_bf16(sa); sb = round_bf16(sb); }
  float acc = 0.0f;
  for (int k = 0; k < p.K; ++k) {
    float av = f8e4m3fn_to_f32(p.a[(size_t)m * p.K + k]) * sa;
    float bv = f8e4m3fn_to_f32(b_is_nk ? p.b[(size_t)n * p.K + k] : p.b[(size_t)k * p.N + n]) * sb;
    if (deq_bf16) { av = round_bf16(av); bv = round_bf16(bv); }
    acc = acc + av * bv;
  }
  float bias = 0.0f;
  if (p.bias) bias = p.bias_is_bf16 ? bf16_to_f32(((const uint16_t*)p.bias)[n]) : ((const float*)p.bias)[n];
  p.out[idx] = f32_to_bf16(epilogue_dispatch(acc, bias, p.epilogue, p.bf16_dot, p.bf16_ops));
}

}  // namespace

// bf16 x s8 per-channel prefill.  Returns -1 when the tiled kernel does not cover the shape
// (the caller then falls back), 0 on success, or an error code.
int LaunchDequantDotPrefill(const XlaAmdDequantDot& p, hipStream_t stream) {
  if (p.weight_dtype != XLA_FFI_DataType_S8 || p.group != p.K ||
      p.dequant_type != XLA_FFI_DataType_F32)
    return -1;
  if (p.K % 8 != 0 || p.N % 4 != 0 || ((uintptr_t)p.lhs % 16) || ((uintptr_t)p.weights % 4)) return -1;
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
  dim3 grid((unsigned)(tp.tiles_m * tp.tiles_n), (unsigned)p.batch);
  hipLaunchKernelGGL(tiled_dot_kernel<kS8>, grid, dim3(256), 0, stream, tp);
  SetLastKernel("dequant_dot_tiled_s8_factored");
  return CheckLaunch("dequant_dot_tiled_s8");
}

size_t Fp8ScaledDotWorkspaceBytes(int64_t K, int64_t N, int rhs_contracting_dim) {
  return rhs_contracting_dim == 0 ? (size_t)K * N : 0;
}

int LaunchFp8ScaledDot(const XlaAmdFp8ScaledDot& p, hipStream_t stream) {
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
  if (p.M == 0 || p.N == 0) {
    SetLastKernel("fp8_scaled_dot:empty");
    return 0;
  }
  if (!p.a || !p.b || !p.a_scale || !p.b_scale || !p.out)
    return Fail(XLA_FFI_Error_Code_INVALID_ARGUMENT, "fp8_scaled_dot: null buffer");

  TiledParams tp{};
  tp.a = (const uint8_t*)p.a;
  tp.b = (const uint8_t*)p.b;
  tp.a_scale = p.a_scale;
  tp.b_scale = p.b_scale;
  tp.bias = (p.epilogue & 1) ? p.bias : nullptr;
  tp.out = (uint16_t*)p.out;
  tp.M = (int)p.M; tp.K = (int)p.K; tp.N = (int)p.N;
  tp.bias_is_bf16 = p.bias_dtype == XLA_FFI_DataType_BF16;
  tp.bf16_dot = p.dot_type == XLA_FFI_DataType_BF16;
  tp.bf16_ops = p.epilogue_type == XLA_FFI_DataType_BF16;
  tp.epilogue = p.epilogue;
  tp.tiles_m = (tp.M + kTM - 1) / kTM;
  tp.tiles_n = (tp.N + kTN - 1) / kTN;
  const bool deq_bf16 = p.dequant_type == XLA_FFI_DataType_BF16;
  tp.require_pow2_scales = deq_bf16;

  const int force = GetOption("fp8_dot_kernel");  // 0 auto, 1 exact (slow), 2 tiled
  const bool nk = p.rhs_contracting_dim == 1;
  bool tiled_ok = p.K % 16 == 0 && p.K > 0 && ((uintptr_t)p.a % 16 == 0) && force != 1;
  const uint8_t* b_nk = (const uint8_t*)p.b;
  if (tiled_ok && !nk) {
    if (p.workspace && p.workspace_bytes >= (size_t)p.K * p.N && ((uintptr_t)p.workspace % 16 == 0)) {
      dim3 tgrid((unsigned)((p.N + 63) / 64), (unsigned)((p.K + 63) / 64));
      hipLaunchKernelGGL(transpose_bytes_kernel, tgrid, dim3(256), 0, stream, (const uint8_t*)p.b,
                         (uint8_t*)p.workspace, (int)p.K, (int)p.N);
      int rc = CheckLaunch("fp8_scaled_dot_transpose");
      if (rc) return rc;
      b_nk = (const uint8_t*)p.workspace;
    } else {
      tiled_ok = false;
    }
  }
  if (tiled_ok && ((uintptr_t)b_nk % 16 != 0)) tiled_ok = false;
  if (force == 2 && !tiled_ok)
    return Fail(XLA_FFI_Error_Code_FAILED_PRECONDITION,
                "fp8_scaled_dot: the tiled kernel needs K %% 16 == 0, 16-byte aligned operands and, "
                "for a [K,N] rhs, a workspace of K*N bytes");
  if (p.K == 0) tiled_ok = false;

  dim3 egrid((unsigned)(((size_t)p.M * p.N + 255) / 256));
  if (tiled_ok) {
    TiledParams tt = tp;
    tt.b = b_nk;
    dim3 grid((unsigned)(tt.tiles_m * tt.tiles_n), 1);
    hipLaunchKernelGGL(tiled_dot_kernel<kFp8>, grid, dim3(256), 0, stream, tt);
    int rc = CheckLaunch("fp8_scaled_dot_tiled");
    if (rc) return rc;
    if (deq_bf16) {
      // runs only if a scale is not a power of two (decided on the device, no host read)
      hipLaunchKernelGGL(fp8_dot_exact_kernel, egrid, dim3(256), 0, stream, tp, nk ? 1 : 0, 1, 1);
      rc = CheckLaunch("fp8_scaled_dot_exact");
      if (rc) return rc;
    }
    SetLastKernel(nk ? "fp8_scaled_dot_tiled" : "fp8_scaled_dot_tiled+transpose");
    return 0;
  }
  hipLaunchKernelGGL(fp8_dot_exact_kernel, egrid, dim3(256), 0, stream, tp, nk ? 1 : 0, deq_bf16 ? 1 : 0, 0);
  SetLastKernel("fp8_scaled_dot_exact");
  return CheckLaunch("fp8_scaled_dot_exact");
}

}  // namespace xla_amd
