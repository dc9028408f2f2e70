// HQQ-style int4 (group 64, per-row-group fp16 scale / zero) linear layers for gfx950:
//   y[M, N] = x[M, K] * ((Wq - zero) * scale)^T (+ bias)
//
// Replaces the draft's quantized projections: HQQLinear on the GemLite A16W4 backend, set up by
// HqqQuantizer.quantize_model (specdecodes/helpers/quantizers/hqq/__init__.py:17-120) for the
// BaseQuantizeConfig(nbits=4, group_size=64, axis=1) of
// specdecodes/helpers/recipes/subspec/hqq_4bit_postspec.py:17-58.  The arithmetic of hqq / gemlite is
// not part of the reference tree; the contract here is the affine dequantization above.
//
// Weight layout (written once at quantization time so that every wavefront load is one
// contiguous 512-byte block):
//   wq  uint2 [N/16][K/64][4][16]   entry (c, r): the 16 codes of row 16*nt + r for
//                                   k = 64*g + 16*c .. +15; word j holds k = .. + 8*j .. +7 with
//                                   code(k = 8j + 2i) in bits 4i..4i+3 and code(8j + 2i + 1) in
//                                   bits 16+4i..16+4i+3, so (w >> 4i) & 0x000f000f is the pair
//                                   (k, k+1) in the two 16-bit halves
//   sz  half2 [N/16][K/64][16]      (scale, zero) of row 16*nt + r, group g
// A code q becomes the 16-bit float 128 + q (bf16) or 1024 + q (fp16) by OR-ing it into the
// mantissa of a magic constant; the offset is folded into the zero point, so dequantization costs
// one v_and_or_b32 per two weights and the products accumulate in fp32:
//   sum_k (q_k - z) s x_k = s * (sum_k (off + q_k) x_k - (z + off) * sum_k x_k)    per group.
// M = 1   : int4_gemv_kernel, v_dot2_f32 on (weight pair, activation pair); HBM-bound,
//           algorithmic bytes = N*K/2 + N*(K/64)*4 (+ activations).
// M = 2-64: int4_gemm_kernel, v_mfma_f32_16x16x16 with the weight tile as A operand; the 16 k of
//           one MFMA step all come from one quantization group, so the raw accumulator of a
//           group is scaled once.  Split-K partials are reduced in a fixed order.
#include "common.h"
#include <algorithm>

namespace subspec {

constexpr int kI4Threads = 256;
constexpr int kGroup = 64;

typedef short i4_v4s __attribute__((ext_vector_type(4)));
typedef _Float16 i4_v4h __attribute__((ext_vector_type(4)));
typedef float i4_v4f __attribute__((ext_vector_type(4)));
typedef __bf16 i4_v2bf __attribute__((ext_vector_type(2)));
typedef _Float16 i4_v2h __attribute__((ext_vector_type(2)));

template <int DT> struct I4 {
  static constexpr uint32_t kMagic = DT == SUBSPEC_BF16 ? 0x43004300u : 0x64006400u;
  static constexpr float kOffset = DT == SUBSPEC_BF16 ? 128.f : 1024.f;
  static __device__ __forceinline__ float dot2(uint32_t a, uint32_t b, float c) {
    if constexpr (DT == SUBSPEC_BF16)
      return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(i4_v2bf, a), __builtin_bit_cast(i4_v2bf, b), c, false);
    else
      return __builtin_amdgcn_fdot2(__builtin_bit_cast(i4_v2h, a), __builtin_bit_cast(i4_v2h, b), c, false);
  }
  static __device__ __forceinline__ i4_v4f mfma(uint2 a, uint2 b, i4_v4f c) {
    if constexpr (DT == SUBSPEC_BF16)
      return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(i4_v4s, a), __builtin_bit_cast(i4_v4s, b), c, 0, 0, 0);
    else
      return __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(i4_v4h, a), __builtin_bit_cast(i4_v4h, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ float to_float(uint32_t bits16) {
    return DT == SUBSPEC_BF16 ? bf16_bits_to_float(bits16) : f16_bits_to_float(bits16);
  }
};
__device__ __forceinline__ uint32_t code_pair(uint32_t w, int shift, uint32_t magic) {
  return ((w >> shift) & 0x000f000fu) | magic;
}

// ------------------------------------------------------------------ M = 1
template <int DT>
__global__ __launch_bounds__(kI4Threads) void int4_gemv_kernel(
    const uint16_t* __restrict__ x, const uint2* __restrict__ wq, const uint32_t* __restrict__ sz,
    const uint16_t* __restrict__ bias, uint16_t* __restrict__ y, int64_t N, int64_t K) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  uint16_t* xs = (uint16_t*)smem;                               // [K]
  float* xsum16 = (float*)(smem + K * 2);                       // [K / 16]
  float* red = xsum16 + K / 16;                                 // [4][16]
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r = lane & 15, c = lane >> 4;
  const int64_t nt = blockIdx.x;
  const int G = (int)(K / kGroup);

  for (int64_t i = tid; i < K / 8; i += kI4Threads) ((uint4*)xs)[i] = ((const uint4*)x)[i];
  __syncthreads();
  for (int64_t sgm = tid; sgm < K / 16; sgm += kI4Threads) {
    float a = 0.f;
#pragma unroll
    for (int e = 0; e < 16; ++e) a += I4<DT>::to_float(xs[sgm * 16 + e]);
    xsum16[sgm] = a;
  }
  __syncthreads();

  float acc = 0.f;
  const uint2* wrow = wq + nt * G * 64 + lane;
  const uint32_t* szrow = sz + nt * G * 16 + r;
  constexpr int U = 4;
  for (int g0 = wave * U; g0 < G; g0 += 4 * U) {
    uint2 wv[U];
    uint32_t szv[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int g = min(g0 + u, G - 1);
      wv[u] = wrow[(int64_t)g * 64];
      szv[u] = szrow[(int64_t)g * 16];
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int g = g0 + u;
      if (g < G) {
        const uint4* xp = (const uint4*)(xs + g * kGroup + c * 16);
        const uint4 xa = xp[0], xb = xp[1];
        float raw = 0.f;
        raw = I4<DT>::dot2(code_pair(wv[u].x, 0, I4<DT>::kMagic), xa.x, raw);
        raw = I4<DT>::dot2(code_pair(wv[u].x, 4, I4<DT>::kMagic), xa.y, raw);
        raw = I4<DT>::dot2(code_pair(wv[u].x, 8, I4<DT>::kMagic), xa.z, raw);
        raw = I4<DT>::dot2(code_pair(wv[u].x, 12, I4<DT>::kMagic), xa.w, raw);
        raw = I4<DT>::dot2(code_pair(wv[u].y, 0, I4<DT>::kMagic), xb.x, raw);
        raw = I4<DT>::dot2(code_pair(wv[u].y, 4, I4<DT>::kMagic), xb.y, raw);
        raw = I4<DT>::dot2(code_pair(wv[u].y, 8, I4<DT>::kMagic), xb.z, raw);
        raw = I4<DT>::dot2(code_pair(wv[u].y, 12, I4<DT>::kMagic), xb.w, raw);
        const float s = f16_bits_to_float(szv[u] & 0xffffu), z = f16_bits_to_float(szv[u] >> 16);
        acc = fmaf(s, raw - (z + I4<DT>::kOffset) * xsum16[g * 4 + c], acc);
      }
    }
  }
  acc += __shfl_xor(acc, 16, kWave);
  acc += __shfl_xor(acc, 32, kWave);
  if (c == 0) red[wave * 16 + r] = acc;
  __syncthreads();
  if (tid < 16) {
    float v = red[tid] + red[16 + tid] + red[32 + tid] + red[48 + tid];
    const int64_t n = nt * 16 + tid;
    if (bias) v += I4<DT>::to_float(bias[n]);
    Elem<DT>::store(y, n, v);
  }
}

// ------------------------------------------------------------------ per-group activation sums
template <int DT>
__global__ __launch_bounds__(256) void group_sum_kernel(const uint16_t* __restrict__ x, float* __restrict__ xsum,
                                                        int64_t K) {
  const int64_t m = blockIdx.x;
  const int G = (int)(K / kGroup);
  for (int g = threadIdx.x; g < G; g += 256) {
    const uint16_t* p = x + m * K + (int64_t)g * kGroup;
    float a = 0.f;
    for (int e = 0; e < kGroup; ++e) a += I4<DT>::to_float(p[e]);
    xsum[m * G + g] = a;
  }
}

// ------------------------------------------------------------------ 2 <= M <= 64
constexpr int kXStride = kGroup + 8;        // LDS row stride (elements) of one group's activations

template <int DT, int MT>
__global__ __launch_bounds__(kI4Threads) void int4_gemm_kernel(
    const uint16_t* __restrict__ x, const float* __restrict__ xsum, const uint2* __restrict__ wq,
    const uint32_t* __restrict__ sz, const uint16_t* __restrict__ bias, uint16_t* __restrict__ y,
    float* __restrict__ partial, int64_t M, int64_t N, int64_t K, int splits, int groups_per_split) {
  constexpr int GB = 4;                                         // groups staged per barrier
  __shared__ __attribute__((aligned(16))) uint16_t xt[GB][MT * 16 * kXStride];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int lm = lane & 15, c = lane >> 4;
  const int G = (int)(K / kGroup);
  const int64_t nt = (int64_t)blockIdx.x * 4 + wave;
  const bool tile_ok = nt * 16 < N;
  const int ks = blockIdx.y;
  const int g_begin = ks * groups_per_split, g_end = min(G, g_begin + groups_per_split);

  i4_v4f acc[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) acc[mt] = i4_v4f{0.f, 0.f, 0.f, 0.f};
  const uint2* wrow = wq + (tile_ok ? nt : 0) * G * 64 + lane;
  const uint32_t* szrow = sz + (tile_ok ? nt : 0) * G * 16 + c * 4;

  for (int g0 = g_begin; g0 < g_end; g0 += GB) {
    __syncthreads();
    // stage the activations of GB groups: rows m < M (zero beyond), 64 k each
    for (int i = tid; i < GB * MT * 16 * 8; i += kI4Threads) {
      const int gi = i / (MT * 16 * 8), rem = i % (MT * 16 * 8);
      const int m = rem / 8, part = rem % 8;
      uint4 v = make_uint4(0, 0, 0, 0);
      if (m < M && g0 + gi < g_end) v = *(const uint4*)(x + (int64_t)m * K + (int64_t)(g0 + gi) * kGroup + part * 8);
      *(uint4*)(&xt[gi][m * kXStride + part * 8]) = v;
    }
    uint2 wv[GB];
    uint4 szv[GB];
#pragma unroll
    for (int gi = 0; gi < GB; ++gi) {
      const int g = min(g0 + gi, g_end - 1);
      wv[gi] = wrow[(int64_t)g * 64];
      szv[gi] = *(const uint4*)(szrow + (int64_t)g * 16);
    }
    __syncthreads();
#pragma unroll
    for (int gi = 0; gi < GB; ++gi) {
      const int g = g0 + gi;
      if (g >= g_end) break;
      uint2 a[4];
      a[0] = make_uint2(code_pair(wv[gi].x, 0, I4<DT>::kMagic), code_pair(wv[gi].x, 4, I4<DT>::kMagic));
      a[1] = make_uint2(code_pair(wv[gi].x, 8, I4<DT>::kMagic), code_pair(wv[gi].x, 12, I4<DT>::kMagic));
      a[2] = make_uint2(code_pair(wv[gi].y, 0, I4<DT>::kMagic), code_pair(wv[gi].y, 4, I4<DT>::kMagic));
      a[3] = make_uint2(code_pair(wv[gi].y, 8, I4<DT>::kMagic), code_pair(wv[gi].y, 12, I4<DT>::kMagic));
      const uint32_t szw[4] = {szv[gi].x, szv[gi].y, szv[gi].z, szv[gi].w};
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        i4_v4f raw = i4_v4f{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < 4; ++s) {
          const uint2 b = *(const uint2*)(&xt[gi][(mt * 16 + lm) * kXStride + c * 16 + s * 4]);
          raw = I4<DT>::mfma(a[s], b, raw);
        }
        const int m = mt * 16 + lm;
        const float xs = m < M ? xsum[(int64_t)m * G + g] : 0.f;
#pragma unroll
        for (int rr = 0; rr < 4; ++rr) {
          const float s = f16_bits_to_float(szw[rr] & 0xffffu), z = f16_bits_to_float(szw[rr] >> 16);
          acc[mt][rr] = fmaf(s, raw[rr] - (z + I4<DT>::kOffset) * xs, acc[mt][rr]);
        }
      }
    }
  }
  if (!tile_ok) return;
  // accumulator layout: rows n = 16*nt + 4*c + rr, column m = 16*mt + lm
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int m = mt * 16 + lm;
    if (m >= M) continue;
    const int64_t n0 = nt * 16 + c * 4;
    if (splits == 1) {
      float v[4];
#pragma unroll
      for (int rr = 0; rr < 4; ++rr) v[rr] = acc[mt][rr] + (bias ? I4<DT>::to_float(bias[n0 + rr]) : 0.f);
#pragma unroll
      for (int rr = 0; rr < 4; ++rr) Elem<DT>::store(y, (int64_t)m * N + n0 + rr, v[rr]);
    } else {
      *(i4_v4f*)(partial + ((int64_t)ks * M + m) * N + n0) = acc[mt];
    }
  }
}

template <int DT>
__global__ __launch_bounds__(256) void int4_reduce_kernel(const float* __restrict__ partial,
                                                          const uint16_t* __restrict__ bias, uint16_t* __restrict__ y,
                                                          int64_t M, int64_t N, int splits) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= M * N) return;
  float v = 0.f;
  for (int s = 0; s < splits; ++s) v += partial[(int64_t)s * M * N + i];
  if (bias) v += I4<DT>::to_float(bias[i % N]);
  Elem<DT>::store(y, i, v);
}

struct I4Plan { int splits, groups_per_split; };

static I4Plan i4_plan(int64_t M, int64_t N, int64_t K) {
  (void)M;
  const int G = (int)(K / kGroup);
  const int64_t wgs = (N + 63) / 64;
  int splits = (int)std::max<int64_t>(1, (384 + wgs - 1) / wgs);
  splits = std::min(splits, std::max(1, G / 8));              // at least 8 groups (512 k) per split
  splits = std::min(splits, 32);
  int gps = (G + splits - 1) / splits;
  gps = (gps + 3) / 4 * 4;
  splits = (G + gps - 1) / gps;
  return I4Plan{splits, gps};
}

template <int DT>
static int run_int4(const void* x, const uint32_t* wq, const uint32_t* sz, const void* bias, void* y, int64_t M,
                    int64_t N, int64_t K, void* workspace, hipStream_t st) {
  if (M == 1) {
    const size_t smem = (size_t)K * 2 + (size_t)(K / 16) * 4 + 64 * 4;
    DominantKernelTimer timer(st);
    hipLaunchKernelGGL((int4_gemv_kernel<DT>), dim3((unsigned)(N / 16)), dim3(kI4Threads), smem, st, (const uint16_t*)x,
                       (const uint2*)wq, sz, (const uint16_t*)bias, (uint16_t*)y, N, K);
  } else {
    const I4Plan pl = i4_plan(M, N, K);
    float* xsum = (float*)workspace;
    float* partial = (float*)((char*)workspace + align_up((size_t)M * (K / kGroup) * sizeof(float), 256));
    hipLaunchKernelGGL((group_sum_kernel<DT>), dim3((unsigned)M), dim3(256), 0, st, (const uint16_t*)x, xsum, K);
    const dim3 grid((unsigned)((N + 63) / 64), (unsigned)pl.splits);
#define SUBSPEC_I4_LAUNCH(MT)                                                                                      \
  hipLaunchKernelGGL((int4_gemm_kernel<DT, MT>), grid, dim3(kI4Threads), 0, st, (const uint16_t*)x, xsum,           \
                     (const uint2*)wq, sz, (const uint16_t*)bias, (uint16_t*)y, partial, M, N, K, pl.splits,        \
                     pl.groups_per_split)
    {
      DominantKernelTimer timer(st);
      if (M <= 16) SUBSPEC_I4_LAUNCH(1);
      else if (M <= 32) SUBSPEC_I4_LAUNCH(2);
      else SUBSPEC_I4_LAUNCH(4);
    }
#undef SUBSPEC_I4_LAUNCH
    if (pl.splits > 1)
      hipLaunchKernelGGL((int4_reduce_kernel<DT>), dim3((unsigned)((M * N + 255) / 256)), dim3(256), 0, st, partial,
                         (const uint16_t*)bias, (uint16_t*)y, M, N, pl.splits);
  }
  SUBSPEC_CHECK_HIP(hipGetLastError());
  return SUBSPEC_OK;
}

}  // namespace subspec

using namespace subspec;

extern "C" size_t subspec_int4_linear_workspace(int64_t M, int64_t N, int64_t K) {
  if (M <= 1 || N <= 0 || K <= 0) return 256;
  const I4Plan pl = i4_plan(M, N, K);
  return align_up((size_t)M * (K / kGroup) * sizeof(float), 256) +
         (pl.splits > 1 ? align_up((size_t)pl.splits * M * N * sizeof(float), 256) : 0) + 256;
}

extern "C" int subspec_int4_linear(const void* x, const uint32_t* wq, const uint32_t* sz, const void* bias, void* y,
                                   int dtype, int64_t M, int64_t N, int64_t K, int64_t group_size, void* workspace,
                                   size_t workspace_bytes, void* stream) {
  if (dtype != SUBSPEC_BF16 && dtype != SUBSPEC_F16)
    SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "int4_linear: dtype %d not supported (bf16 / fp16 activations only)", dtype);
  if (!x || !wq || !sz || !y) SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "int4_linear: null pointer argument");
  if (group_size != kGroup) SUBSPEC_FAIL(SUBSPEC_ERR_LIMIT, "int4_linear: group_size=%lld (built for 64)", (long long)group_size);
  if (M <= 0 || N <= 0 || K <= 0 || N % 16 != 0 || K % kGroup != 0)
    SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "int4_linear: M=%lld N=%lld K=%lld; N must be a multiple of 16 and K of 64",
                 (long long)M, (long long)N, (long long)K);
  if (M > 64) SUBSPEC_FAIL(SUBSPEC_ERR_LIMIT, "int4_linear: M=%lld exceeds the 64-row limit (tree width)", (long long)M);
  if (K > 65536) SUBSPEC_FAIL(SUBSPEC_ERR_LIMIT, "int4_linear: K=%lld too large", (long long)K);
  if ((uintptr_t)x % 16 || (uintptr_t)wq % 16 || (uintptr_t)sz % 16 || (uintptr_t)y % 8)
    SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "int4_linear: x / wq / sz must be 16-byte aligned, y 8-byte aligned");
  if (M > 1) {
    const size_t need = subspec_int4_linear_workspace(M, N, K);
    if (!workspace || workspace_bytes < need)
      SUBSPEC_FAIL(SUBSPEC_ERR_WORKSPACE, "int4_linear: workspace of %zu bytes is smaller than the %zu required",
                   workspace_bytes, need);
    if ((uintptr_t)workspace % 16) SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "int4_linear: workspace must be 16-byte aligned");
  }
  if (dtype == SUBSPEC_BF16) return run_int4<SUBSPEC_BF16>(x, wq, sz, bias, y, M, N, K, workspace, (hipStream_t)stream);
  return run_int4<SUBSPEC_F16>(x, wq, sz, bias, y, M, N, K, workspace, (hipStream_t)stream);
}
