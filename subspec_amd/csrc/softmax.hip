// softmax(logits / temperature) over the vocabulary, in the logits dtype: the draft's probability
// rows that feed the top-k expansion.
//
// Replaces ClassicSDDraftModel.forward(with_softmax=True):
//   torch.softmax(logits / self.draft_params.temperature, dim=-1)
// (specdecodes/models/draft_models/classic_sd.py:10-16).  As there, the quotient is rounded to the
// tensor dtype first (an elementwise tensor op), the softmax is evaluated in fp32 on the rounded
// values (maximum, exp(x - max), sum, quotient) and each probability is rounded once.
//
// Many rows: one workgroup per row, three passes over the row (maximum, sum, write); a 152064-entry
// 16-bit row is 297 KB, so the second and third pass are served by L2.  A draft step has 1 to 16
// rows, far too few workgroups for the chip: then every row is cut into slices, one launch reduces
// each slice to (maximum, sum of exp relative to it) and a second one combines the slices of its row
// and writes its slice (the sums differ from the one-workgroup order only in fp32 rounding).
#include "common.h"
#include <algorithm>

namespace subspec {

constexpr int kSmThreads = 1024;

template <int DT>
__device__ __forceinline__ float scaled(const void* p, int64_t i, const Divisor& t) {
  return Elem<DT>::round(div_rn(Elem<DT>::load(p, i), t));   // IEEE quotient, then one rounding to the row dtype
}

template <int DT>
__global__ __launch_bounds__(kSmThreads) void softmax_temperature_kernel(const void* __restrict__ logits, void* __restrict__ out,
                                                                          int64_t vocab, Divisor temperature) {
  __shared__ float red[kSmThreads / kWave];
  const int64_t base = (int64_t)blockIdx.x * vocab;
  const int tid = threadIdx.x;
  float m = -INFINITY;
  for (int64_t i = tid; i < vocab; i += kSmThreads) m = fmaxf(m, scaled<DT>(logits, base + i, temperature));
  m = block_max<kSmThreads>(m, red);
  float s = 0.f;
  for (int64_t i = tid; i < vocab; i += kSmThreads) s += expf(scaled<DT>(logits, base + i, temperature) - m);
  s = block_sum<kSmThreads>(s, red);
  for (int64_t i = tid; i < vocab; i += kSmThreads)
    Elem<DT>::store(out, base + i, expf(scaled<DT>(logits, base + i, temperature) - m) / s);
}

// ---- few rows: slices of kSliceElems elements, grid (slices, rows)
constexpr int kSliceThreads = 256;
constexpr int kSliceElems = 4096;
constexpr int kMaxSlices = 1024;

template <int DT>
__global__ __launch_bounds__(kSliceThreads) void softmax_slice_stats_kernel(const void* __restrict__ logits, float2* __restrict__ stats,
                                                                            int64_t vocab, Divisor temperature) {
  __shared__ float red[kSliceThreads / kWave];
  const int64_t base = (int64_t)blockIdx.y * vocab;
  const int64_t i0 = (int64_t)blockIdx.x * kSliceElems, i1 = min(i0 + kSliceElems, vocab);
  float v[kSliceElems / kSliceThreads];
  float m = -INFINITY;
#pragma unroll
  for (int j = 0; j < kSliceElems / kSliceThreads; ++j) {
    const int64_t i = i0 + j * kSliceThreads + threadIdx.x;
    v[j] = i < i1 ? scaled<DT>(logits, base + i, temperature) : -INFINITY;
    m = fmaxf(m, v[j]);
  }
  m = block_max<kSliceThreads>(m, red);
  float s = 0.f;
  if (m != -INFINITY) {
#pragma unroll
    for (int j = 0; j < kSliceElems / kSliceThreads; ++j) s += expf(v[j] - m);
  }
  s = block_sum<kSliceThreads>(s, red);
  if (threadIdx.x == 0) stats[(int64_t)blockIdx.y * gridDim.x + blockIdx.x] = make_float2(m, s);
}

template <int DT>
__global__ __launch_bounds__(kSliceThreads) void softmax_slice_write_kernel(const void* __restrict__ logits, void* __restrict__ out,
                                                                            const float2* __restrict__ stats, int64_t vocab,
                                                                            Divisor temperature) {
  __shared__ float red[kSliceThreads / kWave];
  const int slices = gridDim.x;
  const float2* st = stats + (int64_t)blockIdx.y * slices;
  float m = -INFINITY;
  for (int c = threadIdx.x; c < slices; c += kSliceThreads) m = fmaxf(m, st[c].x);
  m = block_max<kSliceThreads>(m, red);
  float s = 0.f;
  for (int c = threadIdx.x; c < slices; c += kSliceThreads)
    if (st[c].x != -INFINITY) s += st[c].y * expf(st[c].x - m);
  s = block_sum<kSliceThreads>(s, red);
  const int64_t base = (int64_t)blockIdx.y * vocab;
  const int64_t i0 = (int64_t)blockIdx.x * kSliceElems, i1 = min(i0 + kSliceElems, vocab);
  for (int64_t i = i0 + threadIdx.x; i < i1; i += kSliceThreads)
    Elem<DT>::store(out, base + i, expf(scaled<DT>(logits, base + i, temperature) - m) / s);
}

// TemperatureLogitsWarper as a stand-alone elementwise pass: out = logits / temperature in the logits dtype
template <int DT>
__global__ __launch_bounds__(256) void temperature_warp_kernel(const void* __restrict__ logits, void* __restrict__ out,
                                                               int64_t n, Divisor temperature) {
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256)
    Elem<DT>::store(out, i, div_rn(Elem<DT>::load(logits, i), temperature));
}

}  // namespace subspec

using namespace subspec;

extern "C" int subspec_temperature_warp(const void* logits, void* out, int dtype, int64_t n, float temperature,
                                        void* stream) {
  if (!dtype_ok(dtype)) SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "temperature_warp: unknown dtype %d", dtype);
  if (!logits || !out) SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "temperature_warp: null pointer argument");
  if (n <= 0) SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "temperature_warp: n=%lld must be positive", (long long)n);
  if (!(temperature > 0.f) || temperature == INFINITY)
    SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "temperature_warp: temperature must be positive and finite");
  hipStream_t st = (hipStream_t)stream;
  const dim3 grid((unsigned)std::min<int64_t>((n + 255) / 256, 8192));
  const Divisor t = make_divisor(temperature);
  if (dtype == SUBSPEC_F32)
    hipLaunchKernelGGL((temperature_warp_kernel<SUBSPEC_F32>), grid, dim3(256), 0, st, logits, out, n, t);
  else if (dtype == SUBSPEC_F16)
    hipLaunchKernelGGL((temperature_warp_kernel<SUBSPEC_F16>), grid, dim3(256), 0, st, logits, out, n, t);
  else
    hipLaunchKernelGGL((temperature_warp_kernel<SUBSPEC_BF16>), grid, dim3(256), 0, st, logits, out, n, t);
  SUBSPEC_CHECK_HIP(hipGetLastError());
  return SUBSPEC_OK;
}

extern "C" size_t subspec_softmax_temperature_workspace(int64_t rows, int64_t vocab) {
  const int64_t slices = (vocab + kSliceElems - 1) / kSliceElems;
  if (rows <= 0 || rows >= 256 || slices <= 1 || slices > kMaxSlices) return 0;
  return align_up((size_t)rows * slices * sizeof(float2), 256);
}

extern "C" int subspec_softmax_temperature(const void* logits, void* out, int dtype, int64_t rows, int64_t vocab,
                                           float temperature, void* workspace, size_t workspace_bytes, void* stream) {
  if (!dtype_ok(dtype)) SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "softmax_temperature: unknown dtype %d", dtype);
  if (!logits || !out) SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "softmax_temperature: null pointer argument");
  if (rows <= 0 || vocab <= 0) SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "softmax_temperature: rows=%lld vocab=%lld", (long long)rows, (long long)vocab);
  if (!(temperature > 0.f)) SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "softmax_temperature: temperature must be positive");
  if (rows > 0x7fffffff) SUBSPEC_FAIL(SUBSPEC_ERR_LIMIT, "softmax_temperature: too many rows");
  hipStream_t st = (hipStream_t)stream;
  const dim3 grid((unsigned)rows);
  const Divisor t = make_divisor(temperature);
  const int64_t slices = (vocab + kSliceElems - 1) / kSliceElems;
  if (workspace && rows < 256 && slices > 1 && slices <= kMaxSlices) {
    if (workspace_bytes < subspec_softmax_temperature_workspace(rows, vocab))
      SUBSPEC_FAIL(SUBSPEC_ERR_WORKSPACE, "softmax_temperature: workspace of %zu bytes is smaller than the %zu required",
                   workspace_bytes, subspec_softmax_temperature_workspace(rows, vocab));
    if ((uintptr_t)workspace % 8 != 0) SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "softmax_temperature: workspace must be 8-byte aligned");
    const dim3 g2((unsigned)slices, (unsigned)rows);
    float2* stats = (float2*)workspace;
#define SUBSPEC_SM_SLICED(DT)                                                                                        \
    hipLaunchKernelGGL((softmax_slice_stats_kernel<DT>), g2, dim3(kSliceThreads), 0, st, logits, stats, vocab, t);     \
    hipLaunchKernelGGL((softmax_slice_write_kernel<DT>), g2, dim3(kSliceThreads), 0, st, logits, out, stats, vocab, t)
    if (dtype == SUBSPEC_F32) { SUBSPEC_SM_SLICED(SUBSPEC_F32); }
    else if (dtype == SUBSPEC_F16) { SUBSPEC_SM_SLICED(SUBSPEC_F16); }
    else { SUBSPEC_SM_SLICED(SUBSPEC_BF16); }
#undef SUBSPEC_SM_SLICED
    SUBSPEC_CHECK_HIP(hipGetLastError());
    return SUBSPEC_OK;
  }
  if (dtype == SUBSPEC_F32)
    hipLaunchKernelGGL((softmax_temperature_kernel<SUBSPEC_F32>), grid, dim3(kSmThreads), 0, st, logits, out, vocab, t);
  else if (dtype == SUBSPEC_F16)
    hipLaunchKernelGGL((softmax_temperature_kernel<SUBSPEC_F16>), grid, dim3(kSmThreads), 0, st, logits, out, vocab, t);
  else
    hipLaunchKernelGGL((softmax_temperature_kernel<SUBSPEC_BF16>), grid, dim3(kSmThreads), 0, st, logits, out, vocab, t);
  SUBSPEC_CHECK_HIP(hipGetLastError());
  return SUBSPEC_OK;
}
