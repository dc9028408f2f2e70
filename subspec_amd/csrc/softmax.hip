// softmax(logits / temperature) over the vocabulary, in the logits dtype: the draft's probability
// rows that feed the top-k expansion.
//
// Replaces ClassicSDDraftModel.forward(with_softmax=True):
//   torch.softmax(logits / self.draft_params.temperature, dim=-1)
// (specdecodes/models/draft_models/classic_sd.py:10-16).  As there, the quotient is rounded to the
// tensor dtype first (an elementwise tensor op), the softmax is evaluated in fp32 on the rounded
// values (maximum, exp(x - max), sum, quotient) and each probability is rounded once.
//
// One workgroup per row, three passes over the row (maximum, sum, write); a 152064-entry 16-bit row
// is 297 KB, so the second and third pass are served by L2.  A draft step has 1 to 16 rows: the
// kernel is latency-bound and replaces two library launches by one.
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

extern "C" int subspec_softmax_temperature(const void* logits, void* out, int dtype, int64_t rows, int64_t vocab,
                                           float temperature, void* stream) {
  if (!dtype_ok(dtype)) SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "softmax_temperature: unknown dtype %d", dtype);
  if (!logits || !out) SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "softmax_temperature: null pointer argument");
  if (rows <= 0 || vocab <= 0) SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "softmax_temperature: rows=%lld vocab=%lld", (long long)rows, (long long)vocab);
  if (!(temperature > 0.f)) SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "softmax_temperature: temperature must be positive");
  if (rows > 0x7fffffff) SUBSPEC_FAIL(SUBSPEC_ERR_LIMIT, "softmax_temperature: too many rows");
  hipStream_t st = (hipStream_t)stream;
  const dim3 grid((unsigned)rows);
  const Divisor t = make_divisor(temperature);
  if (dtype == SUBSPEC_F32)
    hipLaunchKernelGGL((softmax_temperature_kernel<SUBSPEC_F32>), grid, dim3(kSmThreads), 0, st, logits, out, vocab, t);
  else if (dtype == SUBSPEC_F16)
    hipLaunchKernelGGL((softmax_temperature_kernel<SUBSPEC_F16>), grid, dim3(kSmThreads), 0, st, logits, out, vocab, t);
  else
    hipLaunchKernelGGL((softmax_temperature_kernel<SUBSPEC_BF16>), grid, dim3(kSmThreads), 0, st, logits, out, vocab, t);
  SUBSPEC_CHECK_HIP(hipGetLastError());
  return SUBSPEC_OK;
}
