// Shared helpers for the gfx950 kernels of the speculative-decoding hot path.
// Wavefront size is 64 everywhere; nothing here is written for 32-wide execution.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>
#include <math.h>

#include "../../include/subspec_hip.h"

namespace subspec {

constexpr int kWave = 64;

// ---------------------------------------------------------------- error reporting (host)
void set_error(const char* fmt, ...);
#define SUBSPEC_FAIL(code, ...)            \
  do {                                     \
    ::subspec::set_error(__VA_ARGS__);     \
    return (code);                         \
  } while (0)
#define SUBSPEC_CHECK_HIP(expr)                                                              \
  do {                                                                                       \
    hipError_t e_ = (expr);                                                                  \
    if (e_ != hipSuccess) SUBSPEC_FAIL(SUBSPEC_ERR_HIP, "%s failed: %s", #expr, hipGetErrorString(e_)); \
  } while (0)

// ---------------------------------------------------------------- optional timing of the dominant kernel
// When enabled (subspec_profile_enable), every entry point brackets its dominant kernel with a
// pair of events on the launch stream; subspec_profile_last_ms() returns that kernel's duration.
struct DominantKernelTimer {
  explicit DominantKernelTimer(hipStream_t st);
  ~DominantKernelTimer();
  hipStream_t st_;
  bool on_;
};

inline size_t dtype_size(int dtype) { return dtype == SUBSPEC_F32 ? 4 : 2; }
inline bool dtype_ok(int dtype) { return dtype == SUBSPEC_F32 || dtype == SUBSPEC_F16 || dtype == SUBSPEC_BF16; }
inline size_t align_up(size_t x, size_t a) { return (x + a - 1) / a * a; }

// ---------------------------------------------------------------- element types
struct bf16_t { uint16_t bits; };
struct f16_t { uint16_t bits; };

__device__ __forceinline__ float bf16_bits_to_float(uint32_t b) { return __uint_as_float(b << 16); }
__device__ __forceinline__ float f16_bits_to_float(uint32_t b) {
  union { uint16_t u; _Float16 h; } c;
  c.u = (uint16_t)b;
  return (float)c.h;
}
// round-to-nearest-even to bfloat16, result widened back to float (v_cvt_pk_bf16_f32 on gfx950)
__device__ __forceinline__ float round_bf16(float x) { return (float)(__bf16)x; }
__device__ __forceinline__ float round_f16(float x) { return (float)(_Float16)x; }

template <int DT> struct Elem;
template <> struct Elem<SUBSPEC_F32> {
  using storage = float;
  static constexpr int kBytes = 4;
  static __device__ __forceinline__ float load(const void* p, int64_t i) { return ((const float*)p)[i]; }
  static __device__ __forceinline__ float round(float x) { return x; }
  static __device__ __forceinline__ void store(void* p, int64_t i, float v) { ((float*)p)[i] = v; }
  static __device__ __forceinline__ float min_normal() { return 1.17549435e-38f; }
};
template <> struct Elem<SUBSPEC_F16> {
  using storage = uint16_t;
  static constexpr int kBytes = 2;
  static __device__ __forceinline__ float load(const void* p, int64_t i) { return f16_bits_to_float(((const uint16_t*)p)[i]); }
  static __device__ __forceinline__ float round(float x) { return round_f16(x); }
  static __device__ __forceinline__ void store(void* p, int64_t i, float v) {
    union { uint16_t u; _Float16 h; } c;
    c.h = (_Float16)v;
    ((uint16_t*)p)[i] = c.u;
  }
  static __device__ __forceinline__ float min_normal() { return 6.103515625e-05f; }
};
template <> struct Elem<SUBSPEC_BF16> {
  using storage = uint16_t;
  static constexpr int kBytes = 2;
  static __device__ __forceinline__ float load(const void* p, int64_t i) { return bf16_bits_to_float(((const uint16_t*)p)[i]); }
  static __device__ __forceinline__ float round(float x) { return round_bf16(x); }
  static __device__ __forceinline__ void store(void* p, int64_t i, float v) {
    ((uint16_t*)p)[i] = (uint16_t)(__float_as_uint(round_bf16(v)) >> 16);
  }
  static __device__ __forceinline__ float min_normal() { return 1.17549435e-38f; }
};

// x / t correctly rounded (round to nearest even) from inv_t = RN(1 / t): q = RN(x * inv_t) lies within one
// ulp of the quotient, the residual r = x - t * q is exact in one fma, and RN(q + r * inv_t) is the
// correctly rounded quotient (P. Markstein, "Computation of elementary functions on the IBM RISC
// System/6000 processor", IBM J. Res. Dev. 34, 1990, theorem on division by a correctly rounded
// reciprocal).  Three instructions instead of the generic division sequence.  Infinite quotients
// are returned as they are (their residual is not a number).  The residual must be a normal
// number for the step to be exact: guaranteed for |x| >= 2^-100, i.e. for anything a logit can be.
struct Divisor { float t, inv_t; };
inline Divisor make_divisor(float t) { return Divisor{t, (float)(1.0 / (double)t)}; }
__device__ __forceinline__ float div_rn(float x, const Divisor& d) {
  const float q = x * d.inv_t;
  const float r = fmaf(-d.t, q, x);
  const float q1 = fmaf(r, d.inv_t, q);
  return fabsf(q) == INFINITY ? q : q1;
}

// Output element of a linear layer: v = accumulator (+ bias), optionally followed by a residual add with
// the rounding points of the separate tensor ops it replaces: out = round(round(v) + residual[i]).
// `residual` may be the output itself (in-place update of the residual stream): the element is read and
// written by the same thread.
template <int DT>
__device__ __forceinline__ void store_linear_out(void* y, int64_t i, float v, const void* residual) {
  if (residual) v = Elem<DT>::round(v) + Elem<DT>::load(residual, i);
  Elem<DT>::store(y, i, v);
}

// ---------------------------------------------------------------- eight 16-bit elements in one 16-byte piece

typedef uint32_t dec_u4 __attribute__((ext_vector_type(4)));

template <int DT>
__device__ __forceinline__ void unpack8(dec_u4 v, float* f) {
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    if constexpr (DT == SUBSPEC_BF16) {
      f[2 * j] = bf16_bits_to_float(v[j] & 0xffffu);
      f[2 * j + 1] = bf16_bits_to_float(v[j] >> 16);
    } else {
      f[2 * j] = f16_bits_to_float(v[j] & 0xffffu);
      f[2 * j + 1] = f16_bits_to_float(v[j] >> 16);
    }
  }
}
template <int DT>
__device__ __forceinline__ uint32_t to_bits(float v) {
  if constexpr (DT == SUBSPEC_BF16) {
    return __float_as_uint(round_bf16(v)) >> 16;
  } else {
    union { uint16_t u; _Float16 h; } c;
    c.h = (_Float16)v;
    return c.u;
  }
}
typedef float dec_f2 __attribute__((ext_vector_type(2)));
typedef __bf16 dec_bf2 __attribute__((ext_vector_type(2)));
typedef _Float16 dec_h2 __attribute__((ext_vector_type(2)));
// two values rounded to nearest even and packed, low half first (one packed conversion per pair)
template <int DT>
__device__ __forceinline__ uint32_t pack2(float lo, float hi) {
  if constexpr (DT == SUBSPEC_BF16) return __builtin_bit_cast(uint32_t, __builtin_convertvector(dec_f2{lo, hi}, dec_bf2));
  else return __builtin_bit_cast(uint32_t, __builtin_convertvector(dec_f2{lo, hi}, dec_h2));
}
template <int DT>
__device__ __forceinline__ dec_u4 pack8(const float* f) {
  dec_u4 v;
#pragma unroll
  for (int j = 0; j < 4; ++j) v[j] = pack2<DT>(f[2 * j], f[2 * j + 1]);
  return v;
}

// ---------------------------------------------------------------- wave / block reductions
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, kWave));
  return v;
}
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, kWave);
  return v;
}
__device__ __forceinline__ int wave_min_i(int v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = min(v, __shfl_xor(v, o, kWave));
  return v;
}

// Block-wide reductions over THREADS threads; `scratch` holds at least THREADS/64 words and may
// be reused after the call returns (each helper ends with a barrier).
template <int THREADS>
__device__ __forceinline__ float block_max(float v, float* scratch) {
  constexpr int W = THREADS / kWave;
  v = wave_max(v);
  if ((threadIdx.x & (kWave - 1)) == 0) scratch[threadIdx.x / kWave] = v;
  __syncthreads();
  float r = scratch[0];
#pragma unroll
  for (int i = 1; i < W; ++i) r = fmaxf(r, scratch[i]);
  __syncthreads();
  return r;
}
// Sum in a fixed order (wave butterfly, then waves 0..W-1) so results do not depend on timing.
template <int THREADS>
__device__ __forceinline__ float block_sum(float v, float* scratch) {
  constexpr int W = THREADS / kWave;
  v = wave_sum(v);
  if ((threadIdx.x & (kWave - 1)) == 0) scratch[threadIdx.x / kWave] = v;
  __syncthreads();
  float r = scratch[0];
#pragma unroll
  for (int i = 1; i < W; ++i) r += scratch[i];
  __syncthreads();
  return r;
}
template <int THREADS>
__device__ __forceinline__ int block_min_i(int v, int* scratch) {
  constexpr int W = THREADS / kWave;
  v = wave_min_i(v);
  if ((threadIdx.x & (kWave - 1)) == 0) scratch[threadIdx.x / kWave] = v;
  __syncthreads();
  int r = scratch[0];
#pragma unroll
  for (int i = 1; i < W; ++i) r = min(r, scratch[i]);
  __syncthreads();
  return r;
}

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

// A request's page table over one layer of a page pool [max_pages][2 (K, V)][page_len][n_kv_heads][128]
struct KvPages { const int32_t* table; int64_t n_pages, max_pages, page_len; };

// Where the K / V row of (kv head, cache row) lives, for kernels that write rows: contiguous [Hkv, seq_stride, 128]
// caches, or one layer of a page pool (then v_cache is unused and a row outside the request's pages does not exist).
struct KvRowMap {
  uint16_t* k_cache;
  uint16_t* v_cache;
  int64_t seq_stride;            // rows a head holds (contiguous), or pages * page_len (paged)
  const int32_t* page_table;     // null: contiguous
  int page_shift, max_pages, hkv;
  int64_t page_elems;            // paged: elements of one page of K (page_len * hkv * 128); V follows K inside a page
};
// element offset pointers of row `row` of head `kvh`, or false when the row is outside the cache
__device__ __forceinline__ bool kv_row_ptrs(const KvRowMap& m, int kvh, int64_t row, uint16_t** k, uint16_t** v) {
  if (row < 0 || row >= m.seq_stride) return false;
  if (m.page_table) {
    const int page = min(max(m.page_table[row >> m.page_shift], 0), m.max_pages - 1);     // a bad table must not leave the pool
    const int64_t off = (int64_t)page * 2 * m.page_elems + ((row & ((1 << m.page_shift) - 1)) * m.hkv + kvh) * 128;
    *k = m.k_cache + off;
    *v = m.k_cache + off + m.page_elems;
  } else {
    const int64_t off = ((int64_t)kvh * m.seq_stride + row) * 128;
    *k = m.k_cache + off;
    *v = m.v_cache + off;
  }
  return true;
}
inline KvRowMap make_kv_row_map(void* k_cache, void* v_cache, int64_t seq_stride, int64_t hkv, const KvPages* pages) {
  KvRowMap m{};
  m.k_cache = (uint16_t*)k_cache;
  m.v_cache = (uint16_t*)v_cache;
  m.seq_stride = seq_stride;
  m.hkv = (int)hkv;
  if (pages) {
    int shift = 0;
    while ((1ll << shift) < pages->page_len) ++shift;
    m.page_table = pages->table;
    m.page_shift = shift;
    m.max_pages = (int)pages->max_pages;
    m.page_elems = pages->page_len * hkv * 128;
    m.seq_stride = pages->n_pages * pages->page_len;
  }
  return m;
}
// subspec_tree_attention (batch 1, head_dim 128) with two options of the decoder-layer entry points: prefix_dev (the
// kernel reads the prefix length from device memory, prefix_len is its upper bound) and pages (k_cache = one layer of
// a page pool, v_cache unused)
int tree_attention_ex(const void* q, const void* k_cache, const void* v_cache, void* out, int dtype, int64_t n_q_heads,
                      int64_t n_kv_heads, int64_t n_rows, int64_t n_tree_slots, int64_t kv_seq_stride, int64_t prefix_len,
                      const int64_t* prefix_dev, const KvPages* pages, const uint64_t* anc_bits, float scale, void* workspace,
                      size_t workspace_bytes, void* stream);

// Linear layers with a fused residual add (y = x W^T + bias + residual; residual may alias y); the C entry points
// are these with residual = NULL.  Used by the decoder-layer sequence.
int int4_linear_ex(const void* x, const uint32_t* wq, const uint32_t* sz, const void* bias, const void* residual, void* y,
                   int dtype, int64_t M, int64_t N, int64_t K, int64_t group_size, void* workspace, size_t workspace_bytes,
                   void* stream);
// act[M, F] = round(silu(round(gate))) * round(up) with gate | up = x * W^T (+ bias), W of N = 2F rows (gate rows first):
// the SwiGLU MLP's first projection and its activation in one launch
// norm_gain != NULL: x is the un-normalized residual stream and RMSNorm (gain [K], eps) is the projection's prologue (M <= 32)
int int4_gate_up_silu_ex(const void* x, const uint32_t* wq, const uint32_t* sz, const void* bias, void* act, int dtype,
                         int64_t M, int64_t N, int64_t K, const void* norm_gain, float norm_eps, void* stream);
// q|k|v projection (N = (Hq + 2 Hkv) * 128 rows) with the rotary embedding and the cache write in its output stage:
// q to q_out [Hq, M, 128], K / V rows to cache_rows[m] of the layer's [Hkv, seq_stride, 128] caches; optional RMSNorm prologue
int int4_qkv_rope_ex(const void* x, const uint32_t* wq, const uint32_t* sz, const void* bias, int dtype, int64_t M, int64_t K,
                     const void* norm_gain, float norm_eps, const int32_t* positions, const int32_t* cache_rows, void* q_out,
                     const KvRowMap& kv, int64_t n_q_heads, float rope_theta, const float* inv_freq, void* stream);
int dense_gate_up_silu_ex(const void* x, const void* w, const void* bias, void* act, int dtype, int64_t M, int64_t N,
                          int64_t K, void* stream);
// pending_splits != NULL: when K is split over workgroups the launch that sums the fp32 partials
// (workspace: [splits][M][N]) is left to the caller's next kernel, *pending_splits = number of partials (then neither bias
// nor residual has been applied and y is untouched); 1: y is complete
int dense_linear_ex(const void* x, const void* w, const void* bias, const void* residual, void* y, int dtype, int64_t M,
                    int64_t N, int64_t K, void* workspace, size_t workspace_bytes, void* stream, int* pending_splits = nullptr);


}  // namespace subspec
