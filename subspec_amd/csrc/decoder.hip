// One decoder layer over the tree rows, launched from one host call: the substitute draft's int4
// layer, and the target's layer with dense 16-bit projections (same sequence, see the end).
//
// The reference runs the draft as a HuggingFace Qwen2 / Llama decoder layer whose seven projections
// were replaced by HQQ int4 linears (specdecodes/helpers/recipes/subspec/hqq_4bit_postspec.py:17-58)
// and hides the per-module launch cost behind torch.compile / captured graphs
// (specdecodes/models/draft_models/classic_sd.py:85-118 for the step it repeats per tree level).
// Here the layer is a fixed sequence of launches issued by native code on the caller's stream:
//   h      = rmsnorm(x) * w_in
//   qkv    = int4(h) + bias                     [M, (Hq + 2 Hkv) D]
//   q, K/V = rope(qkv), K and V rows written into the static cache at cache_rows
//   a      = tree attention(q, cache)           [M, Hq D]
//   x     += int4(a)                            (o_proj; the add is fused into the next rmsnorm)
//   h      = rmsnorm(x) * w_post
//   act    = silu(gate) * up,  gate|up = int4(h)
//   x     += int4(act)                          (down_proj; the add is fused into its output stage)
// Rounding follows the eager torch layer: every intermediate tensor is rounded to the activation
// dtype where torch would materialise it (normalised activations before the weight product, the
// two rotary products and their sum, silu before the product with `up`, both residual sums).
//
// The target model's layer in the tree-decoding forward (HF Qwen2DecoderLayer under
// ClassicSDGeneratorBase._tree_decoding, specdecodes/models/generators/classic_sd.py:75-109) is the
// same sequence with dense 16-bit projections (dense.hip) in place of the int4 ones.
#include "common.h"
#include <algorithm>

namespace subspec {

// x[m] (+= delta[m], rounded, written back) ; y[m] = w * round(x * rsqrt(mean(x^2) + eps))
// One workgroup per row; H % 8 == 0.  kMaxPieces 16-byte pieces per thread cover H <= 256 * 8 * kMaxPieces.
// splits > 0: delta is not a 16-bit tensor yet but `splits` fp32 partial sums [splits][rows][H] of a projection whose K
// was split over workgroups; they are summed in split order and rounded here (what the projection's own reduction
// launch would have stored), which saves that launch.
constexpr int kNormThreads = 256;
constexpr int kNormMaxPieces = 8;
template <int DT, bool kAdd>
__global__ __launch_bounds__(kNormThreads) void add_rmsnorm_kernel(uint16_t* __restrict__ x, const uint16_t* __restrict__ delta,
                                                                   const uint16_t* __restrict__ w, uint16_t* __restrict__ y,
                                                                   int H, float eps, const float* __restrict__ partial = nullptr,
                                                                   int splits = 0) {
  __shared__ float scratch[kNormThreads / kWave];
  const int m = blockIdx.x, tid = threadIdx.x, pieces = H / 8;
  dec_u4* xr = (dec_u4*)(x + (int64_t)m * H);
  const dec_u4* dr = (const dec_u4*)(delta + (int64_t)m * H);
  float v[kNormMaxPieces][8];
  float ss = 0.f;
#pragma unroll
  for (int p = 0; p < kNormMaxPieces; ++p) {
    const int i = p * kNormThreads + tid;
    if (i < pieces) {
      unpack8<DT>(xr[i], v[p]);
      if constexpr (kAdd) {
        float d[8];
        if (splits > 0) {
#pragma unroll
          for (int j = 0; j < 8; ++j) d[j] = 0.f;
          for (int sp = 0; sp < splits; ++sp) {
            const float4* pp = (const float4*)(partial + ((int64_t)sp * gridDim.x + m) * H) + 2 * i;
            const float4 a = pp[0], b = pp[1];
            d[0] += a.x; d[1] += a.y; d[2] += a.z; d[3] += a.w; d[4] += b.x; d[5] += b.y; d[6] += b.z; d[7] += b.w;
          }
#pragma unroll
          for (int j = 0; j < 8; ++j) d[j] = Elem<DT>::round(d[j]);
        } else {
          unpack8<DT>(dr[i], d);
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) v[p][j] = Elem<DT>::round(v[p][j] + d[j]);
        xr[i] = pack8<DT>(v[p]);
      }
#pragma unroll
      for (int j = 0; j < 8; ++j) ss = fmaf(v[p][j], v[p][j], ss);
    }
  }
  const float tot = block_sum<kNormThreads>(ss, scratch);
  const float r = rsqrtf(tot / (float)H + eps);
#pragma unroll
  for (int p = 0; p < kNormMaxPieces; ++p) {
    const int i = p * kNormThreads + tid;
    if (i < pieces) {
      float wv[8], o[8];
      unpack8<DT>(((const dec_u4*)w)[i], wv);
#pragma unroll
      for (int j = 0; j < 8; ++j) o[j] = wv[j] * Elem<DT>::round(v[p][j] * r);
      ((dec_u4*)(y + (int64_t)m * H))[i] = pack8<DT>(o);
    }
  }
}

// act[m, f] = round(silu(gate)) * up with gate = gu[m, f], up = gu[m, F + f]
template <int DT>
__global__ __launch_bounds__(256) void silu_mul_kernel(const uint16_t* __restrict__ gu, uint16_t* __restrict__ act, int F,
                                                       int64_t pieces) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= pieces) return;
  const int per_row = F / 8;
  const int64_t m = i / per_row;
  const int p = (int)(i % per_row);
  float g[8], u[8];
  unpack8<DT>(((const dec_u4*)(gu + m * 2 * F))[p], g);
  unpack8<DT>(((const dec_u4*)(gu + m * 2 * F + F))[p], u);
#pragma unroll
  for (int j = 0; j < 8; ++j) g[j] = Elem<DT>::round(g[j] / (1.f + __expf(-g[j]))) * u[j];
  ((dec_u4*)(act + m * F))[p] = pack8<DT>(g);
}

// Rotary embedding (rotate-half form, angle = position * theta^(-2i/D)) of the q and k heads of
// qkv [M, (Hq + 2 Hkv) * D]; q goes to q_out [Hq, M, D], k and v to rows cache_rows[m] of the
// layer's [Hkv, S, D] caches.  One wavefront per (row, head); lane i handles dims i and i + D/2.
// splits > 0: qkv is still `splits` fp32 partial sums [splits][M][(Hq + 2 Hkv) * D] of the projection (K split over
// workgroups) and `bias` its bias; sum, bias and the rounding to the activation dtype happen here instead of in a
// reduction launch of their own.
template <int DT>
__global__ __launch_bounds__(64) void rope_write_kernel(const uint16_t* __restrict__ qkv, const int32_t* __restrict__ positions,
                                                        const int32_t* __restrict__ cache_rows, uint16_t* __restrict__ q_out,
                                                        KvRowMap kv, int M, int Hq, int Hkv, int D, float log2_theta,
                                                        const float* __restrict__ inv_freq_table,
                                                        const float* __restrict__ partial = nullptr, int splits = 0,
                                                        const uint16_t* __restrict__ bias = nullptr) {
  const int m = blockIdx.x, hh = blockIdx.y, i = threadIdx.x;
  const int half = D / 2;
  if (i >= half) return;
  float lo, hi;
  if (splits > 0) {
    const int64_t width = (int64_t)(Hq + 2 * Hkv) * D, col = (int64_t)hh * D + i;
    lo = hi = 0.f;
    for (int sp = 0; sp < splits; ++sp) {
      const float* pp = partial + ((int64_t)sp * M + m) * width + col;
      lo += pp[0];
      hi += pp[half];
    }
    lo = Elem<DT>::round(lo + (bias ? Elem<DT>::load(bias, col) : 0.f));
    hi = Elem<DT>::round(hi + (bias ? Elem<DT>::load(bias, col + half) : 0.f));
  } else {
    const uint16_t* src = qkv + ((int64_t)m * (Hq + 2 * Hkv) + hh) * D;
    lo = Elem<DT>::load(src, i);
    hi = Elem<DT>::load(src, i + half);
  }
  uint16_t* dst;
  if (hh < Hq) {
    dst = q_out + ((int64_t)hh * M + m) * D;
  } else {
    // a row outside the layer's cache is dropped: a bad rows tensor must not write beyond the cache
    uint16_t *kp, *vp;
    if (!kv_row_ptrs(kv, (hh - Hq) % Hkv, cache_rows[m], &kp, &vp)) return;
    dst = hh < Hq + Hkv ? kp : vp;
  }
  if (hh >= Hq + Hkv) {                                 // value heads are copied
    Elem<DT>::store(dst, i, lo);
    Elem<DT>::store(dst, i + half, hi);
    return;
  }
  // the caller's table (the values its other code paths use, so that both write identical rows), else theta^(-2i/D)
  const float inv_freq = inv_freq_table ? inv_freq_table[i] : exp2f(-(float)(2 * i) / (float)D * log2_theta);
  float s, c;
  sincosf((float)positions[m] * inv_freq, &s, &c);
  c = Elem<DT>::round(c);
  s = Elem<DT>::round(s);
  // t * cos + rotate_half(t) * sin, each product and the sum rounded like the eager tensor ops
  const float o_lo = Elem<DT>::round(lo * c) + Elem<DT>::round(-hi * s);
  const float o_hi = Elem<DT>::round(hi * c) + Elem<DT>::round(lo * s);
  Elem<DT>::store(dst, i, o_lo);
  Elem<DT>::store(dst, i + half, o_hi);
}

// rows of one call: the int4 stack serves draft levels and post-verify windows, the dense stack also whole large trees
constexpr int kInt4LayerMaxRows = 64, kDenseLayerMaxRows = 384;
struct LayerPlan {
  size_t h, qkv, q, a, o, gu, act, sub, sub_bytes, total;
};
static LayerPlan layer_plan(const subspec_decoder_layer_dims& s) {
  LayerPlan p;
  const size_t es = 2, M = (size_t)s.n_rows, H = (size_t)s.hidden, Q = (size_t)s.n_q_heads * s.head_dim,
               KV = (size_t)s.n_kv_heads * s.head_dim, F = (size_t)s.intermediate;
  size_t off = 0;
  auto take = [&](size_t bytes) { size_t o = off; off += align_up(bytes, 256); return o; };
  p.h = take(M * H * es);
  p.qkv = take(M * (Q + 2 * KV) * es);
  p.q = take(M * Q * es);
  p.a = take(M * Q * es);
  p.o = take(M * H * es);
  p.gu = take(M * 2 * F * es);
  p.act = take(M * F * es);
  size_t sub = 256;
  if (s.n_rows <= kInt4LayerMaxRows) {                 // wider windows are dense only
    sub = std::max(sub, subspec_int4_linear_workspace(s.n_rows, Q + 2 * KV, H));
    sub = std::max(sub, subspec_int4_linear_workspace(s.n_rows, H, Q));
    sub = std::max(sub, subspec_int4_linear_workspace(s.n_rows, 2 * F, H));
    sub = std::max(sub, subspec_int4_linear_workspace(s.n_rows, H, F));
  }
  sub = std::max(sub, subspec_dense_linear_workspace(s.n_rows, Q + 2 * KV, H));
  sub = std::max(sub, subspec_dense_linear_workspace(s.n_rows, H, Q));
  sub = std::max(sub, subspec_dense_linear_workspace(s.n_rows, 2 * F, H));
  sub = std::max(sub, subspec_dense_linear_workspace(s.n_rows, H, F));
  sub = std::max(sub, subspec_tree_attention_workspace(1, s.n_q_heads, s.n_kv_heads, s.n_rows, s.prefix_len, s.n_tree_slots));
  p.sub_bytes = align_up(sub, 256);
  p.sub = take(p.sub_bytes);
  p.total = off;
  return p;
}

static int check_dims(const subspec_decoder_layer_dims* s, int max_rows) {
  if (!s) SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "decoder_layer: null dims");
  if (s->dtype != SUBSPEC_BF16 && s->dtype != SUBSPEC_F16)
    SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "decoder_layer: dtype %d not supported (bf16 / fp16 only)", s->dtype);
  if (s->n_rows < 1 || s->n_rows > max_rows)
    SUBSPEC_FAIL(SUBSPEC_ERR_LIMIT, "decoder_layer: n_rows=%lld outside 1..%d", (long long)s->n_rows, max_rows);
  if (s->head_dim != 128) SUBSPEC_FAIL(SUBSPEC_ERR_LIMIT, "decoder_layer: head_dim=%lld (built for 128)", (long long)s->head_dim);
  if (s->hidden <= 0 || s->hidden % 64 != 0 || s->hidden > 8 * kNormThreads * kNormMaxPieces)
    SUBSPEC_FAIL(SUBSPEC_ERR_LIMIT, "decoder_layer: hidden=%lld must be a multiple of 64 and at most %d", (long long)s->hidden,
                 8 * kNormThreads * kNormMaxPieces);
  if (s->intermediate <= 0 || s->intermediate % 64 != 0)
    SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "decoder_layer: intermediate=%lld must be a multiple of 64", (long long)s->intermediate);
  if (s->n_q_heads <= 0 || s->n_kv_heads <= 0 || s->n_q_heads % s->n_kv_heads != 0)
    SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "decoder_layer: %lld query heads over %lld kv heads", (long long)s->n_q_heads, (long long)s->n_kv_heads);
  if (s->n_tree_slots < 1 || s->n_tree_slots > SUBSPEC_MAX_TREE_NODES || s->prefix_len < 0 || s->prefix_len + s->n_tree_slots > s->kv_seq_stride)
    SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "decoder_layer: prefix_len=%lld, n_tree_slots=%lld do not fit a cache of %lld rows",
                 (long long)s->prefix_len, (long long)s->n_tree_slots, (long long)s->kv_seq_stride);
  if (!(s->rope_theta > 1.f) || !(s->rms_eps > 0.f)) SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "decoder_layer: rope_theta / rms_eps out of range");
  if (s->page_indices) {
    if (s->page_len <= 0 || (s->page_len & (s->page_len - 1)) != 0 || s->page_len > 4096)
      SUBSPEC_FAIL(SUBSPEC_ERR_LIMIT, "decoder_layer: page_len=%lld must be a power of two up to 4096", (long long)s->page_len);
    if (s->n_pages <= 0 || s->max_pages < s->n_pages || s->max_pages > 0x7fffffff)
      SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "decoder_layer: n_pages=%lld max_pages=%lld", (long long)s->n_pages, (long long)s->max_pages);
    if (s->kv_seq_stride != s->n_pages * s->page_len)
      SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "decoder_layer: kv_seq_stride=%lld must equal n_pages * page_len = %lld for a paged cache",
                   (long long)s->kv_seq_stride, (long long)(s->n_pages * s->page_len));
  }
  return SUBSPEC_OK;
}

// The four projections of a layer in either storage: int4 codes + (scale, zero) words, or a dense
// row-major 16-bit matrix (then the second pointer is unused).
struct Projection { const void* w; const void* sz; };
struct LayerWeights {
  const void *input_norm, *post_norm, *qkv_bias;
  Projection qkv, o, gate_up, down;
  bool dense;
};
static int project(const LayerWeights& w, const Projection& p, const void* x, const void* bias, const void* residual, void* y,
                   int dtype, int64_t M, int64_t N, int64_t K, void* sub, size_t sub_bytes, hipStream_t st,
                   int* pending_splits = nullptr) {
  if (pending_splits) *pending_splits = 1;
  if (w.dense) return dense_linear_ex(x, p.w, bias, residual, y, dtype, M, N, K, sub, sub_bytes, st, pending_splits);
  return int4_linear_ex(x, (const uint32_t*)p.w, (const uint32_t*)p.sz, bias, residual, y, dtype, M, N, K, 64, sub, sub_bytes, st);
}

template <int DT>
static int run_layer(const subspec_decoder_layer_dims& s, const LayerWeights& w, uint16_t* x,
                     const int32_t* positions, const int32_t* cache_rows, const uint64_t* anc_bits, uint16_t* k_cache,
                     uint16_t* v_cache, char* ws, hipStream_t st) {
  const LayerPlan p = layer_plan(s);
  const int M = (int)s.n_rows, H = (int)s.hidden, Hq = (int)s.n_q_heads, Hkv = (int)s.n_kv_heads, D = (int)s.head_dim,
            F = (int)s.intermediate;
  const int64_t Q = (int64_t)Hq * D, KV = (int64_t)Hkv * D;
  uint16_t *h = (uint16_t*)(ws + p.h), *qkv = (uint16_t*)(ws + p.qkv), *q = (uint16_t*)(ws + p.q), *a = (uint16_t*)(ws + p.a),
           *o = (uint16_t*)(ws + p.o), *gu = (uint16_t*)(ws + p.gu), *act = (uint16_t*)(ws + p.act);
  void* sub = ws + p.sub;
  const KvPages pages{s.page_indices, s.n_pages, s.max_pages, s.page_len};
  const KvPages* pg = s.page_indices ? &pages : nullptr;
  const KvRowMap kv = make_kv_row_map(k_cache, v_cache, s.kv_seq_stride, Hkv, pg);
  int rc;
  // int4 stack, a level of at most 32 rows: five launches per layer (six with a split-K down projection, seven when
  // the keys are split) -- both norms are prologues of the projections that consume them, rotary + cache write is the
  // output stage of q|k|v, the attention block's residual add the output stage of o_proj
  const bool fused = !w.dense && M <= 32 && subspec_int4_linear_workspace(M, Q + 2 * KV, H) == 256;
  if (fused) {
    if ((rc = int4_qkv_rope_ex(x, (const uint32_t*)w.qkv.w, (const uint32_t*)w.qkv.sz, w.qkv_bias, DT, M, H, w.input_norm, s.rms_eps,
                               positions, cache_rows, q, kv, Hq, s.rope_theta, s.rope_inv_freq, st)))
      return rc;
  } else {
    hipLaunchKernelGGL((add_rmsnorm_kernel<DT, false>), dim3(M), dim3(kNormThreads), 0, st, x, (const uint16_t*)nullptr,
                       (const uint16_t*)w.input_norm, h, H, s.rms_eps);
    // dense projections whose K is split leave the sum of their partials to the kernel that reads them next
    int pending = 0;
    if ((rc = project(w, w.qkv, h, w.qkv_bias, nullptr, qkv, DT, M, Q + 2 * KV, H, sub, p.sub_bytes, st, &pending))) return rc;
    hipLaunchKernelGGL((rope_write_kernel<DT>), dim3(M, Hq + 2 * Hkv), dim3(64), 0, st, qkv, positions, cache_rows, q, kv,
                       M, Hq, Hkv, D, log2f(s.rope_theta), s.rope_inv_freq, (const float*)sub, pending > 1 ? pending : 0,
                       (const uint16_t*)w.qkv_bias);
  }
  if ((rc = tree_attention_ex(q, k_cache, v_cache, a, DT, Hq, Hkv, M, s.n_tree_slots, s.kv_seq_stride, s.prefix_len,
                              s.prefix_len_dev, pg, anc_bits, 1.f / sqrtf((float)D), sub, p.sub_bytes, st)))
    return rc;
  if (fused) {
    // x = round(round(o_proj(a)) + x), then RMSNorm inside the gate|up projection
    if ((rc = project(w, w.o, a, nullptr, x, x, DT, M, H, Q, sub, p.sub_bytes, st))) return rc;
    if ((rc = int4_gate_up_silu_ex(x, (const uint32_t*)w.gate_up.w, (const uint32_t*)w.gate_up.sz, nullptr, act, DT, M,
                                   2 * (int64_t)F, H, w.post_norm, s.rms_eps, st)))
      return rc;
  } else {
  int pending = 0;
  if ((rc = project(w, w.o, a, nullptr, nullptr, o, DT, M, H, Q, sub, p.sub_bytes, st, &pending))) return rc;
  hipLaunchKernelGGL((add_rmsnorm_kernel<DT, true>), dim3(M), dim3(kNormThreads), 0, st, x, o, (const uint16_t*)w.post_norm, h, H,
                     s.rms_eps, (const float*)sub, pending > 1 ? pending : 0);
  if (!w.dense) {
    // the activation sits in the output stage of the gate|up projection
    if ((rc = int4_gate_up_silu_ex(h, (const uint32_t*)w.gate_up.w, (const uint32_t*)w.gate_up.sz, nullptr, act, DT, M,
                                   2 * (int64_t)F, H, nullptr, 0.f, st)))
      return rc;
  } else if (M > 32 || 4 * (int64_t)F * H < ((int64_t)1 << 31)) {   // (up to 32 rows the pair kernel addresses the matrix through one 2 GiB descriptor)
    if ((rc = dense_gate_up_silu_ex(h, w.gate_up.w, nullptr, act, DT, M, 2 * (int64_t)F, H, st))) return rc;
  } else {
    if ((rc = project(w, w.gate_up, h, nullptr, nullptr, gu, DT, M, 2 * (int64_t)F, H, sub, p.sub_bytes, st))) return rc;
    const int64_t act_pieces = (int64_t)M * F / 8;
    hipLaunchKernelGGL((silu_mul_kernel<DT>), dim3((unsigned)((act_pieces + 255) / 256)), dim3(256), 0, st, gu, act, F, act_pieces);
  }
  }
  // down projection with the residual add in its output stage: x = round(round(down(act)) + x)
  if ((rc = project(w, w.down, act, nullptr, x, x, DT, M, H, F, sub, p.sub_bytes, st))) return rc;
  SUBSPEC_CHECK_HIP(hipGetLastError());
  return SUBSPEC_OK;
}

}  // namespace subspec

using namespace subspec;

extern "C" int subspec_rms_norm(const void* x, const void* weight, void* y, int dtype, int64_t rows, int64_t hidden,
                                float eps, void* stream) {
  if (dtype != SUBSPEC_BF16 && dtype != SUBSPEC_F16) SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "rms_norm: dtype %d not supported (bf16 / fp16)", dtype);
  if (!x || !weight || !y) SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "rms_norm: null pointer argument");
  if (rows <= 0 || rows > 0x7fffffff) SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "rms_norm: rows=%lld", (long long)rows);
  if (hidden <= 0 || hidden % 8 != 0 || hidden > 8 * kNormThreads * kNormMaxPieces)
    SUBSPEC_FAIL(SUBSPEC_ERR_LIMIT, "rms_norm: hidden=%lld must be a multiple of 8 and at most %d", (long long)hidden,
                 8 * kNormThreads * kNormMaxPieces);
  if (!(eps > 0.f)) SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "rms_norm: eps out of range");
  if ((uintptr_t)x % 16 || (uintptr_t)weight % 16 || (uintptr_t)y % 16) SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "rms_norm: pointers must be 16-byte aligned");
  hipStream_t st = (hipStream_t)stream;
  // the kernel only writes x when it also adds: here it reads it
  if (dtype == SUBSPEC_BF16)
    hipLaunchKernelGGL((add_rmsnorm_kernel<SUBSPEC_BF16, false>), dim3((unsigned)rows), dim3(kNormThreads), 0, st, (uint16_t*)x,
                       (const uint16_t*)nullptr, (const uint16_t*)weight, (uint16_t*)y, (int)hidden, eps);
  else
    hipLaunchKernelGGL((add_rmsnorm_kernel<SUBSPEC_F16, false>), dim3((unsigned)rows), dim3(kNormThreads), 0, st, (uint16_t*)x,
                       (const uint16_t*)nullptr, (const uint16_t*)weight, (uint16_t*)y, (int)hidden, eps);
  SUBSPEC_CHECK_HIP(hipGetLastError());
  return SUBSPEC_OK;
}

extern "C" size_t subspec_int4_decoder_layer_workspace(const subspec_decoder_layer_dims* dims) {
  if (!dims || check_dims(dims, kDenseLayerMaxRows) != SUBSPEC_OK) return 0;
  return layer_plan(*dims).total;
}

static int decoder_layer_entry(const subspec_decoder_layer_dims* dims, const LayerWeights& w, void* x, const int32_t* positions,
                               const int32_t* cache_rows, const uint64_t* anc_bits, void* k_cache, void* v_cache,
                               void* workspace, size_t workspace_bytes, void* stream) {
  const int rc = check_dims(dims, w.dense ? kDenseLayerMaxRows : kInt4LayerMaxRows);
  if (rc != SUBSPEC_OK) return rc;
  // the wide dense kernels take weight rows in tiles of 32
  if (dims->n_rows > 64 && ((dims->n_q_heads + 2 * dims->n_kv_heads) * dims->head_dim % 32 != 0 || dims->hidden % 32 != 0))
    SUBSPEC_FAIL(SUBSPEC_ERR_LIMIT, "decoder_layer: more than 64 rows need projection widths that are multiples of 32");
  if (!x || !positions || !cache_rows || !anc_bits || !k_cache || (!v_cache && !dims->page_indices))
    SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "decoder_layer: null pointer argument");
  if (!w.input_norm || !w.post_norm || !w.qkv.w || !w.o.w || !w.gate_up.w || !w.down.w ||
      (!w.dense && (!w.qkv.sz || !w.o.sz || !w.gate_up.sz || !w.down.sz)))
    SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "decoder_layer: null weight pointer");
  if ((uintptr_t)x % 16 || (uintptr_t)w.input_norm % 16 || (uintptr_t)w.post_norm % 16 || (uintptr_t)k_cache % 16 ||
      (uintptr_t)v_cache % 16)
    SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "decoder_layer: x, norm weights and caches must be 16-byte aligned");
  const size_t need = layer_plan(*dims).total;
  if (!workspace || workspace_bytes < need)
    SUBSPEC_FAIL(SUBSPEC_ERR_WORKSPACE, "decoder_layer: workspace of %zu bytes is smaller than the %zu required", workspace_bytes, need);
  if ((uintptr_t)workspace % 256) SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "decoder_layer: workspace must be 256-byte aligned");
  if (dims->dtype == SUBSPEC_BF16)
    return run_layer<SUBSPEC_BF16>(*dims, w, (uint16_t*)x, positions, cache_rows, anc_bits, (uint16_t*)k_cache, (uint16_t*)v_cache,
                                   (char*)workspace, (hipStream_t)stream);
  return run_layer<SUBSPEC_F16>(*dims, w, (uint16_t*)x, positions, cache_rows, anc_bits, (uint16_t*)k_cache, (uint16_t*)v_cache,
                                (char*)workspace, (hipStream_t)stream);
}

extern "C" int subspec_int4_decoder_layer(const subspec_decoder_layer_dims* dims, const subspec_decoder_layer_weights* weights,
                                          void* x, const int32_t* positions, const int32_t* cache_rows,
                                          const uint64_t* anc_bits, void* k_cache, void* v_cache, void* workspace,
                                          size_t workspace_bytes, void* stream) {
  if (!weights) SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "decoder_layer: null weights");
  const subspec_decoder_layer_weights& s = *weights;
  const LayerWeights w{s.input_norm, s.post_norm, s.qkv_bias, {s.qkv_wq, s.qkv_sz}, {s.o_wq, s.o_sz},
                       {s.gate_up_wq, s.gate_up_sz}, {s.down_wq, s.down_sz}, false};
  return decoder_layer_entry(dims, w, x, positions, cache_rows, anc_bits, k_cache, v_cache, workspace, workspace_bytes, stream);
}

extern "C" int subspec_dense_decoder_layer(const subspec_decoder_layer_dims* dims, const subspec_dense_layer_weights* weights,
                                           void* x, const int32_t* positions, const int32_t* cache_rows,
                                           const uint64_t* anc_bits, void* k_cache, void* v_cache, void* workspace,
                                           size_t workspace_bytes, void* stream) {
  if (!weights) SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "decoder_layer: null weights");
  const subspec_dense_layer_weights& s = *weights;
  const LayerWeights w{s.input_norm, s.post_norm, s.qkv_bias, {s.qkv_w, nullptr}, {s.o_w, nullptr},
                       {s.gate_up_w, nullptr}, {s.down_w, nullptr}, true};
  return decoder_layer_entry(dims, w, x, positions, cache_rows, anc_bits, k_cache, v_cache, workspace, workspace_bytes, stream);
}
