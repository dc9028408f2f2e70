// Tree-masked GQA attention of the draft tree against the static KV cache, for gfx950.
//
// Replaces the reference's HF sdpa_attention_forward forced to the math backend with an additive
// finfo.min mask over the whole static cache plus repeat_kv (run/pipelines/run_test.py:64;
// specdecodes/models/generators/classic_sd.py:57-109; mask from cpu_tree.py:263-286 and
// utils/utils.py:4-6): O = softmax(Q K^T * scale + M) V, where tree row i sees the whole prefix and,
// among the tree slots, only node i and its ancestors.
//
// Layout and mapping
//   q        [B, Hq, n, D]            (n <= 64 query rows, D = 128)
//   k, v     [B, Hkv, S, D]           static cache; rows [0, prefix) are the prompt, rows
//                                     [prefix, prefix + slots) hold the tree nodes (slots <= 64)
//   anc      [B or 1, n] u64          bit j of word i: query row i may attend to tree slot j
//                                     (the node in slot j is the row's node or one of its ancestors)
//   out      [B, n, Hq, D]
// One workgroup (4 wavefronts) owns one query head's 64 rows and one chunk of the keys; wavefront
// w owns rows 16w..16w+15.  Scores are produced TRANSPOSED, S^T = K Q^T, with
// v_mfma_f32_16x16x16: the accumulator then holds, per lane, four consecutive keys of one query,
// which is exactly the B-operand layout of the second product O^T = V^T P^T, so probabilities go
// from one MFMA to the next without leaving registers, and the row maximum / sum need only two
// cross-lane steps.  The ancestor bitset of the lane's query sits in a register pair; prefix keys
// need no mask at all.  K is staged row-major in LDS, V transposed, both with 16-byte global loads.
// When the keys are split over several workgroups the partial (O, max, sum) triples are merged by
// tree_attention_merge_kernel.
// HBM-bound at the benchmark sizes provided QK^T / PV run on the matrix cores:
// algorithmic bytes per batch element = K+V rows actually attended + Q + O.
#include "common.h"
#include <algorithm>

namespace subspec {

constexpr int kAttnThreads = 256;
constexpr int kAttnRows = 64;          // query rows per workgroup (one q head)
constexpr int kAttnD = 128;
constexpr int kKeyBlock = 64;
constexpr int kKStride = kAttnD + 8;   // LDS row stride (elements) of the K tile
constexpr int kVStride = kKeyBlock + 8;  // LDS row stride (elements) of the transposed V tile

typedef short v4s __attribute__((ext_vector_type(4)));
typedef _Float16 v4h __attribute__((ext_vector_type(4)));
typedef float v4f __attribute__((ext_vector_type(4)));

template <int DT>
__device__ __forceinline__ v4f mfma16(uint2 a, uint2 b, v4f c) {
  if constexpr (DT == SUBSPEC_BF16) {
    return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(v4s, a), __builtin_bit_cast(v4s, b), c, 0, 0, 0);
  } else {
    return __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(v4h, a), __builtin_bit_cast(v4h, b), c, 0, 0, 0);
  }
}

template <int DT>
__device__ __forceinline__ uint32_t pack2(float lo, float hi) {
  if constexpr (DT == SUBSPEC_BF16) {
    return (__float_as_uint(round_bf16(lo)) >> 16) | (__float_as_uint(round_bf16(hi)) & 0xffff0000u);
  } else {
    union { _Float16 h[2]; uint32_t u; } c;
    c.h[0] = (_Float16)lo;
    c.h[1] = (_Float16)hi;
    return c.u;
  }
}

struct AttnParams {
  int64_t batch, hq, hkv, n_rows, n_slots, seq_stride, prefix, anc_batch_stride;
  int chunks;
  int64_t chunk_keys;          // multiple of kKeyBlock
  float scale_log2;            // softmax scale * log2(e)
};

template <int DT>
__global__ __launch_bounds__(kAttnThreads) void tree_attention_kernel(
    const uint16_t* __restrict__ q, const uint16_t* __restrict__ kc, const uint16_t* __restrict__ vc,
    const uint64_t* __restrict__ anc, AttnParams ap, uint16_t* __restrict__ out, float* __restrict__ part_o,
    float* __restrict__ part_ml) {
  __shared__ __attribute__((aligned(16))) uint16_t Ks[kKeyBlock * kKStride];
  __shared__ __attribute__((aligned(16))) uint16_t Vt[kAttnD * kVStride];

  const int chunk = blockIdx.x;
  const int bh = blockIdx.y;                           // b * hq + qh
  const int b = bh / (int)ap.hq, qh = bh % (int)ap.hq;
  const int kvh = qh / (int)(ap.hq / ap.hkv);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int lq = lane & 15, lg = lane >> 4;            // query column of the lane, lane group
  const int n = (int)ap.n_rows;
  const int64_t kv_len = ap.prefix + ap.n_slots;
  const int row = wave * 16 + lq;                      // query row of this lane
  const bool row_ok = row < n;

  // ---- Q^T operands: Q[row][16*ks + 4*lg .. +3]
  uint2 qreg[kAttnD / 16];
  {
    const uint16_t* qp = q + ((int64_t)bh * n + (row_ok ? row : 0)) * kAttnD;
#pragma unroll
    for (int ks = 0; ks < kAttnD / 16; ++ks) {
      qreg[ks] = row_ok ? *(const uint2*)(qp + ks * 16 + lg * 4) : make_uint2(0, 0);
    }
  }
  const uint64_t bits = row_ok ? anc[(int64_t)b * ap.anc_batch_stride + row] : 0ull;

  v4f oacc[kAttnD / 16];
#pragma unroll
  for (int mt = 0; mt < kAttnD / 16; ++mt) oacc[mt] = v4f{0.f, 0.f, 0.f, 0.f};
  float m_run = -INFINITY, l_run = 0.f;

  const uint16_t* kbase = kc + ((int64_t)b * ap.hkv + kvh) * ap.seq_stride * kAttnD;
  const uint16_t* vbase = vc + ((int64_t)b * ap.hkv + kvh) * ap.seq_stride * kAttnD;
  const int64_t key0 = (int64_t)chunk * ap.chunk_keys;
  const int64_t key1 = min(key0 + ap.chunk_keys, kv_len);

  for (int64_t kb = key0; kb < key1; kb += kKeyBlock) {
    // ---- stage K (row-major) and V (transposed) of this 64-key block
    __syncthreads();
#pragma unroll
    for (int it = 0; it < 4; ++it) {
      const int key = it * 16 + (tid >> 4), dc = tid & 15;
      const int64_t pos = min(kb + key, kv_len - 1);
      const uint4 kv = *(const uint4*)(kbase + pos * kAttnD + dc * 8);
      *(uint4*)(Ks + key * kKStride + dc * 8) = kv;
    }
#pragma unroll
    for (int it = 0; it < 4; ++it) {
      const int key = tid & 63, dg = it * 4 + (tid >> 6);
      const int64_t pos = min(kb + key, kv_len - 1);
      const uint4 vv = *(const uint4*)(vbase + pos * kAttnD + dg * 8);
      const uint32_t w[4] = {vv.x, vv.y, vv.z, vv.w};
#pragma unroll
      for (int e = 0; e < 8; ++e)
        Vt[(dg * 8 + e) * kVStride + key] = (uint16_t)((e & 1) ? (w[e >> 1] >> 16) : (w[e >> 1] & 0xffffu));
    }
    __syncthreads();

    // ---- S^T tiles: 4 x (16 keys x 16 queries); lane holds keys 16*kt + 4*lg + r of query lq
    float s[4][4];
    float mloc = -INFINITY;
#pragma unroll
    for (int kt = 0; kt < 4; ++kt) {
      v4f acc = v4f{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < kAttnD / 16; ++ks) {
        const uint2 a = *(const uint2*)(Ks + (kt * 16 + lq) * kKStride + ks * 16 + lg * 4);
        acc = mfma16<DT>(a, qreg[ks], acc);
      }
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int64_t pos = kb + kt * 16 + lg * 4 + r;
        bool ok = pos < kv_len;
        if (pos >= ap.prefix) ok = ok && ((bits >> (int)(pos - ap.prefix)) & 1ull);
        const float t = ok ? acc[r] * ap.scale_log2 : -INFINITY;
        s[kt][r] = t;
        mloc = fmaxf(mloc, t);
      }
    }
    mloc = fmaxf(mloc, __shfl_xor(mloc, 16, kWave));
    mloc = fmaxf(mloc, __shfl_xor(mloc, 32, kWave));
    const float m_new = fmaxf(m_run, mloc);
    const float m_use = m_new == -INFINITY ? 0.f : m_new;
    const float alpha = __builtin_amdgcn_exp2f(m_run - m_use);      // m_run = -inf -> 0
    m_run = m_new;
    l_run *= alpha;
#pragma unroll
    for (int mt = 0; mt < kAttnD / 16; ++mt) oacc[mt] *= alpha;

    // ---- P^T as B operands, straight from the accumulator layout
    uint2 pb[4];
#pragma unroll
    for (int kt = 0; kt < 4; ++kt) {
      float p[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        p[r] = __builtin_amdgcn_exp2f(s[kt][r] - m_use);
        l_run += p[r];
      }
      pb[kt] = make_uint2(pack2<DT>(p[0], p[1]), pack2<DT>(p[2], p[3]));
    }
    // ---- O^T += V^T P^T : 8 tiles of 16 head-dims
#pragma unroll
    for (int mt = 0; mt < kAttnD / 16; ++mt) {
#pragma unroll
      for (int kt = 0; kt < 4; ++kt) {
        const uint2 a = *(const uint2*)(Vt + (mt * 16 + lq) * kVStride + kt * 16 + lg * 4);
        oacc[mt] = mfma16<DT>(a, pb[kt], oacc[mt]);
      }
    }
  }
  // the four lane groups hold disjoint keys of the same query
  l_run += __shfl_xor(l_run, 16, kWave);
  l_run += __shfl_xor(l_run, 32, kWave);

  if (!row_ok) return;
  if (ap.chunks == 1) {
    const float inv = l_run > 0.f ? 1.0f / l_run : 0.f;
    uint16_t* op = out + (((int64_t)b * n + row) * ap.hq + qh) * kAttnD;
#pragma unroll
    for (int mt = 0; mt < kAttnD / 16; ++mt) {
      const uint2 v = make_uint2(pack2<DT>(oacc[mt][0] * inv, oacc[mt][1] * inv), pack2<DT>(oacc[mt][2] * inv, oacc[mt][3] * inv));
      *(uint2*)(op + mt * 16 + lg * 4) = v;
    }
  } else {
    const int64_t slot = ((int64_t)bh * ap.chunks + chunk) * kAttnRows + row;
    float* po = part_o + slot * kAttnD;
#pragma unroll
    for (int mt = 0; mt < kAttnD / 16; ++mt) *(v4f*)(po + mt * 16 + lg * 4) = oacc[mt];
    if (lg == 0) { part_ml[slot * 2] = m_run; part_ml[slot * 2 + 1] = l_run; }
  }
}

template <int DT>
__global__ __launch_bounds__(kAttnD) void tree_attention_merge_kernel(
    const float* __restrict__ part_o, const float* __restrict__ part_ml, AttnParams ap, uint16_t* __restrict__ out) {
  const int row = blockIdx.x, bh = blockIdx.y;
  const int b = bh / (int)ap.hq, qh = bh % (int)ap.hq;
  const int d = threadIdx.x;
  float m = -INFINITY;
  for (int c = 0; c < ap.chunks; ++c) m = fmaxf(m, part_ml[(((int64_t)bh * ap.chunks + c) * kAttnRows + row) * 2]);
  float num = 0.f, den = 0.f;
  for (int c = 0; c < ap.chunks; ++c) {
    const int64_t slot = ((int64_t)bh * ap.chunks + c) * kAttnRows + row;
    const float mc = part_ml[slot * 2];
    if (mc == -INFINITY) continue;
    const float w = __builtin_amdgcn_exp2f(mc - m);
    num = fmaf(w, part_o[slot * kAttnD + d], num);
    den = fmaf(w, part_ml[slot * 2 + 1], den);
  }
  const float o = den > 0.f ? num / den : 0.f;
  Elem<DT>::store(out, (((int64_t)b * ap.n_rows + row) * ap.hq + qh) * kAttnD + d, o);
}

static int attn_chunks(int64_t batch, int64_t hq, int64_t kv_len) {
  const int64_t blocks = (kv_len + kKeyBlock - 1) / kKeyBlock;
  int64_t chunks = std::max<int64_t>(1, 512 / std::max<int64_t>(1, batch * hq));
  chunks = std::min<int64_t>(chunks, std::max<int64_t>(1, blocks / 2));   // at least 128 keys per chunk
  return (int)std::min<int64_t>(chunks, 64);
}

}  // namespace subspec

using namespace subspec;

extern "C" size_t subspec_tree_attention_workspace(int64_t batch, int64_t n_q_heads, int64_t prefix_len, int64_t n_tree_slots) {
  if (batch <= 0 || n_q_heads <= 0) return 256;
  const int chunks = attn_chunks(batch, n_q_heads, prefix_len + n_tree_slots);
  if (chunks == 1) return 256;
  const size_t slots = (size_t)batch * n_q_heads * chunks * kAttnRows;
  return align_up(slots * kAttnD * sizeof(float), 256) + align_up(slots * 2 * sizeof(float), 256);
}

extern "C" int subspec_tree_attention(const void* q, const void* k_cache, const void* v_cache, void* out, int dtype,
                                      int64_t batch, int64_t n_q_heads, int64_t n_kv_heads, int64_t n_rows,
                                      int64_t n_tree_slots, int64_t head_dim, int64_t kv_seq_stride, int64_t prefix_len,
                                      const uint64_t* anc_bits, int64_t anc_batch_stride, float scale,
                                      void* workspace, size_t workspace_bytes, void* stream) {
  if (dtype != SUBSPEC_BF16 && dtype != SUBSPEC_F16)
    SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "tree_attention: dtype %d not supported (bf16 / fp16 only)", dtype);
  if (!q || !k_cache || !v_cache || !out || !anc_bits) SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "tree_attention: null pointer argument");
  if (head_dim != kAttnD) SUBSPEC_FAIL(SUBSPEC_ERR_LIMIT, "tree_attention: head_dim=%lld (built for 128)", (long long)head_dim);
  if (batch <= 0 || n_q_heads <= 0 || n_kv_heads <= 0 || n_q_heads % n_kv_heads != 0)
    SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "tree_attention: batch=%lld heads=%lld/%lld", (long long)batch, (long long)n_q_heads,
                 (long long)n_kv_heads);
  if (n_rows <= 0 || n_rows > kAttnRows)
    SUBSPEC_FAIL(SUBSPEC_ERR_LIMIT, "tree_attention: n_rows=%lld outside [1, %d]", (long long)n_rows, kAttnRows);
  if (n_tree_slots < 1 || n_tree_slots > 64)
    SUBSPEC_FAIL(SUBSPEC_ERR_LIMIT, "tree_attention: n_tree_slots=%lld outside [1, 64] (one 64-bit mask word per row)",
                 (long long)n_tree_slots);
  if (prefix_len < 0 || prefix_len + n_tree_slots > kv_seq_stride)
    SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "tree_attention: prefix_len=%lld + n_tree_slots=%lld exceeds the cache length %lld",
                 (long long)prefix_len, (long long)n_tree_slots, (long long)kv_seq_stride);
  if (batch * n_q_heads > 65535) SUBSPEC_FAIL(SUBSPEC_ERR_LIMIT, "tree_attention: batch*heads=%lld too large", (long long)(batch * n_q_heads));
  if ((uintptr_t)q % 8 || (uintptr_t)k_cache % 16 || (uintptr_t)v_cache % 16 || (uintptr_t)out % 8)
    SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "tree_attention: q/out must be 8-byte and k/v 16-byte aligned");
  AttnParams ap;
  ap.batch = batch; ap.hq = n_q_heads; ap.hkv = n_kv_heads; ap.n_rows = n_rows; ap.n_slots = n_tree_slots;
  ap.seq_stride = kv_seq_stride;
  ap.prefix = prefix_len; ap.anc_batch_stride = anc_batch_stride;
  const int64_t kv_len = prefix_len + n_tree_slots;
  ap.chunks = attn_chunks(batch, n_q_heads, kv_len);
  const int64_t blocks = (kv_len + kKeyBlock - 1) / kKeyBlock;
  ap.chunk_keys = (blocks + ap.chunks - 1) / ap.chunks * kKeyBlock;
  ap.chunks = (int)((kv_len + ap.chunk_keys - 1) / ap.chunk_keys);
  ap.scale_log2 = scale * kLog2e;
  float* part_o = nullptr;
  float* part_ml = nullptr;
  if (ap.chunks > 1) {
    const size_t slots = (size_t)batch * n_q_heads * ap.chunks * kAttnRows;
    const size_t need = align_up(slots * kAttnD * sizeof(float), 256) + align_up(slots * 2 * sizeof(float), 256);
    if (!workspace || workspace_bytes < need)
      SUBSPEC_FAIL(SUBSPEC_ERR_WORKSPACE, "tree_attention: workspace of %zu bytes is smaller than the %zu required",
                   workspace_bytes, need);
    if ((uintptr_t)workspace % 16) SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "tree_attention: workspace must be 16-byte aligned");
    part_o = (float*)workspace;
    part_ml = (float*)((char*)workspace + align_up(slots * kAttnD * sizeof(float), 256));
  }
  hipStream_t st = (hipStream_t)stream;
  const dim3 grid(ap.chunks, (unsigned)(batch * n_q_heads));
  if (dtype == SUBSPEC_BF16) {
    {
      DominantKernelTimer timer(st);
      hipLaunchKernelGGL((tree_attention_kernel<SUBSPEC_BF16>), grid, dim3(kAttnThreads), 0, st, (const uint16_t*)q,
                         (const uint16_t*)k_cache, (const uint16_t*)v_cache, anc_bits, ap, (uint16_t*)out, part_o, part_ml);
    }
    if (ap.chunks > 1)
      hipLaunchKernelGGL((tree_attention_merge_kernel<SUBSPEC_BF16>), dim3((unsigned)n_rows, (unsigned)(batch * n_q_heads)),
                         dim3(kAttnD), 0, st, part_o, part_ml, ap, (uint16_t*)out);
  } else {
    {
      DominantKernelTimer timer(st);
      hipLaunchKernelGGL((tree_attention_kernel<SUBSPEC_F16>), grid, dim3(kAttnThreads), 0, st, (const uint16_t*)q,
                         (const uint16_t*)k_cache, (const uint16_t*)v_cache, anc_bits, ap, (uint16_t*)out, part_o, part_ml);
    }
    if (ap.chunks > 1)
      hipLaunchKernelGGL((tree_attention_merge_kernel<SUBSPEC_F16>), dim3((unsigned)n_rows, (unsigned)(batch * n_q_heads)),
                         dim3(kAttnD), 0, st, part_o, part_ml, ap, (uint16_t*)out);
  }
  SUBSPEC_CHECK_HIP(hipGetLastError());
  return SUBSPEC_OK;
}
