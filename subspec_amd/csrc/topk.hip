// Top-k draft-tree expansion for gfx950: global top-k over (leaves x vocab) of
// round(p[l, v] * parent_prob[l]) with the canonical tie rule (value descending, flat index
// ascending), fused into one pass over the probabilities.
//
// Follows DraftModelBase.topk_sampling / _topk_flatten
// (specdecodes/models/draft_models/base.py:268-305): buf = sampled_probs * parent_probs[..., None]
// rounded to the tensor dtype; topk(buf.view(B, L*V), min(k, V), sorted=True); token = idx % V,
// parent = idx // V.  torch.topk leaves the order of equal values unspecified; this kernel fixes it
// to the lowest flat index first.
//
//   1. topk_slice_kernel - grid (slices, B*L), 512 threads.  A workgroup streams its slice of one
//      row once.  A lower bound of the slice's k-th best is taken from the per-thread maxima of a
//      sample of the first U tiles of every thread; 16-bit rows are then screened eight elements at a time with packed
//      unsigned maxima against the bit pattern of that bound, and the few survivors go to a
//      candidate list in LDS.  Two checkpoints tighten the bound to the exact k-th best so far; at
//      the end the list is pruned to the slice's exact top-k in (key, index) order.
//      HBM-bound: algorithmic bytes = B * L * V * sizeof(dtype).
//   2. topk_merge_kernel - one workgroup per batch item ranks the <= slices*L*k candidates and
//      writes values, token ids and parent indices in sorted order.
#include "common.h"
#include <algorithm>

namespace subspec {

constexpr int kTopkThreads = 512;
constexpr int kTopkCap = 1024;          // candidate slots per workgroup
constexpr int kTopkPruneAt = 512;       // careful mode prunes above this; one step adds at most 512
constexpr int kTopkMaxK = 64;
constexpr int kTopkMaxSlices = 64;
constexpr int kMergeThreads = 1024;
constexpr int kMergeCap = 4096;

// (key, flat index) as one integer that sorts like "larger key first, then smaller index first"
__device__ __forceinline__ uint64_t pack_candidate(float key, uint32_t flat) {
  uint32_t b = __float_as_uint(key);
  b ^= (b & 0x80000000u) ? 0xffffffffu : 0x80000000u;
  return ((uint64_t)b << 32) | (uint64_t)(0xffffffffu - flat);
}
__device__ __forceinline__ float candidate_key(uint64_t c) {
  uint32_t b = (uint32_t)(c >> 32);
  b ^= (b & 0x80000000u) ? 0x80000000u : 0xffffffffu;
  return __uint_as_float(b);
}
__device__ __forceinline__ uint32_t candidate_flat(uint64_t c) { return 0xffffffffu - (uint32_t)c; }

typedef unsigned short u16x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pk_max_u16(uint32_t a, uint32_t b) {
  return __builtin_bit_cast(uint32_t, __builtin_elementwise_max(__builtin_bit_cast(u16x2_t, a), __builtin_bit_cast(u16x2_t, b)));
}

// Smallest non-negative 16-bit pattern u whose key round(value(u) * q) reaches tau_key.  Keys
// grow with u for q > 0, so "key >= tau_key" can be tested on the raw bits with an unsigned
// compare; patterns with the sign bit set compare high and are sorted out by the precise test.
template <int DT>
__device__ __forceinline__ bool pattern_reaches(uint32_t u, float q, float tau_key) {
  const float v = DT == SUBSPEC_BF16 ? bf16_bits_to_float(u) : f16_bits_to_float(u);
  return Elem<DT>::round(v * q) >= tau_key;
}
template <int DT>
__device__ __forceinline__ uint32_t min_pattern_reaching_search(float q, float tau_key) {
  uint32_t lo = 0, hi = DT == SUBSPEC_BF16 ? 0x7f80u : 0x7c00u;     // +inf
  while (lo < hi) {
    const uint32_t mid = (lo + hi) >> 1;
    if (pattern_reaches<DT>(mid, q, tau_key)) hi = mid; else lo = mid + 1;
  }
  return lo;
}
// The answer lies next to the pattern of tau_key / q: start just above it and walk down while the pattern below still
// reaches (a few dependent steps instead of the fifteen of a bisection, which every workgroup would pay three times
// on its critical path).  Whatever the walk returns satisfies "reaches, and the pattern below does not", which
// with monotone keys IS the minimum; anything unexpected falls back to the bisection.
template <int DT>
__device__ __forceinline__ uint32_t min_pattern_reaching(float q, float tau_key) {
  if (!(q > 0.f)) return 0;
  if (!(tau_key > 0.f)) return 0;                      // every non-negative pattern reaches
  constexpr uint32_t kInf = DT == SUBSPEC_BF16 ? 0x7f80u : 0x7c00u;
  const float x = tau_key / q;
  uint32_t u;
  if constexpr (DT == SUBSPEC_BF16) {
    u = (__float_as_uint(x) + 0xffffu) >> 16;          // smallest pattern whose value is >= x (x > 0 or NaN)
  } else {
    union { uint16_t b; _Float16 h; } c;
    c.h = (_Float16)fminf(x, 65504.f);
    u = (uint32_t)c.b + 1;
  }
  u = min(u + 1, kInf);
  if (!pattern_reaches<DT>(u, q, tau_key)) return min_pattern_reaching_search<DT>(q, tau_key);
  for (int step = 0; step < 6; ++step) {
    if (u == 0 || !pattern_reaches<DT>(u - 1, q, tau_key)) return u;
    --u;
  }
  return min_pattern_reaching_search<DT>(q, tau_key);
}

template <int DT, int VEC> struct PTile;
template <> struct PTile<SUBSPEC_F32, 4> {
  float4 r;
  __device__ __forceinline__ void load(const void* p, int64_t i) {
    typedef float f4v __attribute__((ext_vector_type(4)));
    const f4v v = __builtin_nontemporal_load((const f4v*)((const float*)p + i));
    r = make_float4(v.x, v.y, v.z, v.w);
  }
  __device__ __forceinline__ float get(int k) const { return k == 0 ? r.x : k == 1 ? r.y : k == 2 ? r.z : r.w; }
};
template <> struct PTile<SUBSPEC_F32, 1> {
  float r;
  __device__ __forceinline__ void load(const void* p, int64_t i) { r = ((const float*)p)[i]; }
  __device__ __forceinline__ float get(int) const { return r; }
};
template <int DT> struct PTile16x8 {
  uint4 r;
  // streaming (non-temporal) load: every element of the rows is read once, and fetched that way the rows do not
  // displace each other in the L2 on their way through (2048 x 152064 bf16: 109 -> 105 us, 112 -> 103 us)
  __device__ __forceinline__ void load(const void* p, int64_t i) {
    typedef uint32_t u4v __attribute__((ext_vector_type(4)));
    const u4v v = __builtin_nontemporal_load((const u4v*)((const uint16_t*)p + i));
    r = make_uint4(v.x, v.y, v.z, v.w);
  }
  __device__ __forceinline__ float get(int k) const {
    const uint32_t w = (k >> 1) == 0 ? r.x : (k >> 1) == 1 ? r.y : (k >> 1) == 2 ? r.z : r.w;
    if (DT == SUBSPEC_BF16) return (k & 1) ? __uint_as_float(w & 0xffff0000u) : __uint_as_float(w << 16);
    return f16_bits_to_float((k & 1) ? (w >> 16) : (w & 0xffffu));
  }
};
template <> struct PTile<SUBSPEC_BF16, 8> : PTile16x8<SUBSPEC_BF16> {};
template <> struct PTile<SUBSPEC_F16, 8> : PTile16x8<SUBSPEC_F16> {};
template <int DT> struct PTile16x1 {
  uint16_t r;
  __device__ __forceinline__ void load(const void* p, int64_t i) { r = ((const uint16_t*)p)[i]; }
  __device__ __forceinline__ float get(int) const {
    return DT == SUBSPEC_BF16 ? bf16_bits_to_float(r) : f16_bits_to_float(r);
  }
};
template <> struct PTile<SUBSPEC_BF16, 1> : PTile16x1<SUBSPEC_BF16> {};
template <> struct PTile<SUBSPEC_F16, 1> : PTile16x1<SUBSPEC_F16> {};

// k-th best (0-based rank k-1) of `count` packed candidates in LDS by counting; every thread calls.
// Returns 0 (below every candidate) when count < k.  `out` is a one-word LDS scratch.
template <int THREADS>
__device__ uint64_t kth_best(const uint64_t* list, int count, int k, uint64_t* out) {
  if (threadIdx.x == 0) *out = 0;
  __syncthreads();
  for (int i = threadIdx.x; i < count; i += THREADS) {
    const uint64_t mine = list[i];
    int rank = 0;
    for (int j = 0; j < count; ++j) rank += list[j] > mine;
    if (rank == k - 1) *out = mine;                    // packed values are distinct (distinct indices)
  }
  __syncthreads();
  const uint64_t r = *out;
  __syncthreads();
  return r;
}

// Keeps only candidates >= cut (all of them when cut == 0).  Every thread calls.
template <int THREADS>
__device__ int prune_list(uint64_t* list, int count, uint64_t cut, int* counter) {
  uint64_t keep[(kTopkCap + THREADS - 1) / THREADS];
  int nkeep = 0;
#pragma unroll
  for (int s = 0; s < (kTopkCap + THREADS - 1) / THREADS; ++s) {
    const int i = threadIdx.x + s * THREADS;
    keep[s] = 0;
    if (i < count && list[i] >= cut && list[i] != 0) { keep[s] = list[i]; ++nkeep; }
  }
  if (threadIdx.x == 0) *counter = 0;
  __syncthreads();
#pragma unroll
  for (int s = 0; s < (kTopkCap + THREADS - 1) / THREADS; ++s)
    if (keep[s] != 0) list[atomicAdd(counter, 1)] = keep[s];
  __syncthreads();
  (void)nkeep;
  return *counter;
}

template <int DT, int VEC, int U>
__global__ __launch_bounds__(kTopkThreads) __attribute__((amdgpu_waves_per_eu(8, 8))) void topk_slice_kernel(
    const void* __restrict__ probs, const void* __restrict__ parent_probs, int64_t vocab, int leaves, int splits,
    int64_t chunk, int k, uint64_t* __restrict__ cand, int32_t* __restrict__ cand_count,
    int64_t* __restrict__ token_ids, void* __restrict__ topk_probs, int64_t* __restrict__ parent_indices) {
  __shared__ uint64_t list[kTopkCap];
  __shared__ uint64_t kth_slot;
  __shared__ uint32_t wave_prefix[kTopkThreads / kWave];
  __shared__ int count, overflow, tie_total;

  const int64_t row = blockIdx.y;                      // b * leaves + l
  const int c = blockIdx.x;
  const int tid = threadIdx.x;
  const int leaf = (int)(row % leaves);
  const int64_t c0 = (int64_t)c * chunk;
  const int64_t n = min(chunk, vocab - c0);
  const int64_t base = row * vocab + c0;
  const int64_t ntiles = n / VEC;
  const float q = Elem<DT>::load(parent_probs, row);
  const uint32_t flat0 = (uint32_t)((int64_t)leaf * vocab + c0);

  // ---- threshold from a sample: the per-thread maxima over the first U tiles.  Each wavefront
  // finds, by a 16-step bit search with ballots (no memory traffic), the largest 16-bit key prefix
  // that at least m = ceil(k/4) of its lanes reach; the ceil(k/m)-th largest of those prefixes is
  // reached by at least k elements of the slice, hence a valid lower bound for its k-th best.
  // The sample IS the first group of the streaming loop below: its tiles stay in registers
  // and are scanned once the threshold is known, so nothing is read twice.
  // U tiles per thread in flight: 8 for whole rows of a large batch (112 against 117 us at 2048 x 152064 bf16),
  // 4 for the short slices of a draft step, where 8 would mostly re-read the clamped last tile
  PTile<DT, VEC> t[U];
#pragma unroll
  for (int i = 0; i < U; ++i) {                        // unconditional loads (clamped index): back to back
    const int64_t j = min((int64_t)i * kTopkThreads + tid, ntiles - 1);
    t[i].load(probs, base + j * VEC);
  }
  float smax = -INFINITY;
  bool sany = false;
#pragma unroll
  for (int i = 0; i < U; ++i) {
    const int64_t j = tid + (int64_t)i * kTopkThreads;
    if (j < ntiles) {
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        const float key = Elem<DT>::round(t[i].get(e) * q);
        if (!sany || key > smax) { smax = key; sany = true; }
      }
    }
  }
  if (tid == 0) { count = 0; overflow = 0; tie_total = 0; }
  {
    const int m = (k + 3) / 4;
    const uint32_t prefix = sany ? (uint32_t)(pack_candidate(smax, 0) >> 48) : 0u;
    uint32_t best = 0;
    for (int bit = 15; bit >= 0; --bit) {
      const uint32_t trial = best | (1u << bit);
      if (__popcll(__ballot(prefix >= trial)) >= m) best = trial;
    }
    if ((tid & (kWave - 1)) == 0) wave_prefix[tid / kWave] = best;
  }
  __syncthreads();
  uint64_t tau;
  {
    const int m = (k + 3) / 4, need = (k + m - 1) / m;            // need <= 4 wavefronts
    uint32_t chosen = 0;                               // the prefix of rank need-1 among the 8
    for (int w = 0; w < kTopkThreads / kWave; ++w) {
      int r = 0;
      const uint32_t o = wave_prefix[w];
      for (int w2 = 0; w2 < kTopkThreads / kWave; ++w2) r += (wave_prefix[w2] > o) || (wave_prefix[w2] == o && w2 < w);
      if (r == need - 1) chosen = o;
    }
    tau = (uint64_t)chosen << 48;
  }
  float tau_key = tau ? candidate_key(tau) : -INFINITY;

  // ---- stream the slice; survivors go to the LDS list
  // Ties.  The bound is reached by at least k elements of the SAMPLE (the first U tiles of every thread, i.e. the
  // lowest indices of the slice).  An element of a later group whose key only EQUALS the bound has a higher index than
  // all of them and can never be among the best k, so later groups are screened strictly.  Inside the sample, when
  // more than kTieLimit elements equal the bound (rows that are mostly one value: zeros under a low temperature,
  // uniform rows), only the k of them with the lowest indices are taken, in index order; appending them all would
  // overflow the list and send the workgroup through the slow one-element-per-step path.
  constexpr int kTieLimit = 256;
  const int64_t ngroups = (ntiles + kTopkThreads - 1) / kTopkThreads;
  // Flood test: in how many threads does the sample's maximum merely EQUAL the bound?  In a row that is mostly one
  // value that is nearly all of them; a wrong "yes" only costs speed (the plain loop below is exact for any row).
  if (tau != 0) {
    const int n_eq = __popcll(__ballot(sany && smax == tau_key));
    if ((tid & (kWave - 1)) == 0 && n_eq) atomicAdd(&tie_total, n_eq);
    __syncthreads();
  }
  const bool tie_flood = tau != 0 && tie_total > kTieLimit;       // uniform
  const float tie_key = tau_key;                       // the first bound: the ties pass after the loop is about this one
  auto scan_tile = [&](const PTile<DT, VEC>& t, int64_t j, float bound) {    // bound: tau_key, or the next float up
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
      const float key = Elem<DT>::round(t.get(e) * q);
      if (key >= bound) {
        const uint64_t pc = pack_candidate(key, flat0 + (uint32_t)(j * VEC + e));
        if (pc >= tau) {
          const int slot = atomicAdd(&count, 1);
          if (slot < kTopkCap) list[slot] = pc; else overflow = 1;
        }
      }
    }
  };
  // fast path: U tiles per thread in flight, no bookkeeping between groups.  For 16-bit rows a
  // tile is first screened with packed unsigned maxima against the bit pattern of the threshold
  // (five instructions for eight elements); only tiles that may hold a survivor are unpacked.
  uint32_t screen = 0, screen_strict = 0;              // (pattern - 1) in both halves; 0: screen nothing out
  float tau_key_up = tau_key;                          // the next float above the bound: "key > bound" as "key >= this"
  auto set_screens = [&]() {
    tau_key_up = tau ? nextafterf(tau_key, INFINITY) : tau_key;
    if constexpr (VEC == 8) {
      const uint32_t thr = min_pattern_reaching<DT>(q, tau_key);
      screen = thr ? (thr - 1) * 0x10001u : 0;
      const uint32_t thr2 = tau ? min_pattern_reaching<DT>(q, tau_key_up) : 0;
      screen_strict = thr2 ? (thr2 - 1) * 0x10001u : 0;
    }
  };
  set_screens();
  auto tile_may_reach = [&](const PTile<DT, VEC>& t, uint32_t scr) {
    if constexpr (VEC == 8) {
      const uint32_t mm = pk_max_u16(pk_max_u16(t.r.x, t.r.y), pk_max_u16(t.r.z, t.r.w));
      return scr == 0 || pk_max_u16(mm, scr) != scr;
    } else {
      return true;
    }
  };
  for (int64_t g0 = 0; g0 < ngroups; g0 += U) {
    if (g0 > 0) {                                      // group 0 is already in registers (the sample)
#pragma unroll
      for (int i = 0; i < U; ++i) {                    // unconditional loads (clamped index): back to back
        const int64_t j = min((g0 + i) * kTopkThreads + tid, ntiles - 1);
        t[i].load(probs, base + j * VEC);
      }
    }
    const bool strict = tau != 0 && (g0 > 0 || tie_flood);        // uniform
    const uint32_t scr = strict ? screen_strict : screen;
    const float bound = strict ? tau_key_up : tau_key;
#pragma unroll
    for (int i = 0; i < U; ++i) {
      const int64_t j = (g0 + i) * kTopkThreads + tid;
      if (j < ntiles && tile_may_reach(t[i], scr)) scan_tile(t[i], j, bound);
    }
    // two checkpoints tighten the threshold to the exact k-th best of what has been seen, so that
    // few later elements survive and the final selection stays small
    if ((g0 == U || g0 == 4 * U) && g0 + U < ngroups) {
      __syncthreads();
      const int cnt = count;
      const int lost = overflow;
      __syncthreads();
      if (!lost && cnt > k) {
        tau = kth_best<kTopkThreads>(list, cnt, k, &kth_slot);
        tau_key = candidate_key(tau);
        prune_list<kTopkThreads>(list, cnt, tau, &count);
        set_screens();
      }
    }
  }
  if (tie_flood) {                                     // workgroup-uniform
    // The sample was screened strictly; now the k lowest-index elements of it that EQUAL the first bound, tile row by
    // tile row (ranks from a prefix sum over the workgroup).  The tiles are loaded again, one at a time (they are in
    // L2), so that the streaming loop above keeps its registers.  If the bound has been tightened since, these are
    // below the cut and the final selection drops them.
    int taken = 0;                                     // uniform
#pragma unroll 1
    for (int i = 0; i < U && taken < k; ++i) {
      const int64_t j = tid + (int64_t)i * kTopkThreads;
      PTile<DT, VEC> tt;
      tt.load(probs, base + min(j, ntiles - 1) * VEC);
      int eq = 0;
      if (j < ntiles) {
#pragma unroll
        for (int e = 0; e < VEC; ++e) eq += Elem<DT>::round(tt.get(e) * q) == tie_key;
      }
      int incl = eq;                                   // inclusive prefix inside the wavefront
#pragma unroll
      for (int o = 1; o < kWave; o <<= 1) {
        const int up = __shfl_up(incl, o, kWave);
        if ((tid & (kWave - 1)) >= o) incl += up;
      }
      __syncthreads();                                 // wave_prefix is free (the bound has been read)
      if ((tid & (kWave - 1)) == kWave - 1) wave_prefix[tid / kWave] = (uint32_t)incl;
      __syncthreads();
      int before = 0, total = 0;
      for (int w = 0; w < kTopkThreads / kWave; ++w) {
        if (w < tid / kWave) before += (int)wave_prefix[w];
        total += (int)wave_prefix[w];
      }
      int rank = taken + before + incl - eq;           // rank of this thread's first equal element
      if (eq && rank < k) {
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
          if (Elem<DT>::round(tt.get(e) * q) == tie_key) {
            if (rank < k) {
              const int slot = atomicAdd(&count, 1);
              if (slot < kTopkCap) list[slot] = pack_candidate(tie_key, flat0 + (uint32_t)(j * VEC + e)); else overflow = 1;
            }
            ++rank;
          }
        }
      }
      taken += total;
    }
  }
  __syncthreads();
  if (overflow) {                                      // workgroup-uniform
    // too many survivors for the list (heavy ties or adversarial order): start over, one group
    // at a time, pruning to the best k whenever fewer than a group's worth of slots remain, so
    // that nothing is ever dropped
    __syncthreads();
    if (tid == 0) { count = 0; overflow = 0; }
    __syncthreads();
    for (int64_t g = 0; g < ngroups; ++g) {
      const int64_t j = g * kTopkThreads + tid;
      PTile<DT, VEC> t;
      if (j < ntiles) t.load(probs, base + j * VEC);
      for (int e = 0; e < VEC; ++e) {                  // one element per thread and step: <= 512 appends
        if (j < ntiles) {
          float v = t.get(0);
#pragma unroll
          for (int e2 = 1; e2 < VEC; ++e2) v = (e == e2) ? t.get(e2) : v;
          const float key = Elem<DT>::round(v * q);
          if (key >= tau_key) {
            const uint64_t pc = pack_candidate(key, flat0 + (uint32_t)(j * VEC + e));
            if (pc >= tau) list[atomicAdd(&count, 1)] = pc;
          }
        }
        __syncthreads();
        const int cnt = count;
        __syncthreads();                               // nobody appends before everyone has read it
        if (cnt > kTopkPruneAt) {
          tau = kth_best<kTopkThreads>(list, cnt, k, &kth_slot);
          tau_key = candidate_key(tau);
          prune_list<kTopkThreads>(list, cnt, tau, &count);
        }
      }
    }
    __syncthreads();
  }

  // ---- exact top-k of the slice in (key, index) order
  int cnt = min(count, kTopkCap);
  tau = kth_best<kTopkThreads>(list, cnt, k, &kth_slot);
  cnt = prune_list<kTopkThreads>(list, cnt, tau, &count);
  if (leaves * splits == 1) {
    // this workgroup has seen the whole output row: rank the (distinct) candidates and write the
    // result directly, no merge launch
    __syncthreads();
    for (int i = tid; i < cnt; i += kTopkThreads) {
      const uint64_t mine = list[i];
      int rank = 0;
      for (int j = 0; j < cnt; ++j) rank += list[j] > mine;
      if (rank < k) {
        const uint32_t flat = candidate_flat(mine);
        token_ids[row * k + rank] = flat % vocab;
        parent_indices[row * k + rank] = flat / vocab;
        Elem<DT>::store(topk_probs, row * k + rank, candidate_key(mine));
      }
    }
    return;
  }
  const int64_t slot0 = (row * splits + c) * kTopkMaxK;
  for (int i = tid; i < cnt; i += kTopkThreads) cand[slot0 + i] = list[i];
  if (tid == 0) cand_count[row * splits + c] = cnt;
}

template <int DT>
__global__ __launch_bounds__(kMergeThreads) void topk_merge_kernel(
    const uint64_t* __restrict__ cand, const int32_t* __restrict__ cand_count, int64_t vocab, int leaves, int splits,
    int k, int64_t* __restrict__ token_ids, void* __restrict__ topk_probs, int64_t* __restrict__ parent_indices) {
  __shared__ uint64_t list[kMergeCap];
  __shared__ int total;
  const int b = blockIdx.x;
  if (threadIdx.x == 0) total = 0;
  __syncthreads();
  const int lists = leaves * splits;
  for (int s = threadIdx.x; s < lists * kTopkMaxK; s += kMergeThreads) {
    const int li = s / kTopkMaxK, i = s % kTopkMaxK;
    const int64_t g = (int64_t)b * lists + li;
    if (i < cand_count[g]) list[atomicAdd(&total, 1)] = cand[g * kTopkMaxK + i];
  }
  __syncthreads();
  const int cnt = total;
  for (int i = threadIdx.x; i < cnt; i += kMergeThreads) {
    const uint64_t mine = list[i];
    int rank = 0;
    for (int j = 0; j < cnt; ++j) rank += list[j] > mine;
    if (rank < k) {
      const uint32_t flat = candidate_flat(mine);
      token_ids[(int64_t)b * k + rank] = flat % vocab;
      parent_indices[(int64_t)b * k + rank] = flat / vocab;
      Elem<DT>::store(topk_probs, (int64_t)b * k + rank, candidate_key(mine));
    }
  }
}

struct TopkPlan { int vec, splits; int64_t chunk; };

static bool topk_plan(const void* probs, int dtype, int64_t rows, int64_t vocab, int k, int leaves, TopkPlan* pl) {
  const int vec_full = dtype == SUBSPEC_F32 ? 4 : 8;
  const bool aligned = (vocab % vec_full == 0) && ((uintptr_t)probs % 16 == 0);
  pl->vec = aligned ? vec_full : 1;
  const int64_t quantum = (int64_t)kTopkThreads * pl->vec;
  int64_t splits = (1024 + rows - 1) / rows;
  splits = std::min<int64_t>(splits, std::max<int64_t>(1, vocab / 16384));
  splits = std::min<int64_t>(splits, std::max<int64_t>(1, kMergeCap / ((int64_t)leaves * k)));
  splits = std::max<int64_t>(1, std::min<int64_t>(splits, kTopkMaxSlices));
  int64_t chunk = (vocab + splits - 1) / splits;
  chunk = (chunk + quantum - 1) / quantum * quantum;
  splits = (vocab + chunk - 1) / chunk;
  pl->splits = (int)splits;
  pl->chunk = chunk;
  return (int64_t)leaves * splits * k <= kMergeCap;
}

template <int DT>
static int run_topk(const void* probs, const void* parent_probs, int64_t batch, int leaves, int64_t vocab, int k,
                    const TopkPlan& pl, uint64_t* cand, int32_t* cand_count, int64_t* token_ids, void* topk_probs,
                    int64_t* parent_indices, hipStream_t st) {
  const dim3 grid(pl.splits, (unsigned)(batch * leaves));
  {
    DominantKernelTimer timer(st);
    constexpr int kVecFull = DT == SUBSPEC_F32 ? 4 : 8;
    if (pl.vec == 1)
      hipLaunchKernelGGL((topk_slice_kernel<DT, 1, 4>), grid, dim3(kTopkThreads), 0, st, probs, parent_probs, vocab, leaves,
                         pl.splits, pl.chunk, k, cand, cand_count, token_ids, topk_probs, parent_indices);
    else if (pl.chunk / kVecFull >= 2 * (int64_t)kTopkThreads * 8)
      hipLaunchKernelGGL((topk_slice_kernel<DT, kVecFull, 8>), grid, dim3(kTopkThreads), 0, st, probs,
                         parent_probs, vocab, leaves, pl.splits, pl.chunk, k, cand, cand_count, token_ids, topk_probs,
                         parent_indices);
    else
      hipLaunchKernelGGL((topk_slice_kernel<DT, kVecFull, 4>), grid, dim3(kTopkThreads), 0, st, probs,
                         parent_probs, vocab, leaves, pl.splits, pl.chunk, k, cand, cand_count, token_ids, topk_probs,
                         parent_indices);
  }
  if (leaves * pl.splits > 1)
    hipLaunchKernelGGL((topk_merge_kernel<DT>), dim3((unsigned)batch), dim3(kMergeThreads), 0, st, cand, cand_count,
                     vocab, leaves, pl.splits, k, token_ids, topk_probs, parent_indices);
  SUBSPEC_CHECK_HIP(hipGetLastError());
  return SUBSPEC_OK;
}

}  // namespace subspec

using namespace subspec;

extern "C" size_t subspec_topk_expand_workspace(int64_t batch, int64_t leaves, int64_t vocab, int32_t k) {
  (void)vocab; (void)k;
  if (batch <= 0 || leaves <= 0) return 256;
  const size_t lists = (size_t)batch * leaves * kTopkMaxSlices;
  return align_up(lists * kTopkMaxK * sizeof(uint64_t), 256) + align_up(lists * sizeof(int32_t), 256);
}

extern "C" int subspec_topk_expand(const void* probs, const void* parent_probs, int dtype, int64_t batch,
                                   int64_t leaves, int64_t vocab, int32_t k, void* workspace, size_t workspace_bytes,
                                   int64_t* token_ids, void* topk_probs, int64_t* parent_indices, void* stream) {
  if (!dtype_ok(dtype)) SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "topk_expand: unknown dtype %d", dtype);
  if (!probs || !parent_probs || !workspace || !token_ids || !topk_probs || !parent_indices)
    SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "topk_expand: null pointer argument");
  if (batch <= 0 || leaves <= 0 || vocab <= 0 || k <= 0)
    SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "topk_expand: batch=%lld leaves=%lld vocab=%lld k=%d must be positive",
                 (long long)batch, (long long)leaves, (long long)vocab, k);
  if (k > vocab) SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "topk_expand: k=%d exceeds vocab=%lld (clamp k on the host)", k, (long long)vocab);
  if (k > kTopkMaxK) SUBSPEC_FAIL(SUBSPEC_ERR_LIMIT, "topk_expand: k=%d exceeds the limit of %d", k, kTopkMaxK);
  if (leaves * vocab >= ((int64_t)1 << 32) || batch * leaves > 65535)
    SUBSPEC_FAIL(SUBSPEC_ERR_LIMIT, "topk_expand: leaves*vocab=%lld or batch*leaves=%lld too large",
                 (long long)(leaves * vocab), (long long)(batch * leaves));
  if (workspace_bytes < subspec_topk_expand_workspace(batch, leaves, vocab, k))
    SUBSPEC_FAIL(SUBSPEC_ERR_WORKSPACE, "topk_expand: workspace of %zu bytes is smaller than the %zu required",
                 workspace_bytes, subspec_topk_expand_workspace(batch, leaves, vocab, k));
  if ((uintptr_t)workspace % 16 != 0) SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "topk_expand: workspace must be 16-byte aligned");
  if ((uintptr_t)probs % dtype_size(dtype) != 0 || (uintptr_t)parent_probs % dtype_size(dtype) != 0)
    SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "topk_expand: misaligned input");
  TopkPlan pl;
  if (!topk_plan(probs, dtype, batch * leaves, vocab, k, (int)leaves, &pl))
    SUBSPEC_FAIL(SUBSPEC_ERR_LIMIT, "topk_expand: leaves=%lld x k=%d candidates exceed the merge capacity",
                 (long long)leaves, k);
  const size_t lists = (size_t)batch * leaves * kTopkMaxSlices;
  uint64_t* cand = (uint64_t*)workspace;
  int32_t* cand_count = (int32_t*)((char*)workspace + align_up(lists * kTopkMaxK * sizeof(uint64_t), 256));
  hipStream_t st = (hipStream_t)stream;
  switch (dtype) {
    case SUBSPEC_F32:
      return run_topk<SUBSPEC_F32>(probs, parent_probs, batch, (int)leaves, vocab, k, pl, cand, cand_count, token_ids,
                                   topk_probs, parent_indices, st);
    case SUBSPEC_F16:
      return run_topk<SUBSPEC_F16>(probs, parent_probs, batch, (int)leaves, vocab, k, pl, cand, cand_count, token_ids,
                                   topk_probs, parent_indices, st);
    default:
      return run_topk<SUBSPEC_BF16>(probs, parent_probs, batch, (int)leaves, vocab, k, pl, cand, cand_count,
                                    token_ids, topk_probs, parent_indices, st);
  }
}
