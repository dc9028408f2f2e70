// Fused tree verification for gfx950.
//
// Launch sequence (all on the caller's stream, no host synchronisation):
//   1. row_partial_kernel  - grid (slices, batch*rows), 512 threads.  A workgroup streams its
//      slice of one logits row with 16-byte loads, several per thread in flight, and reduces it in
//      a single pass to (sum exp, sum t*exp, max, first index of the max); the row is read from
//      HBM exactly once.  HBM-bound: algorithmic bytes = rows * vocab * sizeof(dtype).
//   2. exact pass          - only for rows that need the reference's per-element rounding
//      (entropy within the guard band of the threshold, fp16 rows, or a possible tie between
//      *rounded* probabilities at the row maximum): run by the same workgroup right after step 1
//      when a row is one slice (always, for a greedy target), otherwise by row_exact_kernel (same
//      grid, exits at once for rows that do not need it; rows are cut into slices for a sampling target).
//   3. tree_accept_kernel  - one workgroup per tree: combines the partials, gathers
//      p[parent(i), token(i)], runs the greedy walk or the bottom-up DP on the <= 512 nodes in LDS
//      and writes the accepted path, contexts and bonus token.
//
// Sampling target (do_sample=True): the rows are first warped as TemperatureLogitsWarper does
// (x / T rounded to the row dtype), steps 1-2 run on the warped values, and row_sample_kernel
// draws one token per row from the rounded probabilities by an exponential race,
// argmax_i p_i / E_i with E_i = -log(u_i) and u_i from Philox4x32-10 keyed by the caller's seed
// (the formulation torch.multinomial uses for one sample); the walk / DP of step 3 then uses the
// drawn token where the greedy target uses the argmax (classic_sd.py:111-116,
// lossy_tree_verify.py:75-77).
//
// Semantics follow the reference's verify_tree / lossy_bottom_up_verify
// (specdecodes/models/utils/tree_verify.py:49-163, lossy_tree_verify.py:66-168,247-291):
// argmax is the FIRST index whose probability, rounded to the logits dtype, equals the rounded
// row maximum; the normalized entropy of a 16-bit row is sum(entr(p)) with p, log p and p*log p
// each rounded to that dtype, the sum rounded once, divided by float(ln V) and rounded again.
#include "common.h"
#include <mutex>
#include <algorithm>

namespace subspec {

constexpr int kRowThreads = 512;
constexpr int kMaxSplits = 64;
constexpr int kTailThreads = 64;

// per (row, slice): reference point of the exponentials, sum exp2(t), sum t*exp2(t) with
// t = (x - ref) * log2(e), true maximum of the slice and the first index holding it
struct Part1 { float ref; float s; float u; float m; int32_t idx; int32_t pad[3]; };
struct Part2 { float esum; int32_t tie_idx; };
struct Part3 { float key; int32_t idx; };             // best race key of a slice and its first index

// ------------------------------------------------------------------ packed register tiles
template <int DT, int VEC> struct Tile;
template <> struct Tile<SUBSPEC_F32, 4> {
  float4 r;
  __device__ __forceinline__ void load(const void* p, int64_t i) {
    typedef float f4v __attribute__((ext_vector_type(4)));
    const f4v v = __builtin_nontemporal_load((const f4v*)((const float*)p + i));
    r = make_float4(v.x, v.y, v.z, v.w);
  }
  __device__ __forceinline__ void load_cached(const void* p, int64_t i) { r = *(const float4*)((const float*)p + i); }
  __device__ __forceinline__ void fill_neg_inf() { r = make_float4(-INFINITY, -INFINITY, -INFINITY, -INFINITY); }
  __device__ __forceinline__ float get(int k) const { return k == 0 ? r.x : k == 1 ? r.y : k == 2 ? r.z : r.w; }
  __device__ __forceinline__ void fence() { asm volatile("" : "+v"(r.x), "+v"(r.y), "+v"(r.z), "+v"(r.w)); }
};
template <> struct Tile<SUBSPEC_F32, 1> {
  float r;
  __device__ __forceinline__ void load(const void* p, int64_t i) { r = ((const float*)p)[i]; }
  __device__ __forceinline__ void load_cached(const void* p, int64_t i) { load(p, i); }
  __device__ __forceinline__ void fill_neg_inf() { r = -INFINITY; }
  __device__ __forceinline__ float get(int) const { return r; }
  __device__ __forceinline__ void fence() { asm volatile("" : "+v"(r)); }
};
template <int DT> struct Tile16x8 {
  uint4 r;
  // streaming (non-temporal) load: every element of the rows is read once, and fetched that way the rows do not
  // displace each other in the L2 on their way through (2048 x 152064 bf16: 109 -> 105 us, 112 -> 103 us)
  __device__ __forceinline__ void load(const void* p, int64_t i) {
    typedef uint32_t u4v __attribute__((ext_vector_type(4)));
    const u4v v = __builtin_nontemporal_load((const u4v*)((const uint16_t*)p + i));
    r = make_uint4(v.x, v.y, v.z, v.w);
  }
  // ordinary load, for a tile that is read again soon (the reference tile of a slice)
  __device__ __forceinline__ void load_cached(const void* p, int64_t i) { r = *(const uint4*)((const uint16_t*)p + i); }
  __device__ __forceinline__ void fill_neg_inf() {
    const uint32_t w = DT == SUBSPEC_BF16 ? 0xff80ff80u : 0xfc00fc00u;
    r = make_uint4(w, w, w, w);
  }
  __device__ __forceinline__ float get(int k) const {
    const uint32_t w = (k >> 1) == 0 ? r.x : (k >> 1) == 1 ? r.y : (k >> 1) == 2 ? r.z : r.w;
    if (DT == SUBSPEC_BF16) return (k & 1) ? __uint_as_float(w & 0xffff0000u) : __uint_as_float(w << 16);
    return f16_bits_to_float((k & 1) ? (w >> 16) : (w & 0xffffu));
  }
  // Makes the packed registers opaque to the optimiser so that the unpacked floats of one pass
  // are not kept alive for the next one (that would double the register footprint of the slice).
  __device__ __forceinline__ void fence() { asm volatile("" : "+v"(r.x), "+v"(r.y), "+v"(r.z), "+v"(r.w)); }
  // -inf (masked logits) and anything below kFloorBits become a large finite negative, two values per
  // instruction: as unsigned 16-bit patterns the negative floats are ordered by magnitude, so an unsigned
  // minimum with the pattern of the floor leaves positive values alone and pulls -inf up to the floor.
  // bf16: floor -2^100 (its product with log2(e) stays finite in fp32); fp16: the lowest finite value.
  static constexpr uint32_t kFloorBits = DT == SUBSPEC_BF16 ? 0xf180f180u : 0xfbfffbffu;
  __device__ __forceinline__ void floor_neg_inf() {
    typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));
    const u16x2 lim = __builtin_bit_cast(u16x2, kFloorBits);
    r.x = __builtin_bit_cast(uint32_t, __builtin_elementwise_min(__builtin_bit_cast(u16x2, r.x), lim));
    r.y = __builtin_bit_cast(uint32_t, __builtin_elementwise_min(__builtin_bit_cast(u16x2, r.y), lim));
    r.z = __builtin_bit_cast(uint32_t, __builtin_elementwise_min(__builtin_bit_cast(u16x2, r.z), lim));
    r.w = __builtin_bit_cast(uint32_t, __builtin_elementwise_min(__builtin_bit_cast(u16x2, r.w), lim));
  }
};
template <> struct Tile<SUBSPEC_BF16, 8> : Tile16x8<SUBSPEC_BF16> {};
template <> struct Tile<SUBSPEC_F16, 8> : Tile16x8<SUBSPEC_F16> {};
template <int DT> struct Tile16x1 {
  uint16_t r;
  __device__ __forceinline__ void load(const void* p, int64_t i) { r = ((const uint16_t*)p)[i]; }
  __device__ __forceinline__ void load_cached(const void* p, int64_t i) { load(p, i); }
  __device__ __forceinline__ void fill_neg_inf() { r = DT == SUBSPEC_BF16 ? 0xff80 : 0xfc00; }
  __device__ __forceinline__ float get(int) const {
    return DT == SUBSPEC_BF16 ? bf16_bits_to_float(r) : f16_bits_to_float(r);
  }
  __device__ __forceinline__ void fence() { uint32_t w = r; asm volatile("" : "+v"(w)); r = (uint16_t)w; }
};
template <> struct Tile<SUBSPEC_BF16, 1> : Tile16x1<SUBSPEC_BF16> {};
template <> struct Tile<SUBSPEC_F16, 1> : Tile16x1<SUBSPEC_F16> {};

// ------------------------------------------------------------------ combining the slices of a row
struct RowStat {
  float m, S, h;        // row max, sum exp(x - m), normalized entropy from the fp32 pass
  float pmax;           // max probability rounded to the row dtype
  int first_idx;        // first index holding the max logit
  bool need_emu;        // entropy must be re-evaluated with per-element rounding
  bool need_tie;        // rounded probabilities of distinct logits may tie with the max
};

struct VerifyParams {
  int64_t vocab;
  int splits;
  int64_t chunk;
  int gate_entropy;     // 1 when the entropy gate is active (lossy + entropy)
  int entropy_policy;
  float theta;
  float ln_vocab;       // float(ln V), or 1 when V == 1 (lossy_tree_verify.py:68)
  int sample;           // 1: the target token of a row is drawn from its distribution
  int ties_in_accept;   // 1: sliced rows without the exact pass (no entropy gate): the acceptance kernel resolves ties
  Divisor temperature;  // rows are divided by .t (and rounded to their dtype) when .t != 1
  uint32_t key[2];      // Philox key: the caller's 64-bit seed
  uint32_t offset[2];   // Philox counter words 2, 3: the caller's 64-bit stream offset
};

// TemperatureLogitsWarper on one element: IEEE quotient, one rounding to the row dtype
template <int DT, bool WARP>
__device__ __forceinline__ float warped(float x, const Divisor& temperature) {
  if constexpr (WARP) return Elem<DT>::round(div_rn(x, temperature));
  return x;
}
template <int DT>
__device__ __forceinline__ float load_warped(const void* logits, int64_t i, const VerifyParams& vp) {
  const float x = Elem<DT>::load(logits, i);
  return vp.temperature.t != 1.0f ? Elem<DT>::round(div_rn(x, vp.temperature)) : x;
}

template <int DT>
__device__ __forceinline__ float finish_entropy(float H, float ln_vocab) {
  // sum rounded to the row dtype, divided by float(ln V), rounded again
  return Elem<DT>::round(Elem<DT>::round(H) / ln_vocab);
}

template <int DT>
__device__ RowStat combine_row(const Part1* __restrict__ p, const VerifyParams& vp) {
  RowStat r;
  float m = -INFINITY;
  for (int c = 0; c < vp.splits; ++c) m = fmaxf(m, p[c].m);
  float S = 0.f, U = 0.f;
  int first = 0x7fffffff;
  for (int c = 0; c < vp.splits; ++c) {
    if (p[c].m == -INFINITY) continue;
    const float d = fmaxf((p[c].ref - m) * kLog2e, -200.f);   // ref <= slice max <= m
    const float w = __builtin_amdgcn_exp2f(d);
    S = fmaf(p[c].s, w, S);
    U = fmaf(fmaf(d, p[c].s, p[c].u), w, U);
    if (p[c].m == m) first = min(first, p[c].idx);
  }
  r.m = m;
  r.S = S;
  r.first_idx = first;
  r.pmax = Elem<DT>::round(1.0f / S);
  const float H = logf(S) - kLn2 * U / S;
  r.h = finish_entropy<DT>(H, vp.ln_vocab);
  const float h_raw = H / vp.ln_vocab;
  r.need_emu = false;
  if (vp.gate_entropy && DT != SUBSPEC_F32) {
    const float band = 0.02f * fabsf(vp.theta) + 1e-3f;
    r.need_emu = vp.entropy_policy == SUBSPEC_ENTROPY_ALWAYS || DT == SUBSPEC_F16 ||
                 fabsf(h_raw - vp.theta) <= band;
  }
  // Two distinct logits of the row dtype differ by >= 2 ulp-of-one when |max| >= 2, so their
  // probabilities differ by more than one ulp and cannot round to the same value unless the
  // rounded maximum is subnormal.
  r.need_tie = !(fabsf(m) >= 2.0f && (1.0f / S) >= Elem<DT>::min_normal());
  return r;
}

// probability of logit x in a row, as the reference stores it: exp(x - m) / S rounded to dtype
template <int DT>
__device__ __forceinline__ float rounded_prob(float x, float m, float S) {
  return Elem<DT>::round(expf(x - m) / S);
}

// ------------------------------------------------------------------ rare exact pass over one slice
// Re-reads the slice (normally still in L2) and evaluates what the reference evaluates element by
// element: the entropy terms with p, log p and p*log p rounded to the row dtype, and the first
// index whose rounded probability equals the rounded maximum.
template <int DT>
__device__ __forceinline__ void row_exact_body(const void* __restrict__ logits, const VerifyParams& vp,
                                               const RowStat& rs, int64_t row, int c, float* red_f, int* red_i,
                                               Part2* __restrict__ part2) {
  const int64_t c0 = (int64_t)c * vp.chunk;
  const int64_t n = min(vp.chunk, vp.vocab - c0);
  const int64_t base = row * vp.vocab + c0;
  float acc = 0.f;
  int tie = 0x7fffffff;
  for (int64_t i = threadIdx.x; i < n; i += kRowThreads) {
    const float x = load_warped<DT>(logits, base + i, vp);
    const float p = rounded_prob<DT>(x, rs.m, rs.S);
    if (rs.need_emu && p > 0.f) acc += Elem<DT>::round(-p * Elem<DT>::round(logf(p)));
    if (p == rs.pmax && tie == 0x7fffffff) tie = (int)(c0 + i);
  }
  acc = block_sum<kRowThreads>(acc, red_f);
  tie = block_min_i<kRowThreads>(tie, red_i);
  if (threadIdx.x == 0) part2[row * vp.splits + c] = Part2{acc, tie};
}

// Separate launch, used when a row is split over several workgroups (the slices of a row must all
// be reduced before any of them knows the row's statistics).
template <int DT>
__global__ __launch_bounds__(kRowThreads) void row_exact_kernel(
    const void* __restrict__ logits, VerifyParams vp, const Part1* __restrict__ part1,
    Part2* __restrict__ part2) {
  __shared__ float red_f[kRowThreads / kWave];
  __shared__ int red_i[kRowThreads / kWave];
  const int64_t row = blockIdx.y;
  const RowStat rs = combine_row<DT>(part1 + row * vp.splits, vp);
  if (!rs.need_emu && !rs.need_tie) return;           // uniform across the workgroup
  row_exact_body<DT>(logits, vp, rs, row, blockIdx.x, red_f, red_i, part2);
}

// ------------------------------------------------------------------ kernel 1: one pass over HBM
// sum exp and sum t*exp of one tile relative to the reference `mb = -ref * log2(e)`;
// t is clamped so that exp2(t) == 0 implies t * exp2(t) == 0 (x may be -inf).
template <int DT, int VEC, bool WARP>
__device__ __forceinline__ float tile_accumulate(const Tile<DT, VEC>& t, float mb, const Divisor& temperature,
                                                 float (&s)[2], float (&u)[2]) {
  float x[VEC];
  // Packed 16-bit tiles are floored while still packed (half an instruction per element instead of one
  // fp32 maximum): t stays finite, and whatever lies that far below the reference contributes exp2(t) == 0
  // and t * 0 == 0 either way.  The maximum of a fully masked tile is then the floor instead of -inf; it
  // can only surface as a row maximum when the whole row is masked.
  constexpr bool kPackedFloor = !WARP && DT != SUBSPEC_F32 && VEC == 8;
  if constexpr (kPackedFloor) {
    Tile<DT, VEC> tc = t;
    tc.floor_neg_inf();
#pragma unroll
    for (int k = 0; k < VEC; ++k) x[k] = tc.get(k);
  } else {
#pragma unroll
    for (int k = 0; k < VEC; ++k) x[k] = warped<DT, WARP>(t.get(k), temperature);
  }
  float tmax = x[0];
#pragma unroll
  for (int k = 1; k < VEC; ++k) tmax = fmaxf(tmax, x[k]);
#pragma unroll
  for (int k = 0; k < VEC; ++k) {
    const float raw = fmaf(x[k], kLog2e, mb);
    const float tt = kPackedFloor ? raw : fmaxf(raw, -200.f);
    const float e = __builtin_amdgcn_exp2f(tt);
    s[k & 1] += e;
    u[k & 1] = fmaf(tt, e, u[k & 1]);
  }
  return tmax;
}

template <int DT, int VEC, int U, bool WARP>
__global__ __launch_bounds__(kRowThreads) void row_partial_kernel(
    const void* __restrict__ logits, VerifyParams vp, Part1* __restrict__ part, Part2* __restrict__ part2) {
  const int64_t vocab = vp.vocab, chunk = vp.chunk;
  const int splits = vp.splits;
  __shared__ float red_f[kRowThreads / kWave];
  __shared__ int red_i[kRowThreads / kWave];
  __shared__ float red_s[kRowThreads / kWave], red_u[kRowThreads / kWave];
  const int64_t row = blockIdx.y;
  const int c = blockIdx.x;
  const int tid = threadIdx.x;
  const int64_t c0 = (int64_t)c * chunk;
  const int64_t n = min(chunk, vocab - c0);           // elements of this slice (a multiple of VEC)
  const int64_t base = row * vocab + c0;
  const int64_t ntiles = n / VEC;

  float vmax = -INFINITY;
  int best_tile = 0;                                   // tile index inside the slice (a slice has < 2^31 elements)
  Tile<DT, VEC> best;                                  // and its contents: the first index of the maximum is found in registers
  best.fill_neg_inf();
  float s[2], u[2];
  const int nt = (int)ntiles;
  constexpr int kStep = kRowThreads * U;               // tiles per trip of the whole workgroup
  const int n_full = nt / kStep;                       // trips in which every thread's U tiles exist
  // One tile after the other: the two empty statements are ordered among themselves, the first makes the tile opaque
  // (nothing of it is unpacked earlier), the second waits for its sums.  Left alone, the compiler works on the tiles
  // of a trip side by side and needs 107 registers instead of 74 (2048 x 152064 bf16: 104.5 against 101.3 us).
  auto take = [&](Tile<DT, VEC> t, int j, float mb) {
    t.fence();
    const float tmax = tile_accumulate<DT, VEC, WARP>(t, mb, vp.temperature, s, u);
    if (tmax > vmax) { vmax = tmax; best_tile = j; best = t; }
    asm volatile("" : "+v"(s[0]), "+v"(s[1]), "+v"(u[0]), "+v"(u[1]), "+v"(vmax));
  };

  // Reference point for the exponentials: the largest value among the first tile of every
  // thread.  It is at most the true maximum; the slice is redone against the true maximum in the
  // (pathological) case that the two are so far apart that exp2 could overflow.
  float ref;
  {
    Tile<DT, VEC> t0;
    if (tid < ntiles) t0.load_cached(logits, base + (int64_t)tid * VEC); else t0.fill_neg_inf();   // the loop reads it again
    float r = warped<DT, WARP>(t0.get(0), vp.temperature);
#pragma unroll
    for (int k = 1; k < VEC; ++k) r = fmaxf(r, warped<DT, WARP>(t0.get(k), vp.temperature));
    ref = block_max<kRowThreads>(r, red_f);
    if (ref == -INFINITY) ref = -1e30f;
  }

  // one pass over the slice
  auto run_trips = [&](float mb) {
    // full trips: no bounds, the U loads of a thread go out back to back
    for (int it = 0; it < n_full; ++it) {
      const int j0 = it * kStep + tid;
      Tile<DT, VEC> t[U];
#pragma unroll
      for (int i = 0; i < U; ++i) t[i].load(logits, base + (int64_t)(j0 + i * kRowThreads) * VEC);
#pragma unroll
      for (int i = 0; i < U; ++i) take(t[i], j0 + i * kRowThreads, mb);
    }
    // the last, ragged trip: clamped loads, missing tiles count as -inf
    if (n_full * kStep + tid < nt) {
      const int j0 = n_full * kStep + tid;
      Tile<DT, VEC> t[U];
#pragma unroll
      for (int i = 0; i < U; ++i) t[i].load(logits, base + (int64_t)min(j0 + i * kRowThreads, nt - 1) * VEC);
#pragma unroll
      for (int i = 0; i < U; ++i) {
        if (j0 + i * kRowThreads >= nt) t[i].fill_neg_inf();
        take(t[i], j0 + i * kRowThreads, mb);
      }
    }
  };
  s[0] = s[1] = u[0] = u[1] = 0.f;
  run_trips(-ref * kLog2e);
  const float m = block_max<kRowThreads>(vmax, red_f);  // the slice's maximum
  if ((m - ref) * kLog2e > 100.f) {                    // workgroup-uniform, pathological: redo against the true maximum
    ref = m;
    s[0] = s[1] = u[0] = u[1] = 0.f;
    run_trips(-ref * kLog2e);
  }

  int idx = 0x7fffffff;
  if (vmax == m && m != -INFINITY) {                  // first index of the maximum inside this thread's tiles
#pragma unroll
    for (int k = VEC - 1; k >= 0; --k)
      if (warped<DT, WARP>(best.get(k), vp.temperature) == m) idx = (int)(c0 + (int64_t)best_tile * VEC + k);
  }
  // the two sums and the index in one exchange: wavefront butterflies, then wavefronts 0..7 in order (the order of
  // block_sum, so the sums do not depend on timing)
  float ssum = wave_sum(s[0] + s[1]), usum = wave_sum(u[0] + u[1]);
  idx = wave_min_i(idx);
  if ((tid & (kWave - 1)) == 0) { red_s[tid / kWave] = ssum; red_u[tid / kWave] = usum; red_i[tid / kWave] = idx; }
  __syncthreads();
  ssum = red_s[0]; usum = red_u[0]; idx = red_i[0];
#pragma unroll
  for (int w = 1; w < kRowThreads / kWave; ++w) { ssum += red_s[w]; usum += red_u[w]; idx = min(idx, red_i[w]); }
  __syncthreads();                                     // red_i is used again by the exact pass
  const Part1 mine{ref, ssum, usum, m, idx, {0, 0, 0}};
  if (tid == 0) part[row * splits + c] = mine;
  if (splits == 1) {
    // the workgroup holds the statistics of the whole row: decide here whether the row needs the
    // exact pass and run it while the row is still in cache
    const RowStat rs = combine_row<DT>(&mine, vp);
    if (rs.need_emu || rs.need_tie) row_exact_body<DT>(logits, vp, rs, row, 0, red_f, red_i, part2);
  }
}

// ------------------------------------------------------------------ kernel 2b: one draw per row
// Philox4x32-10 (Salmon et al., "Parallel random numbers: as easy as 1, 2, 3", SC'11).
__device__ __forceinline__ void philox4x32_10(uint32_t c0, uint32_t c1, uint32_t c2, uint32_t c3, uint32_t k0,
                                              uint32_t k1, uint32_t (&out)[4]) {
#pragma unroll
  for (int r = 0; r < 10; ++r) {
    const uint64_t p0 = (uint64_t)0xD2511F53u * c0;    // one 32 x 32 -> 64 bit multiply each
    const uint64_t p1 = (uint64_t)0xCD9E8D57u * c2;
    c0 = (uint32_t)(p1 >> 32) ^ c1 ^ k0;
    c1 = (uint32_t)p1;
    c2 = (uint32_t)(p0 >> 32) ^ c3 ^ k1;
    c3 = (uint32_t)p0;
    k0 += 0x9E3779B9u;
    k1 += 0xBB67AE85u;
  }
  out[0] = c0; out[1] = c1; out[2] = c2; out[3] = c3;
}

// Relative and absolute rounding bounds of one value stored in the row dtype (generous).
template <int DT> struct RoundBound;
template <> struct RoundBound<SUBSPEC_F32> { static constexpr float rel = 0x1p-21f, abs = 0.f; };
template <> struct RoundBound<SUBSPEC_F16> { static constexpr float rel = 0x1p-10f, abs = 0x1p-24f; };
template <> struct RoundBound<SUBSPEC_BF16> { static constexpr float rel = 0x1p-8f, abs = 0.f; };

// Element i of global row `row` uses word i % 4 of Philox(counter = {i / 4, row, offset}, key = seed);
// u = ((word >> 9) + 0.5) * 2^-23 lies strictly inside (0, 1) and is exact in fp32.
// A slice starts at a multiple of 4, so a 4-element group never straddles two workgroups.
//
// The race key of an element is p / -log(u), evaluated exactly as defined (rounded probability,
// accurate logarithm, IEEE quotient) only for the few elements that can still win: -log(u) >= 1 - u
// and p <= an upper bound from the hardware exponential give key <= bound / (1 - u), and an
// element whose bound stays below the best key any lane of the wavefront has seen is skipped.
// What is left per element is the Philox block, one exponential and a compare.
// QUAD: the slice starts and ends on multiples of four elements and the rows are aligned for it, so the four logits
// of a Philox block are one load (8 bytes of a 16-bit row, 16 of an fp32 row) and need no bounds.
template <int DT, bool QUAD>
__global__ __launch_bounds__(kRowThreads) void row_sample_kernel(
    const void* __restrict__ logits, VerifyParams vp, const Part1* __restrict__ part1, Part3* __restrict__ part3) {
  __shared__ float red_f[kRowThreads / kWave];
  __shared__ int red_i[kRowThreads / kWave];
  const int64_t row = blockIdx.y;
  const int c = blockIdx.x;
  const RowStat rs = combine_row<DT>(part1 + row * vp.splits, vp);
  const int64_t c0 = (int64_t)c * vp.chunk;
  const int64_t n = min(vp.chunk, vp.vocab - c0);
  const int64_t base = row * vp.vocab + c0;
  const bool warp = vp.temperature.t != 1.0f;
  const float inv_t = warp ? vp.temperature.inv_t : 1.0f;
  const float round_up = warp ? RoundBound<DT>::rel : 0.f;          // x / T rounded to the dtype, relative
  const float round_abs = warp ? RoundBound<DT>::abs + 1e-30f : 0.f;
  const float mb = -rs.m * kLog2e;
  // p <= exp2((x' - m) log2 e) / S * (1 + rounding of p, of the hardware exp2 and of this arithmetic)
  const float p_scale = (1.0f / rs.S) * (1.0f + 4.0f * RoundBound<DT>::rel + 1e-4f);
  float best = -1.f;
  int idx = 0x7fffffff;
  float thr = 0.f;                                     // 0.9999 * 2^-23 * best key of the wavefront
  for (int64_t g0 = 0; g0 * 4 < n; g0 += kRowThreads) {   // same trip count for every lane: the votes below see whole wavefronts
    const int64_t g = g0 + threadIdx.x;
    float xs[4];
    if constexpr (QUAD) {                              // one load, clamped to the last block of the slice
      const int64_t q = min(g, n / 4 - 1);
      if constexpr (DT == SUBSPEC_F32) {
        const float4 v = *(const float4*)((const float*)logits + base + q * 4);
        xs[0] = v.x; xs[1] = v.y; xs[2] = v.z; xs[3] = v.w;
      } else {
        const uint2 v = *(const uint2*)((const uint16_t*)logits + base + q * 4);
        if constexpr (DT == SUBSPEC_BF16) {
          xs[0] = __uint_as_float(v.x << 16); xs[1] = __uint_as_float(v.x & 0xffff0000u);
          xs[2] = __uint_as_float(v.y << 16); xs[3] = __uint_as_float(v.y & 0xffff0000u);
        } else {
          xs[0] = f16_bits_to_float(v.x & 0xffffu); xs[1] = f16_bits_to_float(v.x >> 16);
          xs[2] = f16_bits_to_float(v.y & 0xffffu); xs[3] = f16_bits_to_float(v.y >> 16);
        }
      }
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e)                      // unconditional loads (clamped index), in flight during the Philox rounds
        xs[e] = Elem<DT>::load(logits, base + min(g * 4 + e, n - 1));
    }
    uint32_t w[4];
    philox4x32_10((uint32_t)(c0 / 4 + g), (uint32_t)row, vp.offset[0], vp.offset[1], vp.key[0], vp.key[1], w);
    bool cand[4];
    bool any_cand = false;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int64_t i = g * 4 + e;
      const float xa = fmaxf(xs[e] * inv_t, -1e30f);                 // masked (-inf) logits stay finite below
      const float xu = fmaf(fabsf(xa), round_up, xa) + round_abs;
      const float bound = fmaf(__builtin_amdgcn_exp2f(fmaf(xu, kLog2e, mb)), p_scale, RoundBound<DT>::abs);
      const float one_minus_u = (float)((~w[e]) >> 9) + 0.5f;        // (1 - u) * 2^23, exact
      cand[e] = (QUAD ? g * 4 < n : i < n) && !(bound < thr * one_minus_u);
      any_cand |= cand[e];
    }
    // one vote per block of four: the threshold only prunes, so refreshing it less often changes no result
    if (__any(any_cand)) {                             // wavefront-uniform
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        if (cand[e]) {
          const float x = xs[e];
          const float xw = warp ? Elem<DT>::round(div_rn(x, vp.temperature)) : x;
          const float p = rounded_prob<DT>(xw, rs.m, rs.S);
          const float u = ((float)(w[e] >> 9) + 0.5f) * 0x1p-23f;
          const float key = p / -logf(u);
          if (key > best) { best = key; idx = (int)(c0 + g * 4 + e); }   // indices ascend: the first maximum stays
        }
      }
      thr = fmaxf(wave_max(best), 0.f) * (0.9999f * 0x1p-23f);
    }
  }
  const float top = block_max<kRowThreads>(best, red_f);
  idx = block_min_i<kRowThreads>(best == top ? idx : 0x7fffffff, red_i);
  if (threadIdx.x == 0) part3[row * vp.splits + c] = Part3{top, idx};
}

// ------------------------------------------------------------------ kernel 3: per-tree tail
// One wavefront per tree.  Lane l owns nodes l, l+64, l+128, l+192 in registers; the tree is
// walked with ballots (greedy walk) or reduced bottom-up in lockstep (lossy DP): nodes are visited
// from the last to the first, the visited node's finished state is broadcast with readlane and
// the lane owning its parent folds it in.  Choosing a child is a lexicographic maximum over
// (path length, exact match, probability of a lossy child, lower index), which is exactly the
// update rule of lossy_tree_verify.py:148-164 and does not depend on the visiting order.
struct TreeParams {
  int64_t rows, n_nodes;
  int root, skip;
  int64_t eos;
  int method, gate;
  double theta;
  int window;
};


__device__ __forceinline__ int bcast_i(int v, int lane) { return __builtin_amdgcn_readlane(v, lane); }
__device__ __forceinline__ uint64_t bcast_u64(uint64_t v, int lane) {
  const uint32_t lo = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)v, lane);
  const uint32_t hi = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)(v >> 32), lane);
  return ((uint64_t)hi << 32) | lo;
}
template <typename T, int kSlots>
__device__ __forceinline__ T pick_slot(const T (&a)[kSlots], int slot) {
  T r = a[0];
#pragma unroll
  for (int s = 1; s < kSlots; ++s) r = (slot == s) ? a[s] : r;
  return r;
}

// kSlots = nodes per lane (1, 2, 4 or 8: trees of up to 64, 128, 256, 512 nodes); LOSSY selects the
// verifier.  Both are compile-time so that the common 64-node case stays a few hundred
// instructions: a single wavefront pays for every instruction-cache miss it takes.
template <int DT, int kSlots, bool LOSSY>
__global__ __launch_bounds__(kTailThreads) void tree_accept_kernel(
    const void* __restrict__ logits, VerifyParams vp, TreeParams tp,
    const Part1* __restrict__ part1, const Part2* __restrict__ part2, const Part3* __restrict__ part3,
    const int32_t* __restrict__ token_ids, const int32_t* __restrict__ parents,
    int64_t* __restrict__ out_tokens, int64_t* __restrict__ out_ctx, int32_t* __restrict__ out_counts,
    int64_t* __restrict__ node_target, float* __restrict__ node_entropy, float* __restrict__ node_child_prob) {
  constexpr int N = kSlots * kWave;
  __shared__ float sm_m[N], sm_S[N], sm_h[N];
  __shared__ int sm_tgt[N], sm_par[N], sm_ea[N];
  __shared__ unsigned long long sm_best[N];

  const int b = blockIdx.x;
  const int lane = threadIdx.x;
  const int rows = (int)tp.rows, n_nodes = (int)tp.n_nodes, skip = tp.skip;
  constexpr bool lossy = LOSSY;
  token_ids += (int64_t)b * n_nodes;
  parents += (int64_t)b * n_nodes;
  out_tokens += (int64_t)b * (n_nodes + 1);
  out_ctx += (int64_t)b * (n_nodes + 1);
  int status = 0;

  // ---- per scored row: max, sum, argmax token, entropy
  bool tie_rows[kSlots];
  float tie_pmax[kSlots];
#pragma unroll
  for (int s = 0; s < kSlots; ++s) {
    const int r = s * kWave + lane;
    tie_rows[s] = false;
    tie_pmax[s] = 0.f;
    if (r < rows) {
      const int64_t grow = (int64_t)b * rows + r;
      const RowStat rs = combine_row<DT>(part1 + grow * vp.splits, vp);
      int tgt = rs.first_idx;
      float h = rs.h;
      if (vp.ties_in_accept) {
        tie_rows[s] = rs.need_tie;                     // resolved below, by the whole wavefront
        tie_pmax[s] = rs.pmax;
      } else if (rs.need_emu || rs.need_tie) {
        float H = 0.f;
        int tie = 0x7fffffff;
        for (int c = 0; c < vp.splits; ++c) {
          H += part2[grow * vp.splits + c].esum;
          tie = min(tie, part2[grow * vp.splits + c].tie_idx);
        }
        if (rs.need_tie && tie != 0x7fffffff) tgt = tie;
        if (rs.need_emu) h = finish_entropy<DT>(H, vp.ln_vocab);
      }
      if (vp.sample) {                                 // the drawn token replaces the argmax
        float top = -1.f;
        int drawn = 0x7fffffff;
        for (int c = 0; c < vp.splits; ++c) {
          const Part3 q = part3[grow * vp.splits + c];
          if (q.key > top || (q.key == top && q.idx < drawn)) { top = q.key; drawn = q.idx; }
        }
        if (drawn != 0x7fffffff) tgt = drawn;
      }
      sm_m[r] = rs.m;
      sm_S[r] = rs.S;
      sm_tgt[r] = tgt;
      sm_h[r] = h;
      node_target[grow] = tgt;
      node_entropy[grow] = vp.gate_entropy ? h : 0.f;   // always written: the caller need not clear the buffer
    }
  }
  __syncthreads();
  // Sliced rows of a run without the entropy gate come without the exact pass.  A row whose rounded probabilities
  // may tie with the maximum (a maximum below 2 in magnitude, or a subnormal rounded maximum) is resolved here by the
  // whole wavefront: first index whose rounded probability equals the rounded maximum, as row_exact_body finds it.
  // Only slices that can hold such an index are read: exp(x - m) must lie within the dtype's relative spacing at the
  // rounded maximum of 1, i.e. the slice's own maximum within `delta` of the row's, and the slice must not lie behind the
  // first index of the maximum logit (which ties with itself).  For rows as a language model emits them that is the one
  // slice holding the maximum (64 steps), where a scan of the whole row would cost the launch a millisecond per tree.
  if (vp.ties_in_accept) {
#pragma unroll
    for (int s = 0; s < kSlots; ++s) {
      uint64_t pending = __ballot(tie_rows[s]);
      while (pending) {                                // uniform
        const int src = __builtin_ctzll(pending);
        pending &= pending - 1;
        const int r = s * kWave + src;
        const float m = sm_m[r], S = sm_S[r], pmax = __shfl(tie_pmax[s], src, kWave);
        const int first_idx = sm_tgt[r];
        const int64_t grow = (int64_t)b * rows + r;
        const int64_t base = grow * vp.vocab;
        // relative spacing of the dtype at 1 / S (twice over, for the rounding of the exponential itself)
        const float spacing_normal = DT == SUBSPEC_BF16 ? 0.015625f : DT == SUBSPEC_F16 ? 0.001953125f : 2.4e-7f;
        const float spacing_sub = DT == SUBSPEC_F16 ? 1.2e-7f : DT == SUBSPEC_BF16 ? 1.9e-40f : 3e-45f;   // twice 2^-24 / 2^-133 / 2^-149
        const float rel = fmaxf(spacing_normal, spacing_sub * S);
        const float delta = rel < 0.5f ? -logf(1.0f - rel) : INFINITY;
        int tie = 0x7fffffff;
        for (int c = 0; c < vp.splits && tie == 0x7fffffff; ++c) {                     // uniform
          const int64_t c0 = (int64_t)c * vp.chunk;
          if (c0 > first_idx) break;
          if (!(part1[grow * vp.splits + c].m >= m - delta)) continue;
          const int64_t c1 = min(c0 + vp.chunk, vp.vocab);
          for (int64_t i0 = c0; i0 < c1 && tie == 0x7fffffff; i0 += kWave) {             // uniform
            const int64_t i = i0 + lane;
            int hit = 0x7fffffff;
            if (i < c1 && rounded_prob<DT>(load_warped<DT>(logits, base + i, vp), m, S) == pmax) hit = (int)i;
            tie = wave_min_i(hit);
          }
        }
        if (lane == src && tie != 0x7fffffff) {
          sm_tgt[r] = tie;
          node_target[grow] = tie;
        }
      }
    }
    __syncthreads();
  }

  // ---- per node: token, parent, p[parent(i), token(i)]
  int tok[kSlots], par[kSlots];
  float cp[kSlots];
#pragma unroll
  for (int s = 0; s < kSlots; ++s) {
    const int i = s * kWave + lane;
    tok[s] = -1;
    par[s] = -2;                                       // matches no node
    cp[s] = -1.f;
    if (i < n_nodes) {
      tok[s] = token_ids[i];
      par[s] = parents[i];
      if (par[s] >= i) status |= 2;                    // precondition: parents precede children
      if (par[s] >= 0) {
        int rp = par[s] - skip;
        if (rp < 0 && !lossy) rp += rows;              // the exact walk indexes rows like a python list
        if (rp >= 0 && rp < rows && tok[s] >= 0 && tok[s] < vp.vocab) {
          const float x = load_warped<DT>(logits, ((int64_t)b * rows + rp) * vp.vocab + tok[s], vp);
          cp[s] = rounded_prob<DT>(x, sm_m[rp], sm_S[rp]);
        }
      }
      const int local = i - skip;
      if (local >= 0 && local < rows) node_child_prob[(int64_t)b * rows + local] = cp[s];
    }
  }
  status = __any(status != 0) ? 2 : 0;

  int emitted = 0, accept = 0, total = 0;
  auto emit = [&](int64_t token, int ctx) {
    if (lane == 0) { out_tokens[emitted] = token; out_ctx[emitted] = ctx; }
    ++emitted;
  };
  int64_t last_token = -1;

  if constexpr (!LOSSY) {
    // ---------------- greedy walk in original indexing (tree_verify.py:49-106)
    auto row_of = [&](int node) { int r = node - skip; if (r < 0) r += rows; return r; };
    auto first_child = [&](int node, int want_tok, bool match_tok) {
      int found = -1;
#pragma unroll
      for (int s = kSlots - 1; s >= 0; --s) {
        const uint64_t m = __ballot(par[s] == node && (!match_tok || tok[s] == want_tok));
        if (m) found = s * kWave + __builtin_ctzll(m);
      }
      return found;
    };
    int cur = tp.root;
    int bonus = -1;
    bool bad = cur < 0 || cur >= n_nodes;
    while (!bad && first_child(cur, 0, false) >= 0) {
      ++total;
      const int r = row_of(cur);
      if (r < 0 || r >= rows) { bad = true; break; }
      const int t = sm_tgt[r];
      const int hit = first_child(cur, t, true);
      if (hit < 0) { bonus = t; break; }
      ++accept;
      emit(t, cur);
      last_token = t;
      if (tp.eos >= 0 && (int64_t)t == tp.eos) break;
      cur = hit;
      const int kid = first_child(cur, 0, false);
      if (kid < 0) break;
      if (kid - skip >= rows) break;                   // children were not scored in this call
    }
    if (!bad && (emitted == 0 || tp.eos < 0 || last_token != tp.eos)) {
      if (bonus < 0) {
        const int r = row_of(cur);
        if (r < 0 || r >= rows) bad = true; else bonus = sm_tgt[r];
      }
      if (!bad) emit(bonus, cur);
    }
    if (bad) status |= 1;
  } else {
    // ---------------- bottom-up DP in local indexing (lossy_tree_verify.py:112-168)
    const int nl = min(rows, n_nodes - skip);
    if (nl <= 0) {
      emit(rows > 0 ? sm_tgt[0] : 0, tp.root);
    } else {
      int root = tp.root - skip;
      if (root < 0 || root >= nl) root = 0;
      const bool use_entropy = tp.gate == SUBSPEC_GATE_ENTROPY;
      const int need = max(0, tp.window);
      // Level-parallel reduction: all nodes of one depth fold themselves into their parents at
      // once with LDS atomic max, deepest level first (a node's own state is final once every
      // deeper level has been folded).
      int pl[kSlots], depth[kSlots];                   // parent in local indexing (-1: none in the slice)
      int max_depth = 0;
#pragma unroll
      for (int s = 0; s < kSlots; ++s) {
        const int li = s * kWave + lane - skip;
        pl[s] = -1;
        depth[s] = 0;
        if (s * kWave + lane < N) { sm_ea[s * kWave + lane] = 0; sm_best[s * kWave + lane] = 0; }
        if (li >= 1 && li < nl) {
          const int p = par[s] - skip;
          if (p >= 0 && p < nl && p < li) pl[s] = p;
        }
        if (li >= 0 && li < nl) sm_par[li] = pl[s];
      }
      __syncthreads();
#pragma unroll
      for (int s = 0; s < kSlots; ++s) {
        int d = 0;
        for (int c = pl[s]; c >= 0; c = sm_par[c]) ++d;
        depth[s] = d;
        max_depth = max(max_depth, d);
      }
#pragma unroll
      for (int o = 32; o > 0; o >>= 1) max_depth = max(max_depth, __shfl_xor(max_depth, o, kWave));
      for (int d = max_depth; d >= 1; --d) {
#pragma unroll
        for (int s = 0; s < kSlots; ++s) {
          if (depth[s] == d && pl[s] >= 0) {
            const int li = s * kWave + lane - skip;
            const int p = pl[s];
            const bool ex = tok[s] == sm_tgt[p];
            const int ea = sm_ea[li];
            const int blen = (int)(sm_best[li] >> 54);
            const bool gate_blocks = use_entropy ? ((double)sm_h[p] >= tp.theta) : ((double)cp[s] < tp.theta);
            const bool admissible = ex || (ea >= need && !gate_blocks);
            if (ex) atomicMax(&sm_ea[p], 1 + ea);
            if (admissible) {
              const uint32_t pb = ex ? 0u : __float_as_uint(fmaxf(cp[s], 0.f));
              const unsigned long long key = ((unsigned long long)(1 + blen) << 54) | ((unsigned long long)ex << 53) |
                                             ((unsigned long long)pb << 21) | ((unsigned long long)(511 - li) << 12) | 1ull;
              atomicMax(&sm_best[p], key);
            }
          }
        }
        __syncthreads();
      }
      int ctx = root;
      while (true) {                                   // lossy_tree_verify.py:247-286
        const unsigned long long bk = sm_best[ctx];
        if (bk == 0) break;
        const int nxt = 511 - (int)((bk >> 12) & 0x1ff);
        const int on = nxt + skip;
        const int t = bcast_i(pick_slot<int, kSlots>(tok, on >> 6), on & (kWave - 1));
        emit(t, ctx + skip);
        last_token = t;
        if (tp.eos >= 0 && (int64_t)t == tp.eos) break;
        ctx = nxt;
      }
      accept = emitted;
      if (emitted == 0 || tp.eos < 0 || last_token != tp.eos) emit(sm_tgt[ctx], ctx + skip);
      total = emitted;
    }
  }
  if (lane == 0) {
    out_counts[b * 4 + 0] = emitted;
    out_counts[b * 4 + 1] = accept;
    out_counts[b * 4 + 2] = total;
    out_counts[b * 4 + 3] = status;
  }
}

// ------------------------------------------------------------------ host side
struct Plan { int vec, splits; int64_t chunk; };

// Slices per row; a slice is a whole number of 512-thread tiles.
// Greedy target: one slice from 256 rows on.  The workgroup that holds a whole row decides by itself whether the row
// needs the exact pass and runs it while the row is in cache.  Fewer rows are cut into up to 8 slices, about 256
// workgroups in all: a compute unit streams at a fixed rate, and 64 workgroups leave three quarters of the chip idle
// (64 x 152064 fp32: statistics pass 15.7 -> 6 us).  With the entropy gate that costs a second launch (row_exact_kernel,
// which recombines the slices and returns at once for a row that needs nothing); without it the only thing the exact
// pass could find is a tie of rounded probabilities with the maximum, and the acceptance kernel looks for that itself
// in the rows that can have one.  A prepared call: 20.7 us with one workgroup per row, 15.1 with slices and the second
// launch, 12.6 without it; calls that allocate their outputs are bound by the host at 26 us either way.
// Sampling target: the draw is bound by the vector ALU (a Philox block per four elements), so few rows are cut
// into enough slices to cover the chip several times over.
static bool make_plan(const void* logits, int dtype, int64_t total_rows, int64_t vocab, bool sample, Plan* pl) {
  const int vec_full = dtype == SUBSPEC_F32 ? 4 : 8;
  const bool aligned = (vocab % vec_full == 0) && ((uintptr_t)logits % 16 == 0);
  pl->vec = aligned ? vec_full : 1;
  const int64_t quantum = (int64_t)kRowThreads * pl->vec;
  int64_t splits = sample ? (2048 + total_rows - 1) / total_rows : std::min<int64_t>(8, std::max<int64_t>(1, 256 / total_rows));
  splits = std::min<int64_t>(splits, std::max<int64_t>(1, vocab / 8192));
  splits = std::max<int64_t>(1, std::min<int64_t>(splits, kMaxSplits));
  int64_t chunk = (vocab + splits - 1) / splits;
  chunk = (chunk + quantum - 1) / quantum * quantum;
  splits = (vocab + chunk - 1) / chunk;
  if (splits > kMaxSplits) return false;
  pl->splits = (int)splits;
  pl->chunk = chunk;
  return true;
}

template <int DT, int VEC>
static void launch_partial(dim3 grid, hipStream_t st, const void* logits, const VerifyParams& vp, Part1* p1, Part2* p2) {
  // loads in flight per thread: 8 when a slice is long enough for whole trips of that size (whole rows of a
  // large batch: 111 against 113 us at 2048 x 152064 bf16), 4 for the short slices of a few rows split many ways
  const bool long_slices = vp.chunk / VEC >= 2 * (int64_t)kRowThreads * 8;
  if (vp.temperature.t != 1.0f)
    hipLaunchKernelGGL((row_partial_kernel<DT, VEC, 4, true>), grid, dim3(kRowThreads), 0, st, logits, vp, p1, p2);
  else if (long_slices)
    hipLaunchKernelGGL((row_partial_kernel<DT, VEC, 8, false>), grid, dim3(kRowThreads), 0, st, logits, vp, p1, p2);
  else
    hipLaunchKernelGGL((row_partial_kernel<DT, VEC, 4, false>), grid, dim3(kRowThreads), 0, st, logits, vp, p1, p2);
}

template <int DT>
static int run_verify(const void* logits, int64_t batch, int64_t rows, int64_t vocab, const Plan& pl,
                      const VerifyParams& vp, const TreeParams& tp, Part1* p1, Part2* p2, Part3* p3,
                      const int32_t* token_ids, const int32_t* parents, int64_t* out_tokens, int64_t* out_ctx,
                      int32_t* out_counts, int64_t* node_target, float* node_entropy, float* node_child_prob,
                      hipStream_t st) {
  const dim3 grid(pl.splits, (unsigned)(batch * rows));
  auto partial = [&] {
    if (pl.vec == 1) launch_partial<DT, 1>(grid, st, logits, vp, p1, p2);
    else launch_partial<DT, (DT == SUBSPEC_F32 ? 4 : 8)>(grid, st, logits, vp, p1, p2);
  };
  // the timed kernel is the longest one: the statistics pass, or the draw when sampling
  if (vp.sample) partial(); else { DominantKernelTimer timer(st); partial(); }
  if (pl.splits > 1 && !vp.ties_in_accept)
    hipLaunchKernelGGL((row_exact_kernel<DT>), grid, dim3(kRowThreads), 0, st, logits, vp, p1, p2);
  if (vp.sample) {
    DominantKernelTimer timer(st);
    // slices are whole numbers of 512-thread tiles of pl.vec elements: with pl.vec > 1 rows and slices are quad-aligned
    if (pl.vec > 1 && vocab % 4 == 0)
      hipLaunchKernelGGL((row_sample_kernel<DT, true>), grid, dim3(kRowThreads), 0, st, logits, vp, p1, p3);
    else
      hipLaunchKernelGGL((row_sample_kernel<DT, false>), grid, dim3(kRowThreads), 0, st, logits, vp, p1, p3);
  }
  const int64_t widest = std::max<int64_t>(rows, tp.n_nodes);
  const int slots = widest <= kWave ? 1 : widest <= 2 * kWave ? 2 : widest <= 4 * kWave ? 4 : 8;
  const bool lossy = tp.method == SUBSPEC_VERIFY_LOSSY;
#define SUBSPEC_LAUNCH_TAIL(SLOTS, LOSSY)                                                                        \
  hipLaunchKernelGGL((tree_accept_kernel<DT, SLOTS, LOSSY>), dim3((unsigned)batch), dim3(kTailThreads), 0, st,    \
                     logits, vp, tp, p1, p2, p3, token_ids, parents, out_tokens, out_ctx, out_counts, node_target,   \
                     node_entropy, node_child_prob)
  if (slots == 1) { if (lossy) SUBSPEC_LAUNCH_TAIL(1, true); else SUBSPEC_LAUNCH_TAIL(1, false); }
  else if (slots == 2) { if (lossy) SUBSPEC_LAUNCH_TAIL(2, true); else SUBSPEC_LAUNCH_TAIL(2, false); }
  else if (slots == 4) { if (lossy) SUBSPEC_LAUNCH_TAIL(4, true); else SUBSPEC_LAUNCH_TAIL(4, false); }
  else { if (lossy) SUBSPEC_LAUNCH_TAIL(8, true); else SUBSPEC_LAUNCH_TAIL(8, false); }
#undef SUBSPEC_LAUNCH_TAIL
  SUBSPEC_CHECK_HIP(hipGetLastError());
  return SUBSPEC_OK;
}

}  // namespace subspec

using namespace subspec;

extern "C" size_t subspec_tree_verify_workspace(int64_t batch, int64_t rows, int64_t vocab, int dtype) {
  (void)vocab; (void)dtype;
  if (batch <= 0 || rows <= 0) return 256;
  const size_t n = (size_t)batch * rows * kMaxSplits;
  return align_up(n * sizeof(Part1), 256) + align_up(n * sizeof(Part2), 256) + align_up(n * sizeof(Part3), 256);
}

struct SampleArgs { int sample; float temperature; uint64_t seed, offset; };

static int tree_verify_impl(const void* logits, int dtype, int64_t batch, int64_t rows, int64_t vocab,
                            const int32_t* token_ids, const int32_t* parents, int64_t n_nodes,
                            int32_t root, int32_t skip_nodes, int64_t eos_token_id,
                            int verify_method, int threshold_method, double threshold, int32_t window_size,
                            int entropy_policy, void* workspace, size_t workspace_bytes,
                            int64_t* out_tokens, int64_t* out_ctx, int32_t* out_counts,
                            int64_t* node_target, float* node_entropy, float* node_child_prob,
                            const SampleArgs& sa, void* stream) {
  if (!dtype_ok(dtype)) SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "tree_verify: unknown dtype %d", dtype);
  if (!logits || !token_ids || !parents || !workspace || !out_tokens || !out_ctx || !out_counts || !node_target ||
      !node_entropy || !node_child_prob)
    SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "tree_verify: null pointer argument");
  if (batch <= 0 || rows <= 0 || vocab <= 0 || n_nodes <= 0)
    SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "tree_verify: batch=%lld rows=%lld vocab=%lld n_nodes=%lld must be positive",
                 (long long)batch, (long long)rows, (long long)vocab, (long long)n_nodes);
  if (rows > SUBSPEC_MAX_TREE_NODES || n_nodes > SUBSPEC_MAX_TREE_NODES)
    SUBSPEC_FAIL(SUBSPEC_ERR_LIMIT, "tree_verify: rows=%lld / n_nodes=%lld exceed the %d-node limit",
                 (long long)rows, (long long)n_nodes, SUBSPEC_MAX_TREE_NODES);
  if (vocab >= (int64_t)1 << 31 || batch * rows > 65535)
    SUBSPEC_FAIL(SUBSPEC_ERR_LIMIT, "tree_verify: vocab=%lld or batch*rows=%lld too large", (long long)vocab,
                 (long long)(batch * rows));
  if (verify_method != SUBSPEC_VERIFY_EXACT && verify_method != SUBSPEC_VERIFY_LOSSY)
    SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "tree_verify: unsupported verify_method %d", verify_method);
  if (threshold_method != SUBSPEC_GATE_ENTROPY && threshold_method != SUBSPEC_GATE_PROB)
    SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "tree_verify: unsupported threshold_method %d", threshold_method);
  if (skip_nodes < 0 || skip_nodes >= n_nodes + rows)
    SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "tree_verify: skip_nodes=%d out of range", skip_nodes);
  if (workspace_bytes < subspec_tree_verify_workspace(batch, rows, vocab, dtype))
    SUBSPEC_FAIL(SUBSPEC_ERR_WORKSPACE, "tree_verify: workspace of %zu bytes is smaller than the %zu required",
                 workspace_bytes, subspec_tree_verify_workspace(batch, rows, vocab, dtype));
  if ((uintptr_t)workspace % 16 != 0) SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "tree_verify: workspace must be 16-byte aligned");
  if ((uintptr_t)logits % dtype_size(dtype) != 0) SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "tree_verify: logits misaligned");

  Plan pl;
  if (!make_plan(logits, dtype, batch * rows, vocab, sa.sample != 0, &pl))
    SUBSPEC_FAIL(SUBSPEC_ERR_LIMIT, "tree_verify: vocab=%lld needs more than %d slices per row", (long long)vocab,
                 kMaxSplits);
  const size_t n = (size_t)batch * rows * kMaxSplits;
  Part1* p1 = (Part1*)workspace;
  Part2* p2 = (Part2*)((char*)workspace + align_up(n * sizeof(Part1), 256));
  Part3* p3 = (Part3*)((char*)p2 + align_up(n * sizeof(Part2), 256));

  VerifyParams vp;
  vp.vocab = vocab;
  vp.splits = pl.splits;
  vp.chunk = pl.chunk;
  vp.gate_entropy = (verify_method == SUBSPEC_VERIFY_LOSSY && threshold_method == SUBSPEC_GATE_ENTROPY) ? 1 : 0;
  vp.entropy_policy = entropy_policy;
  vp.theta = (float)threshold;
  vp.ln_vocab = vocab > 1 ? (float)log((double)vocab) : 1.0f;
  vp.sample = sa.sample;
  vp.ties_in_accept = (pl.splits > 1 && !vp.gate_entropy && !sa.sample) ? 1 : 0;
  vp.temperature = make_divisor(sa.temperature);
  vp.key[0] = (uint32_t)sa.seed;
  vp.key[1] = (uint32_t)(sa.seed >> 32);
  vp.offset[0] = (uint32_t)sa.offset;
  vp.offset[1] = (uint32_t)(sa.offset >> 32);
  TreeParams tp;
  tp.rows = rows;
  tp.n_nodes = n_nodes;
  tp.root = root;
  tp.skip = skip_nodes;
  tp.eos = eos_token_id;
  tp.method = verify_method;
  tp.gate = threshold_method;
  tp.theta = threshold;
  tp.window = window_size;
  hipStream_t st = (hipStream_t)stream;
  switch (dtype) {
    case SUBSPEC_F32:
      return run_verify<SUBSPEC_F32>(logits, batch, rows, vocab, pl, vp, tp, p1, p2, p3, token_ids, parents, out_tokens,
                                     out_ctx, out_counts, node_target, node_entropy, node_child_prob, st);
    case SUBSPEC_F16:
      return run_verify<SUBSPEC_F16>(logits, batch, rows, vocab, pl, vp, tp, p1, p2, p3, token_ids, parents, out_tokens,
                                     out_ctx, out_counts, node_target, node_entropy, node_child_prob, st);
    default:
      return run_verify<SUBSPEC_BF16>(logits, batch, rows, vocab, pl, vp, tp, p1, p2, p3, token_ids, parents, out_tokens,
                                      out_ctx, out_counts, node_target, node_entropy, node_child_prob, st);
  }
}

extern "C" int subspec_tree_verify(const void* logits, int dtype, int64_t batch, int64_t rows, int64_t vocab,
                                   const int32_t* token_ids, const int32_t* parents, int64_t n_nodes,
                                   int32_t root, int32_t skip_nodes, int64_t eos_token_id,
                                   int verify_method, int threshold_method, double threshold, int32_t window_size,
                                   int entropy_policy, void* workspace, size_t workspace_bytes,
                                   int64_t* out_tokens, int64_t* out_ctx, int32_t* out_counts,
                                   int64_t* node_target, float* node_entropy, float* node_child_prob,
                                   void* stream) {
  const SampleArgs greedy{0, 1.0f, 0, 0};
  return tree_verify_impl(logits, dtype, batch, rows, vocab, token_ids, parents, n_nodes, root, skip_nodes,
                          eos_token_id, verify_method, threshold_method, threshold, window_size, entropy_policy,
                          workspace, workspace_bytes, out_tokens, out_ctx, out_counts, node_target, node_entropy,
                          node_child_prob, greedy, stream);
}

extern "C" int subspec_tree_verify_sample(const void* logits, int dtype, int64_t batch, int64_t rows, int64_t vocab,
                                          const int32_t* token_ids, const int32_t* parents, int64_t n_nodes,
                                          int32_t root, int32_t skip_nodes, int64_t eos_token_id,
                                          int verify_method, int threshold_method, double threshold,
                                          int32_t window_size, int entropy_policy, float temperature, uint64_t seed,
                                          uint64_t offset, void* workspace, size_t workspace_bytes,
                                          int64_t* out_tokens, int64_t* out_ctx, int32_t* out_counts,
                                          int64_t* node_target, float* node_entropy, float* node_child_prob,
                                          void* stream) {
  if (!(temperature > 0.f) || temperature == INFINITY)
    SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "tree_verify_sample: temperature=%g must be positive and finite", (double)temperature);
  const SampleArgs drawn{1, temperature, seed, offset};
  return tree_verify_impl(logits, dtype, batch, rows, vocab, token_ids, parents, n_nodes, root, skip_nodes,
                          eos_token_id, verify_method, threshold_method, threshold, window_size, entropy_policy,
                          workspace, workspace_bytes, out_tokens, out_ctx, out_counts, node_target, node_entropy,
                          node_child_prob, drawn, stream);
}

// ------------------------------------------------------------------ allocation-free variant
// The per-slice partial records (Part1 / Part2 / Part3) of the verifier in a file-scope device array instead of a
// caller-supplied workspace, for callers that cannot allocate.  kStaticVerifyRows logits rows (batch * rows) is the
// limit: 2048 rows x 64 slices x 48 bytes.  Every GPU holds its own copy of the array at its own address, looked up
// once per device; all calls on a GPU share it and calls that overlap there race.  The kernels write every record
// they later read, so the array needs no clearing between calls.
namespace subspec {
constexpr int64_t kStaticVerifyRows = SUBSPEC_TREE_VERIFY_STATIC_MAX_ROWS;
constexpr size_t kStaticVerifyBytes =
    (size_t)kStaticVerifyRows * kMaxSplits * (sizeof(Part1) + sizeof(Part2) + sizeof(Part3)) + 3 * 256;
static __device__ __align__(256) unsigned char scratch[kStaticVerifyBytes];
constexpr int kMaxDevices = 64;
static void* g_scratch_ptr[kMaxDevices];            // device address of `scratch` on each GPU, 0 until looked up
static std::mutex g_scratch_mutex;

static int static_scratch(void** out) {
  int dev = -1;
  SUBSPEC_CHECK_HIP(hipGetDevice(&dev));
  if (dev < 0 || dev >= kMaxDevices) SUBSPEC_FAIL(SUBSPEC_ERR_LIMIT, "tree_verify_static: device %d outside 0..%d", dev, kMaxDevices - 1);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    void* p = nullptr;
    SUBSPEC_CHECK_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    if (!p) SUBSPEC_FAIL(SUBSPEC_ERR_HIP, "tree_verify_static: hipGetSymbolAddress returned a null address");
    g_scratch_ptr[dev] = p;
  }
  *out = g_scratch_ptr[dev];
  return SUBSPEC_OK;
}
}  // namespace subspec

extern "C" int subspec_tree_verify_static(const void* logits, int dtype, int64_t batch, int64_t rows, int64_t vocab,
                                          const int32_t* token_ids, const int32_t* parents, int64_t n_nodes,
                                          int32_t root, int32_t skip_nodes, int64_t eos_token_id,
                                          int verify_method, int threshold_method, double threshold, int32_t window_size,
                                          int entropy_policy, int64_t* out_tokens, int64_t* out_ctx, int32_t* out_counts,
                                          int64_t* node_target, float* node_entropy, float* node_child_prob,
                                          void* stream) {
  if (batch > 0 && rows > 0 && batch * rows > kStaticVerifyRows)
    SUBSPEC_FAIL(SUBSPEC_ERR_LIMIT, "tree_verify_static: batch * rows = %lld exceeds the %lld rows the built-in scratch array holds "
                 "(use subspec_tree_verify with a workspace)", (long long)(batch * rows), (long long)kStaticVerifyRows);
  if (!dtype_ok(dtype)) SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "tree_verify_static: unknown dtype %d", dtype);
  if (!logits || !token_ids || !parents || !out_tokens || !out_ctx || !out_counts || !node_target || !node_entropy ||
      !node_child_prob)
    SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "tree_verify_static: null pointer argument");
  void* ws = nullptr;
  const int rc = static_scratch(&ws);
  if (rc != SUBSPEC_OK) return rc;
  const SampleArgs greedy{0, 1.0f, 0, 0};
  return tree_verify_impl(logits, dtype, batch, rows, vocab, token_ids, parents, n_nodes, root, skip_nodes,
                          eos_token_id, verify_method, threshold_method, threshold, window_size, entropy_policy,
                          ws, kStaticVerifyBytes, out_tokens, out_ctx, out_counts, node_target, node_entropy,
                          node_child_prob, greedy, stream);
}
