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
//           algorithmic bytes = N*K/2 + N*(K/64)*4 (+ activations).  (K of at most 2048 only; longer K: next line.)
// M = 1-16, K > 2048: int4_rows8_kernel, the same MFMA arithmetic with nothing pipelined: every request of a
//           wavefront is issued before its first wait.  This is the shape of a draft level (8 or 16 rows, one workgroup per
//           compute unit), where a pipeline of a few groups is bound by round trips, not by bytes.
//           A K of more than 56 groups over at least 128 tiles (the down projection): int4_rows8_long_kernel, one
//           workgroup per tile over the whole of K, in rounds whose registers refill while they are used.
// M = 2-64: int4_gemm_kernel, v_mfma_f32_16x16x32 with the activations as A and the weight tile as
//           B operand; the 32 k of one MFMA step all come from one quantization group, so the raw
//           accumulator of a group is scaled once.  The wavefronts of a workgroup split K, their
//           partial sums and the split-K partials across workgroups are reduced in a fixed order.
#include "common.h"
#include <algorithm>

namespace subspec {

constexpr int kI4Threads = 256;
constexpr int kGroup = 64;

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
  static __device__ __forceinline__ float to_float(uint32_t bits16) {
    return DT == SUBSPEC_BF16 ? bf16_bits_to_float(bits16) : f16_bits_to_float(bits16);
  }
};
__device__ __forceinline__ uint32_t code_pair(uint32_t w, int shift, uint32_t magic, uint32_t mask = 0x000f000fu) {
  return ((w >> shift) & mask) | magic;
}

// ------------------------------------------------------------------ M = 1
template <int DT>
__global__ __launch_bounds__(kI4Threads) void int4_gemv_kernel(
    const uint16_t* __restrict__ x, const uint2* __restrict__ wq, const uint32_t* __restrict__ sz,
    const uint16_t* __restrict__ bias, const uint16_t* residual, uint16_t* y, int64_t N, int64_t K) {
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
    store_linear_out<DT>(y, n, v, residual);
  }
}

// ------------------------------------------------------------------ 2 <= M <= 64
// y^T is not formed: the activations are the MFMA A operand (rows m) and the weight tile the B
// operand (columns n), so a lane's accumulators all belong to ONE weight row n = lane % 16 and its
// scale / zero is a single word per (tile, group).  v_mfma_f32_16x16x32: one step covers 32 k, the
// k permutation "step s, lane group c, element e -> k = 16c + 8s + e" is applied to both operands.
//
// A workgroup owns up to RT consecutive 16-row weight tiles; its 4 wavefronts split K by GROUP
// (wavefront w takes groups w, w + 4, ... of the workgroup's K range) and never synchronise until
// the end: each one fetches its activation block (L2-resident) through a private LDS stage and its
// weight words from HBM two groups ahead into two register sets, so every wavefront is an
// independent software pipeline.  One activation operand feeds RT + 1 MFMAs: one per tile and
// one against a B operand of ones, which yields the group's activation sums in exactly the
// accumulator layout the zero-point term needs.  The four partial accumulators are summed through
// LDS in wavefront order at the end.
constexpr int kXlStride = kGroup + 8;                          // LDS row stride (elements) of a parked activation block
typedef uint32_t i4_u4 __attribute__((ext_vector_type(4)));
typedef uint32_t i4_u2 __attribute__((ext_vector_type(2)));
typedef __bf16 i4_v8bf __attribute__((ext_vector_type(8)));
typedef _Float16 i4_v8h __attribute__((ext_vector_type(8)));
template <int DT>
__device__ __forceinline__ i4_v4f i4_mfma32(i4_u4 a, i4_u4 b, i4_v4f c) {
  if constexpr (DT == SUBSPEC_BF16)
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(i4_v8bf, a), __builtin_bit_cast(i4_v8bf, b), c, 0, 0, 0);
  else
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(i4_v8h, a), __builtin_bit_cast(i4_v8h, b), c, 0, 0, 0);
}

// SILU (the gate|up projection of a SwiGLU MLP, N = 2F rows: gate rows first, up rows behind them): a workgroup
// owns PAIRS of tiles, (gate tile p, up tile p + F/16), and its output stage writes act[m, f] =
// round(silu(round(gate))) * round(up) to y[M, F] instead of the 2F projections -- the arithmetic of the separate
// activation kernel on the values the plain projection would have stored, one launch and one round trip less.
//
// ROPE (the fused q|k|v projection of an attention block): a workgroup owns the tile pair (j, j + 4) of one head (the
// columns d and d + 64 that the rotate-half form combines), or two consecutive tiles of a value head, and its output
// stage applies the rotary embedding and writes q to [Hq, M, 128] and the K / V rows into the layer's cache: the
// [M, N] projection never travels through memory and the separate rotary launch is gone.
//
// NORM (RMSNorm as the prologue of the projection that consumes it): x is the residual stream itself.  The
// per-element gain is applied where a block is parked in LDS (one rounding of x * gain), the squares are summed on
// the way (every workgroup reads all of x anyway), and 1 / rms -- a per-row scalar -- multiplies the accumulators in
// the output stage:  y = rstd[m] * sum_k round(x[m,k] g[k]) W[n,k].  Only without a K split across workgroups.
constexpr int kEpiPlain = 0, kEpiSilu = 1, kEpiRope = 2;
struct I4Fused {
  const uint16_t* norm_gain;   // NORM: [K]
  float norm_eps;
  // ROPE
  const int32_t* positions;    // [M]
  const int32_t* cache_rows;   // [M]
  uint16_t* q_out;             // [Hq, M, 128]
  KvRowMap kv;                 // where the K / V rows go (contiguous caches or a page pool)
  const float* inv_freq;       // [64] or null
  int hq, hkv;
  float log2_theta;
};

// XHALF (at most 8 activation rows, MT = 1): only rows 0..7 of a block are fetched, scaled and parked; rows 8..15 of the
// LDS stages are cleared once.  Half the activation traffic and half the prologue arithmetic of a 16-row block.
template <int DT, int MT, int RT, int EPI = kEpiPlain, bool NORM = false, bool XHALF = false>
__global__ __launch_bounds__(kI4Threads) void int4_gemm_kernel(
    const uint16_t* __restrict__ x, const uint2* __restrict__ wq, const uint32_t* __restrict__ sz,
    const uint16_t* __restrict__ bias, const uint16_t* residual, uint16_t* y, float* __restrict__ partial, int M, int64_t N,
    int K, int splits, int groups_per_split, I4Fused fz) {
  constexpr bool SILU = EPI == kEpiSilu, ROPE = EPI == kEpiRope, PAIRED = EPI != kEpiPlain;
  constexpr int NW = 4;                                          // wavefronts of the workgroup; wavefront w takes groups w, w + 4, ...
  __shared__ float sq_s[NORM ? NW * MT * 16 : 1];                 // NORM: per wavefront, per row: sum of squares of its groups
  __shared__ float rstd_s[NORM ? MT * 16 : 1];
  // 4 wavefronts x 2 stages of a [16*MT][64] activation block; reused for the final reduction
  // (two rounds of one accumulator tile set per wavefront)
  constexpr int kStageBytes = 4 * 2 * MT * 16 * kXlStride * 2, kRedBytes = 2 * NW * MT * 256 * 4;
  __shared__ __attribute__((aligned(16))) unsigned char lds_raw[kStageBytes > kRedBytes ? kStageBytes : kRedBytes];
  uint16_t* const xstage = (uint16_t*)lds_raw;
  float* const red = (float*)lds_raw;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int ln = lane & 15, c = lane >> 4;
  const int G = K / kGroup;
  const int n_tiles = (int)(N / 16);
  const int ks = blockIdx.y;
  const int g_begin = ks * groups_per_split, g_end = min(G, g_begin + groups_per_split);
  const int g_first = g_begin + wave;                            // this wavefront's groups: g_first + 4j
  const int nj = g_first < g_end ? (g_end - g_first + NW - 1) / NW : 0;

  // tiles [tile0, tile0 + ntl) of this workgroup: an even split of all tiles (SILU / ROPE: of all tile pairs) over the grid
  const int n_units = PAIRED ? n_tiles / 2 : n_tiles;
  // (32-bit unsigned quotients: the host refuses N / 16 >= 65536, so the products fit; a 64-bit division would be a
  // few hundred instructions on every wavefront's way to its first request)
  const int unit0 = (int)((uint32_t)blockIdx.x * (uint32_t)n_units / gridDim.x);
  const int n_own = (int)(((uint32_t)blockIdx.x + 1u) * (uint32_t)n_units / gridDim.x) - unit0;
  const int tile0 = unit0;                                                             // plain: first tile
  const int ntl = PAIRED ? 2 * n_own : n_own;                                          // 1 .. RT
  const int qk_units = ROPE ? (fz.hq + fz.hkv) * 4 : 0;                                // ROPE: pairs of the rotated heads
  auto tile_of = [&](int t) {
    if constexpr (SILU) return unit0 + (t >> 1) + (t & 1) * (n_tiles / 2);
    if constexpr (ROPE) {
      const int u = unit0 + (t >> 1);
      return u < qk_units ? (u >> 2) * 8 + (u & 3) + (t & 1) * 4 : 2 * u + (t & 1);   // value heads: tiles 2u, 2u + 1
    }
    return tile0 + t;
  };

  i4_v4f acc[RT][MT];
#pragma unroll
  for (int t = 0; t < RT; ++t)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[t][mt] = i4_v4f{0.f, 0.f, 0.f, 0.f};

  // Loads go through buffer descriptors: the builtin calls keep their place in the program (plain
  // loads feeding a loop-carried value get merged into one load at the loop head, which would undo
  // the prefetch distance), uniform address parts ride in the scalar offset, and a request outside
  // the tensor returns zeros instead of faulting.
  //
  // Activations: an MFMA operand wants lane (ln, c) to hold row ln, which no coalesced load can
  // deliver (adjacent lanes would sit a whole row apart).  Each wavefront therefore fetches its
  // group's [16*MT rows][64 k] block with 8 lanes per 128-byte row segment, parks it in a
  // wavefront-private LDS stage (row stride 144 bytes: conflict-free 16-byte reads) and reads the
  // operands back from there.  No other wavefront touches the stage, so no barrier is involved.
  // Rows past M read zeros and only feed accumulator rows that are never stored; requests past
  // the last group re-read it and meet a zero scale.
  const __amdgpu_buffer_rsrc_t x_rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)x, 0, M * K * 2, 0x00027000);
  const __amdgpu_buffer_rsrc_t w_rsrc =
      __builtin_amdgcn_make_buffer_rsrc((void*)wq, 0, (int)(n_tiles * (int64_t)G * 512), 0x00027000);
  const __amdgpu_buffer_rsrc_t sz_rsrc =
      __builtin_amdgcn_make_buffer_rsrc((void*)sz, 0, (int)(n_tiles * (int64_t)G * 64), 0x00027000);
  const __amdgpu_buffer_rsrc_t g_rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)(NORM ? fz.norm_gain : x), 0, K * 2, 0x00027000);
  static_assert(!XHALF || MT == 1, "the 8-row block exists for one 16-row tile only");
  constexpr int kXg = XHALF ? 1 : MT * 2;                        // 16-byte pieces per lane of one group block
  const int xg_off = ((lane >> 3) * K + (lane & 7) * 8) * 2;     // byte offset of piece 0; piece i is 8 rows further
  uint16_t* const xl = xstage + wave * (2 * MT * 16 * kXlStride);  // this wavefront's two stages
  const int xl_write = (lane >> 3) * kXlStride + (lane & 7) * 8;
  const int xl_read = ln * kXlStride + c * 16;
  int wofs[RT];                                                  // (tile, group 0) in units of groups
#pragma unroll
  for (int t = 0; t < RT; ++t) wofs[t] = tile_of(min(t, ntl - 1)) * G;

  // Activation blocks on their way from global memory to LDS: requested kXSlots steps before they are parked (a
  // block that is parked one step after its request makes every step wait for a whole round trip to L2).
  constexpr int kXSlots = MT == 4 ? 1 : 2;   // 64 rows: one (with two the compiler waits for every request at the top of the loop body)
  i4_u4 xg[kXSlots][kXg];
  i4_u4 gq[kXSlots];                                             // NORM: the gains of the lane's 8 k of the block on its way
  float sq[kXg];                                                 // NORM: sum of squares of rows (lane >> 3) + 8 i over this wavefront's groups
  (void)gq; (void)sq;
  if constexpr (NORM) {
#pragma unroll
    for (int i = 0; i < kXg; ++i) sq[i] = 0.f;
  }
  // Weight words on their way: two groups ahead.  With one tile per workgroup they rotate through THREE register
  // slots, so that a request never targets the slot the current step still reads: the compiler issues the request
  // before those reads, gives it other registers and copies them at the end of the loop body, and that copy waits for
  // EVERY request in flight, once per trip.  With more tiles it orders reads and requests so that two slots do.
  constexpr int kWSlots = RT == 1 ? 3 : 2;
  i4_u2 wbuf[kWSlots][RT];
  uint32_t szbuf[kWSlots][RT];
  // Both constants of ((w >> s) & mask) | magic as run-time values (M >> 30 is zero): with two
  // literals the compiler emits v_and + v_or, with a scalar and a vector register operand one v_and_or_b32.
  // (xg_off >> 31 is zero too and lives in a vector register.)
  const uint32_t kmask = 0x000f000fu | (uint32_t)(M >> 30), kmagic = I4<DT>::kMagic | ((uint32_t)xg_off >> 31);
  const uint32_t one2 = DT == SUBSPEC_BF16 ? 0x3f803f80u : 0x3c003c00u;
  const i4_u4 ones = i4_u4{one2, one2, one2, one2};

#define SUBSPEC_I4_FETCH_X(XS, J)                                                                       \
  {                                                                                                     \
    const int kc = min(g_first + 4 * (J), G - 1) * (kGroup * 2);                                        \
    _Pragma("unroll") for (int i = 0; i < kXg; ++i)                                                     \
      xg[XS][i] = __builtin_amdgcn_raw_buffer_load_b128(x_rsrc, xg_off + i * 16 * K, kc, 0);            \
    if constexpr (NORM) gq[XS] = __builtin_amdgcn_raw_buffer_load_b128(g_rsrc, (lane & 7) * 16, kc, 0); \
  }
  // JP: index of the group being parked among this wavefront's groups (its squares count only if it exists)
#define SUBSPEC_I4_PARK_X(SLOT, JP)                                                                     \
  _Pragma("unroll") for (int i = 0; i < kXg; ++i) {                                                     \
    i4_u4 piece = xg[(SLOT) % kXSlots][i];                                                              \
    if constexpr (NORM) {                                                                               \
      float f_[8], g_[8];                                                                               \
      unpack8<DT>(piece, f_);                                                                           \
      unpack8<DT>(gq[(SLOT) % kXSlots], g_);                                                            \
      float ss_ = 0.f;                                                                                  \
      _Pragma("unroll") for (int e = 0; e < 8; ++e) { ss_ = fmaf(f_[e], f_[e], ss_); f_[e] *= g_[e]; }  \
      sq[i] += (JP) < nj ? ss_ : 0.f;                                                                   \
      piece = pack8<DT>(f_);                                                                            \
    }                                                                                                   \
    *(i4_u4*)(&xl[(SLOT) * (MT * 16 * kXlStride) + i * 8 * kXlStride + xl_write]) = piece;              \
  }
#define SUBSPEC_I4_FETCH_W(SLOT, J, T)                                                                  \
  {                                                                                                     \
    const int g = wofs[T] + min(g_first + 4 * (J), G - 1);                                              \
    wbuf[SLOT][T] = __builtin_amdgcn_raw_buffer_load_b64(w_rsrc, lane * 8, g * 512, 0);                 \
    szbuf[SLOT][T] = __builtin_amdgcn_raw_buffer_load_b32(sz_rsrc, ln * 4, g * 64, 0);                  \
  }
  // Step J works on LDS stage SLOT = J & 1.  Once its operands are in registers the stage is free:
  // the block of group J + 2 (requested kXSlots steps ago) is parked there and group J + 2 + kXSlots requested.
#define SUBSPEC_I4_STEP(SLOT, WS, WNEXT, J)                                                             \
  {                                                                                                     \
    const bool step_live = (J) < nj;                /* a dead step multiplies by a zero scale: no branch */ \
    i4_u4 xa[MT][2];                                                                                    \
    _Pragma("unroll") for (int mt = 0; mt < MT; ++mt) {                                                 \
      const uint16_t* xr = &xl[(SLOT) * (MT * 16 * kXlStride) + mt * 16 * kXlStride + xl_read];         \
      xa[mt][0] = *(const i4_u4*)xr;                                                                    \
      xa[mt][1] = *(const i4_u4*)(xr + 8);                                                              \
    }                                                                                                   \
    SUBSPEC_I4_PARK_X(SLOT, (J) + 2);                                                                   \
    SUBSPEC_I4_FETCH_X((SLOT) % kXSlots, (J) + 2 + kXSlots);                                            \
    __builtin_amdgcn_sched_barrier(0);              /* keep the requests here: a full step ahead of their use */ \
    i4_v4f xs[MT];                                  /* sum of the group's activations, rows 16mt + 4c + rr */ \
    _Pragma("unroll") for (int mt = 0; mt < MT; ++mt) {                                                 \
      xs[mt] = i4_mfma32<DT>(xa[mt][0], ones, i4_v4f{0.f, 0.f, 0.f, 0.f});                              \
      xs[mt] = i4_mfma32<DT>(xa[mt][1], ones, xs[mt]);                                                  \
    }                                                                                                   \
    _Pragma("unroll") for (int t = 0; t < RT; ++t) {                                                    \
      const uint32_t w0 = wbuf[WS][t].x, w1 = wbuf[WS][t].y, szw = szbuf[WS][t];                        \
      const i4_u4 b0 = i4_u4{code_pair(w0, 0, kmagic, kmask), code_pair(w0, 4, kmagic, kmask),          \
                             code_pair(w0, 8, kmagic, kmask), code_pair(w0, 12, kmagic, kmask)};        \
      const i4_u4 b1 = i4_u4{code_pair(w1, 0, kmagic, kmask), code_pair(w1, 4, kmagic, kmask),          \
                             code_pair(w1, 8, kmagic, kmask), code_pair(w1, 12, kmagic, kmask)};        \
      const float sc = (step_live && t < ntl) ? f16_bits_to_float(szw & 0xffffu) : 0.f;                 \
      const float szo = -sc * (f16_bits_to_float(szw >> 16) + I4<DT>::kOffset);                         \
      SUBSPEC_I4_FETCH_W(WNEXT, (J) + 2, t);                                                            \
      _Pragma("unroll") for (int mt = 0; mt < MT; ++mt) {                                               \
        i4_v4f raw = i4_mfma32<DT>(xa[mt][0], b0, i4_v4f{0.f, 0.f, 0.f, 0.f});                          \
        raw = i4_mfma32<DT>(xa[mt][1], b1, raw);                                                        \
        _Pragma("unroll") for (int rr = 0; rr < 4; ++rr)                                                \
          acc[t][mt][rr] = fmaf(sc, raw[rr], fmaf(szo, xs[mt][rr], acc[t][mt][rr]));                    \
      }                                                                                                 \
    }                                                                                                   \
    __builtin_amdgcn_sched_barrier(0);                                                                  \
  }

  if constexpr (XHALF) {
    // rows 8..15 of both stages stay zero for the whole kernel
    *(i4_u4*)(&xl[8 * kXlStride + xl_write]) = i4_u4{0u, 0u, 0u, 0u};
    *(i4_u4*)(&xl[(MT * 16 * kXlStride) + 8 * kXlStride + xl_write]) = i4_u4{0u, 0u, 0u, 0u};
  }
  // The requests before the loop are issued in the order the loop issues them (activation block, then the weights of
  // the group two steps back), so that the first trip finds the same queue of outstanding requests as every later
  // one: the compiler gives each wait ONE count that must hold on every path into the loop, and a prologue that ends
  // with the activation requests makes that count "nothing may be outstanding but the newest block" on every trip --
  // the weights would be waited for one step after their request, whatever the distance in the source.
  SUBSPEC_I4_FETCH_X(0, 0);
  if constexpr (kXSlots == 2) SUBSPEC_I4_FETCH_X(1, 1);
  SUBSPEC_I4_PARK_X(0, 0);
  if constexpr (kXSlots == 2) { SUBSPEC_I4_FETCH_X(0, 2); } else { SUBSPEC_I4_FETCH_X(0, 1); }
#pragma unroll
  for (int t = 0; t < RT; ++t) SUBSPEC_I4_FETCH_W(0, 0, t);
  SUBSPEC_I4_PARK_X(1, 1);
  if constexpr (kXSlots == 2) { SUBSPEC_I4_FETCH_X(1, 3); } else { SUBSPEC_I4_FETCH_X(0, 2); }
#pragma unroll
  for (int t = 0; t < RT; ++t) SUBSPEC_I4_FETCH_W(1, 1, t);
  if constexpr (RT == 1) {
    // step J: LDS stage J % 2, weight slot J % 3, request for group J + 2 into slot (J + 2) % 3
    for (int j = 0; j < nj; j += 6) {
      SUBSPEC_I4_STEP(0, 0, 2, j);
      SUBSPEC_I4_STEP(1, 1, 0, j + 1);
      if (j + 2 >= nj) break;
      SUBSPEC_I4_STEP(0, 2, 1, j + 2);
      SUBSPEC_I4_STEP(1, 0, 2, j + 3);
      if (j + 4 >= nj) break;
      SUBSPEC_I4_STEP(0, 1, 0, j + 4);
      SUBSPEC_I4_STEP(1, 2, 1, j + 5);
    }
  } else {
    for (int j = 0; j < nj; j += 2) {
      SUBSPEC_I4_STEP(0, 0, 0, j);
      SUBSPEC_I4_STEP(1, 1, 1, j + 1);
    }
  }
  if constexpr (NORM) {
    // the eight lanes that share a row hold its squares over different k; one value per (wavefront, row) goes to LDS
#pragma unroll
    for (int i = 0; i < kXg; ++i) {
      float v = sq[i];
      v += __shfl_xor(v, 1, kWave);
      v += __shfl_xor(v, 2, kWave);
      v += __shfl_xor(v, 4, kWave);
      if ((lane & 7) == 0) sq_s[wave * (MT * 16) + (lane >> 3) + 8 * i] = v;
    }
    if constexpr (XHALF) {
      if ((lane & 7) == 0) sq_s[wave * (MT * 16) + (lane >> 3) + 8] = 0.f;
    }
  }
  __syncthreads();                                               // the stages are reused for the reduction below
  if constexpr (NORM) {
    // ordered before its first use by the barrier of the first reduction round
    if (tid < MT * 16)
    {
      float ss = 0.f;
#pragma unroll
      for (int w = 0; w < NW; ++w) ss += sq_s[w * MT * 16 + tid];
      rstd_s[tid] = rsqrtf(ss / (float)K + fz.norm_eps);
    }
  }
#undef SUBSPEC_I4_PARK_X
#undef SUBSPEC_I4_FETCH_X
#undef SUBSPEC_I4_FETCH_W
#undef SUBSPEC_I4_STEP

  // ---- sum the four wavefronts' partial accumulators in wavefront order (0, 1, 2, 3), one tile per
  // round.  LDS holds two rounds, so a round needs one barrier; wavefront w finishes the activation
  // row blocks mt = w, w + 4, ... of the tile, so the sums and stores are spread over the workgroup.
  // accumulator layout: rows m = 16*mt + 4*c + rr, column n = 16*tile + ln
  float held[MT][4];                                             // SILU / ROPE: the rounded values of the even tile between two rounds
  (void)held;
#pragma unroll
  for (int t = 0; t < RT; ++t) {
    if (t >= ntl) break;                                         // uniform
    float* stage = red + (t & 1) * (NW * MT * 256);
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) *(i4_v4f*)(&stage[((wave * MT + mt) * 64 + lane) * 4]) = acc[t][mt];
    __syncthreads();                                             // round t written; round t - 1 fully read
    const int64_t n = (int64_t)tile_of(t) * 16 + ln;
    const float bv = (splits == 1 && bias) ? I4<DT>::to_float(bias[n]) : 0.f;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      if ((mt & 3) != wave) continue;                            // uniform
      i4_v4f v = *(const i4_v4f*)(&stage[((0 * MT + mt) * 64 + lane) * 4]);
#pragma unroll
      for (int w = 1; w < NW; ++w) {
        const i4_v4f o = *(const i4_v4f*)(&stage[((w * MT + mt) * 64 + lane) * 4]);
#pragma unroll
        for (int rr = 0; rr < 4; ++rr) v[rr] += o[rr];
      }
      if constexpr (NORM) {
#pragma unroll
        for (int rr = 0; rr < 4; ++rr) v[rr] *= rstd_s[mt * 16 + c * 4 + rr];
      }
      if constexpr (PAIRED) {
        // even round: the first tile of the pair, kept in registers; odd round: its partner, same wavefront, same lanes
        if ((t & 1) == 0) {
#pragma unroll
          for (int rr = 0; rr < 4; ++rr) held[mt][rr] = Elem<DT>::round(v[rr] + bv);
        } else if constexpr (SILU) {
          const int64_t f = (int64_t)(unit0 + (t >> 1)) * 16 + ln;
#pragma unroll
          for (int rr = 0; rr < 4; ++rr) {
            const int m = mt * 16 + c * 4 + rr;
            if (m >= M) continue;
            const float g = held[mt][rr], u = Elem<DT>::round(v[rr] + bv);
            Elem<DT>::store(y, (int64_t)m * (N / 2) + f, Elem<DT>::round(g / (1.f + __expf(-g))) * u);
          }
        } else {
          const int u = unit0 + (t >> 1);
          if (u < qk_units) {
            // rotary pair (d, d + 64) of head u / 4, d = 16 (u % 4) + ln; t * cos + rotate_half(t) * sin with each
            // product and the sum rounded like the eager tensor ops
            const int head = u >> 2, d = (u & 3) * 16 + ln;
            const float inv_freq = fz.inv_freq ? fz.inv_freq[d] : exp2f(-(float)(2 * d) / 128.f * fz.log2_theta);
#pragma unroll
            for (int rr = 0; rr < 4; ++rr) {
              const int m = mt * 16 + c * 4 + rr;
              if (m >= M) continue;
              float sn, cs;
              sincosf((float)fz.positions[m] * inv_freq, &sn, &cs);
              cs = Elem<DT>::round(cs);
              sn = Elem<DT>::round(sn);
              const float lo = held[mt][rr], hi = Elem<DT>::round(v[rr] + bv);
              const float o_lo = Elem<DT>::round(lo * cs) + Elem<DT>::round(-hi * sn);
              const float o_hi = Elem<DT>::round(hi * cs) + Elem<DT>::round(lo * sn);
              uint16_t *dst, *unused;
              if (head < fz.hq) {
                dst = fz.q_out + ((int64_t)head * M + m) * 128;
              } else if (!kv_row_ptrs(fz.kv, head - fz.hq, fz.cache_rows[m], &dst, &unused)) {
                continue;                                        // a row outside the layer's cache is dropped
              }
              Elem<DT>::store(dst, d, o_lo);
              Elem<DT>::store(dst, d + 64, o_hi);
            }
          } else {
            // two consecutive tiles of a value head: copied
            const int vt = 2 * (u - qk_units), kvh = vt >> 3, d = (vt & 7) * 16 + ln;
#pragma unroll
            for (int rr = 0; rr < 4; ++rr) {
              const int m = mt * 16 + c * 4 + rr;
              if (m >= M) continue;
              uint16_t *dst, *unused;
              if (!kv_row_ptrs(fz.kv, kvh, fz.cache_rows[m], &unused, &dst)) continue;
              Elem<DT>::store(dst, d, held[mt][rr]);
              Elem<DT>::store(dst, d + 16, v[rr] + bv);
            }
          }
        }
      } else {
#pragma unroll
        for (int rr = 0; rr < 4; ++rr) {
          const int m = mt * 16 + c * 4 + rr;
          if (m >= M) continue;
          if (splits == 1) store_linear_out<DT>(y, (int64_t)m * N + n, v[rr] + bv, residual);
          else partial[((int64_t)ks * M + m) * N + n] = v[rr];
        }
      }
    }
  }
}

// ------------------------------------------------------------------ 1 <= M <= 16, at most 56 groups per workgroup
// Nothing is pipelined.  Eight wavefronts split the workgroup's K range by group (wavefront w: groups w, w + 8, ..., at
// most kR8Groups of them); each issues EVERY request it will need before its first wait -- its gains, its activation
// blocks, the (scale, zero) words of all its tiles, the weight words of its first RTR tiles -- parks the activation blocks
// (L2 hits, requested first, so waiting for them does not wait for the weights) in private LDS stages while the weights
// are on their way from HBM, and then runs its steps against registers.  With about one workgroup per compute unit
// (the projections of a draft level) a short pipeline has nothing to hide a round trip behind and pays one per two
// steps; here the wavefront pays one.  The workgroup's tiles are taken in NR rounds of RTR: a step of round r hands its
// weight registers to the same step of round r + 1, so the wavefront keeps kR8Groups * RTR requests in flight until the
// last round, and the parked activations serve all rounds.  Many tiles go in rounds of two: nothing can be multiplied
// before the first round's words are there, so a first round of five tiles (half of the SwiGLU projection's ten) is
// 6.8 us of pure transfer in front of 9.7 us of steps, a first round of two 3 us (37888 x 3584: 22.9 -> 20.2 us per
// call); rounds of one tile gain nothing more (14 requests per wavefront in flight cover the latency, 7 just do).
//
// LDS: a stage holds the 8 rows x 128 bytes of one group, 16-byte piece p of row r at position p ^ (r % 8) (conflict-free
// reads without padding); MFMA rows 8..15 read a block of zeros.  R = 2 (9 to 16 rows): stages of 16 rows, every lane
// fetches and parks two pieces (rows prow and prow + 8), and wavefront m finishes rows m and m + 8.  (scale, zero): a group's 16 words are 64 bytes, and one
// request per (group, tile) would be half of all requests for a ninth of the bytes, so lane group c fetches the words
// of steps c and 4 + c, two requests per tile, and a step picks its word up from lane group J % 4 with a cross-lane read.
//
// Output stage: every wavefront leaves rows 0..7 of its accumulators in LDS, and after one barrier wavefront m finishes
// row m: a lane sums the eight partials of its element in wavefront order and runs the output stage (plain / SwiGLU /
// rotary, as in int4_gemm_kernel) once.
constexpr int kR8Waves = 8, kR8Groups = 7, kR8Threads = kR8Waves * 64;
// Cache policy of this kernel's weight requests (the auxiliary operand of the buffer-load builtins, bit 1 =
// non-temporal): every weight byte is read once per launch, so it is fetched as streaming data that does not displace
// the activations and the other launches' lines in the L2 (37888 x 3584, 8 rows, from HBM: 20.1 -> 18.7 us per call).
// The same hint changes nothing in the pipelined kernel at 16 or 64 rows and costs the dense kernels 15 to 25 %: their
// wavefronts fetch each 128-byte line with two requests (a lane's 32 bytes are two 16-byte loads), and a streamed line
// does not wait in the first-level cache for the second one.  A request of this kernel covers whole lines.
constexpr int kStream = 2;
template <int DT, int RTR, int NR, int EPI, bool NORM, int R = 1>
__global__ __launch_bounds__(kR8Threads) void int4_rows8_kernel(
    const uint16_t* __restrict__ x, const uint2* __restrict__ wq, const uint32_t* __restrict__ sz,
    const uint16_t* __restrict__ bias, const uint16_t* residual, uint16_t* y, float* __restrict__ partial, int M, int64_t N,
    int K, int splits, int groups_per_split, I4Fused fz) {
  // Every argument is wanted in a scalar register HERE: left alone, the compiler fetches the fields of the parameter
  // block where they are first used -- several batches with a wait each before the first request, and more in the
  // output stage (positions, cache rows, the cache map), each a round trip to the scalar cache that is cold at every launch.
  asm volatile("" ::"s"(x), "s"(wq), "s"(sz), "s"(bias), "s"(residual), "s"(y), "s"(partial), "s"(M), "s"(N), "s"(K), "s"(splits),
               "s"(groups_per_split));
  if constexpr (NORM) asm volatile("" ::"s"(fz.norm_gain), "s"(fz.norm_eps));
  if constexpr (EPI == kEpiRope)
    asm volatile("" ::"s"(fz.positions), "s"(fz.cache_rows), "s"(fz.q_out), "s"(fz.kv.k_cache), "s"(fz.kv.v_cache),
                 "s"(fz.kv.seq_stride), "s"(fz.kv.page_table), "s"(fz.kv.page_shift), "s"(fz.kv.max_pages), "s"(fz.kv.hkv),
                 "s"(fz.kv.page_elems), "s"(fz.inv_freq), "s"(fz.hq), "s"(fz.hkv), "s"(fz.log2_theta));
  constexpr bool SILU = EPI == kEpiSilu, ROPE = EPI == kEpiRope, PAIRED = EPI != kEpiPlain;
  constexpr int RT = RTR * NR, NW = kR8Waves, NG = kR8Groups;
  static_assert(NG <= 8, "two (scale, zero) requests per tile cover eight steps");
  static_assert(NG * 8 <= 64, "one gain piece per lane");
  static_assert(R == 1 || R == 2, "8 or 16 activation rows");
  constexpr int kStage = R * 1024;                               // a group's activation block: 8 R rows x 128 bytes
  constexpr int kStageBytes = NW * NG * (kStage + 128) + NW * 16;  // stages, gains, one block of zeros per wavefront
  constexpr int kRedBytes = RT * NW * 32 * R * 16;                 // rows 0..8 R - 1 of every wavefront's accumulators
  __shared__ __attribute__((aligned(16))) unsigned char lds_raw[kStageBytes > kRedBytes ? kStageBytes : kRedBytes];
  __shared__ float sq_s[NORM ? NW * 8 * R : 1];                  // NORM: per wavefront, per row: sum of squares over its groups
  __shared__ float rstd_s[NORM ? 8 * R : 1];
  float* const red = (float*)lds_raw;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int ln = lane & 15, c = lane >> 4;
  const int G = K / kGroup;
  const int n_tiles = (int)(N / 16);
  const int ks = blockIdx.y;
  const int g_begin = ks * groups_per_split, g_end = min(G, g_begin + groups_per_split);
  const int g_first = g_begin + wave;
  const int nj = g_first < g_end ? (g_end - g_first + NW - 1) / NW : 0;      // <= NG (the host's plan)

  // tiles of this workgroup: an even split of all tiles (SILU / ROPE: of all tile pairs) over the grid; 32-bit unsigned
  // quotients (the host refuses N / 16 >= 65536, so the products fit)
  const int n_units = PAIRED ? n_tiles / 2 : n_tiles;
  const int unit0 = (int)((uint32_t)blockIdx.x * (uint32_t)n_units / gridDim.x);
  const int n_own = (int)(((uint32_t)blockIdx.x + 1u) * (uint32_t)n_units / gridDim.x) - unit0;
  const int ntl = PAIRED ? 2 * n_own : n_own;                    // 1 .. RT
  const int qk_units = ROPE ? (fz.hq + fz.hkv) * 4 : 0;
  auto tile_of = [&](int t) {
    if constexpr (SILU) return unit0 + (t >> 1) + (t & 1) * (n_tiles / 2);
    if constexpr (ROPE) {
      const int u = unit0 + (t >> 1);
      return u < qk_units ? (u >> 2) * 8 + (u & 3) + (t & 1) * 4 : 2 * u + (t & 1);
    }
    return unit0 + t;
  };

  const __amdgpu_buffer_rsrc_t x_rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)x, 0, M * K * 2, 0x00027000);
  const __amdgpu_buffer_rsrc_t w_rsrc =
      __builtin_amdgcn_make_buffer_rsrc((void*)wq, 0, (int)(n_tiles * (int64_t)G * 512), 0x00027000);
  const __amdgpu_buffer_rsrc_t sz_rsrc =
      __builtin_amdgcn_make_buffer_rsrc((void*)sz, 0, (int)(n_tiles * (int64_t)G * 64), 0x00027000);
  const __amdgpu_buffer_rsrc_t g_rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)(NORM ? fz.norm_gain : x), 0, K * 2, 0x00027000);
  const int prow = lane >> 3, ppiece = lane & 7;                 // the lane's row and 16-byte piece of an activation block
  const int xg_off = (prow * K + ppiece * 8) * 2;                // rows past M read zeros (outside the descriptor)
  int wofs[RT];                                                  // (tile, group 0) in units of groups; tiles past ntl repeat the last
#pragma unroll
  for (int t = 0; t < RT; ++t) wofs[t] = tile_of(min(t, ntl - 1)) * G;
  // both constants of ((w >> s) & mask) | magic as run-time values, so that the compiler emits one v_and_or_b32
  const uint32_t kmask = 0x000f000fu | (uint32_t)(M >> 30), kmagic = I4<DT>::kMagic | ((uint32_t)xg_off >> 31);
  const uint32_t one2 = DT == SUBSPEC_BF16 ? 0x3f803f80u : 0x3c003c00u;
  const i4_u4 ones = i4_u4{one2, one2, one2, one2};

  unsigned char* const stages = lds_raw + wave * (NG * kStage);
  unsigned char* const gains = lds_raw + NW * NG * kStage + wave * (NG * 128);
  unsigned char* const zeros = lds_raw + NW * NG * (kStage + 128) + wave * 16;

  // ---- every request
  i4_u4 gpiece;
  (void)gpiece;
  if constexpr (NORM) {                                          // piece q = 8 J + p of the wavefront's gains: lane q
    const int q = min(lane, NG * 8 - 1);
    gpiece = __builtin_amdgcn_raw_buffer_load_b128(g_rsrc, (q & 7) * 16, min(g_first + NW * (q >> 3), G - 1) * (kGroup * 2), 0);
  }
  i4_u4 xall[NG][R];                                             // R = 2: rows prow and prow + 8
#pragma unroll
  for (int J = 0; J < NG; ++J)
#pragma unroll
    for (int h = 0; h < R; ++h)
      xall[J][h] = __builtin_amdgcn_raw_buffer_load_b128(x_rsrc, xg_off + h * 8 * K * 2, min(g_first + NW * J, G - 1) * (kGroup * 2), 0);
  // the activation requests stay ahead of all others: a wait for a block that was requested after the weights would
  // be a wait for the weights
  __builtin_amdgcn_sched_barrier(0);
  uint32_t szq[RT][2];
#pragma unroll
  for (int t = 0; t < RT; ++t)
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int g = wofs[t] + min(g_first + NW * min(4 * h + c, NG - 1), G - 1);
      szq[t][h] = __builtin_amdgcn_raw_buffer_load_b32(sz_rsrc, ln * 4 + g * 64, 0, kStream);
    }
  i4_u2 wall[NG][RTR];
#pragma unroll
  for (int J = 0; J < NG; ++J)
#pragma unroll
    for (int tt = 0; tt < RTR; ++tt)
      wall[J][tt] = __builtin_amdgcn_raw_buffer_load_b64(w_rsrc, lane * 8, (wofs[tt] + min(g_first + NW * J, G - 1)) * 512, kStream);
  // What the output stage adds to this thread's elements (wavefront w finishes rows w and w + 8, lane group c the items
  // c, c + 4, ...): requested here, behind everything else, so that the output stage does not end in a round trip of its own.
  constexpr int kItems = PAIRED ? RT / 2 : RT;
  constexpr int kOut = (kItems + 3) / 4;
  // (The 16-bit words are kept as they come and converted where they are used: an instruction that touches a loaded
  // value here would wait for every request issued before it.  Elements this thread does not own repeat one it may read.)
  uint32_t res_pre[kOut][R], bias_pre[kOut];
#pragma unroll
  for (int io = 0; io < kOut; ++io) {
    bias_pre[io] = 0u;
#pragma unroll
    for (int mi = 0; mi < R; ++mi) res_pre[io][mi] = 0u;
  }
  uint32_t bias1_pre[kOut];                                      // paired tiles: the second tile's bias
  int pos_pre[R], crow_pre[R];                                   // rotary: position and cache row of the thread's rows
#pragma unroll
  for (int io = 0; io < kOut; ++io) bias1_pre[io] = 0u;
#pragma unroll
  for (int mi = 0; mi < R; ++mi) { pos_pre[mi] = 0; crow_pre[mi] = 0; }
  (void)bias1_pre; (void)pos_pre; (void)crow_pre;
  // No branch around a request: one that is issued on one path only makes the compiler wait for ALL requests in flight
  // where the paths join.  A tensor that is not there is replaced by the activations' first element.
  const uint16_t* const bias_src = bias ? bias : x;
  const uint16_t* const res_src = residual ? residual : x;
  const int64_t bias_on = bias ? 1 : 0, res_on = residual ? 1 : 0;
  if constexpr (!PAIRED) {
#pragma unroll
    for (int io = 0; io < kOut; ++io) {
      const int64_t n0 = (int64_t)tile_of(min(io * 4 + c, ntl - 1)) * 16 + ln;
      bias_pre[io] = bias_src[n0 * bias_on];
#pragma unroll
      for (int mi = 0; mi < R; ++mi) res_pre[io][mi] = res_src[((int64_t)min(wave + 8 * mi, M - 1) * N + n0) * res_on];
    }
  } else {
#pragma unroll
    for (int io = 0; io < kOut; ++io) {
      const int t0 = 2 * min(io * 4 + c, ntl / 2 - 1);
      bias_pre[io] = bias_src[((int64_t)tile_of(t0) * 16 + ln) * bias_on];
      bias1_pre[io] = bias_src[((int64_t)tile_of(t0 + 1) * 16 + ln) * bias_on];
    }
    if constexpr (ROPE) {
#pragma unroll
      for (int mi = 0; mi < R; ++mi) {
        pos_pre[mi] = fz.positions[min(wave + 8 * mi, M - 1)];
        crow_pre[mi] = fz.cache_rows[min(wave + 8 * mi, M - 1)];
      }
    }
  }

  __builtin_amdgcn_sched_barrier(0);
  // ---- park the activation blocks
  if (lane == 0) *(i4_u4*)zeros = i4_u4{0u, 0u, 0u, 0u};
  if constexpr (NORM) {
    if (lane < NG * 8) *(i4_u4*)(gains + lane * 16) = gpiece;
  }
  float sq[R];                                                   // NORM: squares of rows prow (+ 8) over this wavefront's groups
#pragma unroll
  for (int h = 0; h < R; ++h) sq[h] = 0.f;
  (void)sq;
#pragma unroll
  for (int J = 0; J < NG; ++J) {
#pragma unroll
    for (int h = 0; h < R; ++h) {
      i4_u4 piece = xall[J][h];
      if constexpr (NORM) {
        float f_[8], g_[8];
        unpack8<DT>(piece, f_);
        unpack8<DT>(*(const i4_u4*)(gains + (J * 8 + ppiece) * 16), g_);
        float ss_ = 0.f;
#pragma unroll
        for (int e = 0; e < 8; ++e) { ss_ = fmaf(f_[e], f_[e], ss_); f_[e] *= g_[e]; }
        sq[h] += J < nj ? ss_ : 0.f;
        piece = pack8<DT>(f_);
      }
      *(i4_u4*)(stages + J * kStage + (prow + 8 * h) * 128 + ((ppiece ^ prow) << 4)) = piece;
    }
  }

  // ---- the steps: round r takes tiles r RTR .. r RTR + RTR - 1; a dead step or tile multiplies by a zero scale
  i4_v4f acc[RT];
#pragma unroll
  for (int t = 0; t < RT; ++t) acc[t] = i4_v4f{0.f, 0.f, 0.f, 0.f};
  const int rd0 = ln * 128 + (((2 * c) ^ (ln & 7)) << 4), rd1 = ln * 128 + (((2 * c + 1) ^ (ln & 7)) << 4);
  i4_v4f xsum[NG];
#pragma unroll
  for (int r = 0; r < NR; ++r) {
#pragma unroll
    for (int J = 0; J < NG; ++J) {
      const bool step_live = J < nj;
      const i4_u4 xa0 = *(const i4_u4*)((R == 2 || ln < 8) ? stages + J * kStage + rd0 : zeros);
      const i4_u4 xa1 = *(const i4_u4*)((R == 2 || ln < 8) ? stages + J * kStage + rd1 : zeros);
      if (r == 0) {                                              // the group's activation sums, rows 4c + rr: kept for all rounds
        xsum[J] = i4_mfma32<DT>(xa0, ones, i4_v4f{0.f, 0.f, 0.f, 0.f});
        xsum[J] = i4_mfma32<DT>(xa1, ones, xsum[J]);
      }
      const i4_v4f xs = xsum[J];
#pragma unroll
      for (int tt = 0; tt < RTR; ++tt) {
        const int t = r * RTR + tt;
        const uint32_t w0 = wall[J][tt].x, w1 = wall[J][tt].y;
        if (r + 1 < NR)                                          // the same step of the next round inherits the registers
          wall[J][tt] = __builtin_amdgcn_raw_buffer_load_b64(w_rsrc, lane * 8, (wofs[min(t + RTR, RT - 1)] + min(g_first + NW * J, G - 1)) * 512, kStream);
        const uint32_t szw = (uint32_t)__shfl((int)szq[t][J >> 2], (J & 3) * 16 + ln, kWave);
        const i4_u4 b0 = i4_u4{code_pair(w0, 0, kmagic, kmask), code_pair(w0, 4, kmagic, kmask),
                               code_pair(w0, 8, kmagic, kmask), code_pair(w0, 12, kmagic, kmask)};
        const i4_u4 b1 = i4_u4{code_pair(w1, 0, kmagic, kmask), code_pair(w1, 4, kmagic, kmask),
                               code_pair(w1, 8, kmagic, kmask), code_pair(w1, 12, kmagic, kmask)};
        const float sc = (step_live && t < ntl) ? f16_bits_to_float(szw & 0xffffu) : 0.f;
        const float szo = -sc * (f16_bits_to_float(szw >> 16) + I4<DT>::kOffset);
        i4_v4f raw = i4_mfma32<DT>(xa0, b0, i4_v4f{0.f, 0.f, 0.f, 0.f});
        raw = i4_mfma32<DT>(xa1, b1, raw);
#pragma unroll
        for (int rr = 0; rr < 4; ++rr) acc[t][rr] = fmaf(sc, raw[rr], fmaf(szo, xs[rr], acc[t][rr]));
        // With several rounds the compiler otherwise sinks all these updates below the last MFMA (they are needed only at
        // the end) and keeps every raw product and scale word alive until then, in scratch memory: the empty statement
        // makes the accumulator observable here, so the update is evaluated in its step.
        if constexpr (NR > 1) asm volatile("" : "+v"(acc[t][0]), "+v"(acc[t][1]), "+v"(acc[t][2]), "+v"(acc[t][3]));
      }
    }
  }

  // ---- output stage
  if constexpr (NORM) {
    // the eight lanes that share a row hold its squares over different k; one value per (wavefront, row) goes to LDS
#pragma unroll
    for (int h = 0; h < R; ++h) {
      float v = sq[h];
      v += __shfl_xor(v, 1, kWave);
      v += __shfl_xor(v, 2, kWave);
      v += __shfl_xor(v, 4, kWave);
      if (ppiece == 0) sq_s[wave * 8 * R + prow + 8 * h] = v;
    }
  }
  __syncthreads();                                               // every wavefront is done with its stages
  if constexpr (NORM) {
    if (tid < 8 * R) {
      float ss = 0.f;
#pragma unroll
      for (int w = 0; w < NW; ++w) ss += sq_s[w * 8 * R + tid];
      rstd_s[tid] = rsqrtf(ss / (float)K + fz.norm_eps);
    }
  }
  if (lane < 32 * R) {                                           // accumulator rows 4c + rr: lane groups 0 and 1 hold rows 0..7
#pragma unroll
    for (int t = 0; t < RT; ++t) *(i4_v4f*)(&red[((t * NW + wave) * (32 * R) + lane) * 4]) = acc[t];
  }
  __syncthreads();
#pragma unroll
  for (int mi = 0; mi < R; ++mi) {
  const int m = wave + 8 * mi;                                   // this wavefront's row(s): wave, wave + 8
  if (m >= M) return;
  auto summed = [&](int t) {
    float v = 0.f;
#pragma unroll
    for (int w = 0; w < NW; ++w) v += red[((t * NW + w) * (32 * R) + (m >> 2) * 16 + ln) * 4 + (m & 3)];
    if constexpr (NORM) v *= rstd_s[m];
    return v;
  };
#pragma unroll
  for (int i0 = 0; i0 < kItems; i0 += 4) {                       // lane group c takes items c, c + 4, ...
    const int item = i0 + c;
    const int t0 = PAIRED ? 2 * item : item;
    if (item >= kItems || t0 >= ntl) continue;
    const int64_t n0 = (int64_t)tile_of(t0) * 16 + ln;
    const float v0 = summed(t0);
    if constexpr (!PAIRED) {
      if (splits == 1) {                                         // out = round(round(v) + residual), as store_linear_out
        asm volatile("" : "+v"(bias_pre[i0 / 4]), "+v"(res_pre[i0 / 4][mi]));
        float v = v0 + (bias ? I4<DT>::to_float((uint16_t)bias_pre[i0 / 4]) : 0.f);
        if (residual) v = Elem<DT>::round(v) + I4<DT>::to_float((uint16_t)res_pre[i0 / 4][mi]);
        Elem<DT>::store(y, (int64_t)m * N + n0, v);
      } else {
        partial[((int64_t)ks * M + m) * N + n0] = v0;
      }
    } else {
      asm volatile("" : "+v"(bias_pre[i0 / 4]), "+v"(bias1_pre[i0 / 4]), "+v"(pos_pre[mi]), "+v"(crow_pre[mi]));
      const float b0v = bias ? I4<DT>::to_float((uint16_t)bias_pre[i0 / 4]) : 0.f;
      const float b1v = bias ? I4<DT>::to_float((uint16_t)bias1_pre[i0 / 4]) : 0.f;
      const float first = Elem<DT>::round(v0 + b0v), second_raw = summed(t0 + 1) + b1v;
      const int u = unit0 + item;
      if constexpr (SILU) {
        // act[m, f] = round(silu(round(gate))) * round(up): the arithmetic of the separate activation kernel
        const float up = Elem<DT>::round(second_raw);
        Elem<DT>::store(y, (int64_t)m * (N / 2) + (int64_t)u * 16 + ln, Elem<DT>::round(first / (1.f + __expf(-first))) * up);
      } else if (u < qk_units) {
        // rotary pair (d, d + 64) of head u / 4, d = 16 (u % 4) + ln; t * cos + rotate_half(t) * sin with each
        // product and the sum rounded like the eager tensor ops
        const int head = u >> 2, d = (u & 3) * 16 + ln;
        const float inv_freq = fz.inv_freq ? fz.inv_freq[d] : exp2f(-(float)(2 * d) / 128.f * fz.log2_theta);
        float sn, cs;
        sincosf((float)pos_pre[mi] * inv_freq, &sn, &cs);
        cs = Elem<DT>::round(cs);
        sn = Elem<DT>::round(sn);
        const float lo = first, hi = Elem<DT>::round(second_raw);
        const float o_lo = Elem<DT>::round(lo * cs) + Elem<DT>::round(-hi * sn);
        const float o_hi = Elem<DT>::round(hi * cs) + Elem<DT>::round(lo * sn);
        uint16_t *dst, *unused;
        if (head < fz.hq) dst = fz.q_out + ((int64_t)head * M + m) * 128;
        else if (!kv_row_ptrs(fz.kv, head - fz.hq, crow_pre[mi], &dst, &unused)) continue;   // a row outside the layer's cache is dropped
        Elem<DT>::store(dst, d, o_lo);
        Elem<DT>::store(dst, d + 64, o_hi);
      } else {
        // two consecutive tiles of a value head: copied
        const int vt = 2 * (u - qk_units), kvh = vt >> 3, d = (vt & 7) * 16 + ln;
        uint16_t *dst, *unused;
        if (!kv_row_ptrs(fz.kv, kvh, crow_pre[mi], &unused, &dst)) continue;
        Elem<DT>::store(dst, d, first);
        Elem<DT>::store(dst, d + 16, second_raw);
      }
    }
  }
  }
}

// ------------------------------------------------------------------ 1 <= M <= 8, a long K over at least 128 tiles
// The down projection of a draft level (3584 x 18944: 296 groups) does not fit the K range of the kernel above, and
// splitting K over workgroups costs fp32 partials and a second launch that is all latency (11.6 + 3.9 us).  Here one
// workgroup owns one tile and ALL of K: wavefront w takes groups w, w + 8, ... in rounds of NG.  A round is the step
// sequence of the kernel above against registers; what it adds is that the registers refill while they are used: the
// activation blocks and (scale, zero) words of round r + 1 are requested when round r starts, and a step's weight
// register is requested again for round r + 1 as soon as the step has taken its words, so NG weight requests per
// wavefront stay in flight from the first round to the last.  3584 x 18944, 8 rows, weights from HBM: 14.5 us against
// 12.3 + 3.8 us for the split form -- a launch, one round trip and 38 MB at 4.5 TB/s; a second set of weight registers
// in flight two rounds ahead (15.8 us) and sixteen wavefronts of five groups per round (14.3 us) do not change that.  The eight partial tiles meet in LDS once, at the end, and
// the output stage (bias, residual) runs in the same launch.
template <int DT, int NW, int NG>
__global__ __launch_bounds__(NW * 64) void int4_rows8_long_kernel(
    const uint16_t* __restrict__ x, const uint2* __restrict__ wq, const uint32_t* __restrict__ sz,
    const uint16_t* __restrict__ bias, const uint16_t* residual, uint16_t* y, int M, int64_t N, int K) {
  asm volatile("" ::"s"(x), "s"(wq), "s"(sz), "s"(bias), "s"(residual), "s"(y), "s"(M), "s"(N), "s"(K));
  static_assert(NW >= 8, "wavefront m finishes row m");
  static_assert(NG <= 8, "two (scale, zero) requests per round cover eight steps");
  constexpr int kStageBytes = NW * NG * 1024 + NW * 16;          // stages, one block of zeros per wavefront
  constexpr int kRedBytes = NW * 32 * 16;                        // rows 0..7 of every wavefront's accumulators
  __shared__ __attribute__((aligned(16))) unsigned char lds_raw[kStageBytes > kRedBytes ? kStageBytes : kRedBytes];
  float* const red = (float*)lds_raw;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int ln = lane & 15, c = lane >> 4;
  const int G = K / kGroup;
  const int n_tiles = (int)(N / 16);
  const int tile = blockIdx.x;
  const int n_mine = wave < G ? (G - wave + NW - 1) / NW : 0;    // groups wave, wave + NW, ... of this wavefront
  const int rounds = (n_mine + NG - 1) / NG;

  const __amdgpu_buffer_rsrc_t x_rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)x, 0, M * K * 2, 0x00027000);
  const __amdgpu_buffer_rsrc_t w_rsrc =
      __builtin_amdgcn_make_buffer_rsrc((void*)wq, 0, (int)(n_tiles * (int64_t)G * 512), 0x00027000);
  const __amdgpu_buffer_rsrc_t sz_rsrc =
      __builtin_amdgcn_make_buffer_rsrc((void*)sz, 0, (int)(n_tiles * (int64_t)G * 64), 0x00027000);
  const int prow = lane >> 3, ppiece = lane & 7;                 // the lane's row and 16-byte piece of an activation block
  const int xg_off = (prow * K + ppiece * 8) * 2;                // rows past M read zeros (outside the descriptor)
  const int wofs = tile * G;
  const uint32_t kmask = 0x000f000fu | (uint32_t)(M >> 30), kmagic = I4<DT>::kMagic | ((uint32_t)xg_off >> 31);
  const uint32_t one2 = DT == SUBSPEC_BF16 ? 0x3f803f80u : 0x3c003c00u;
  const i4_u4 ones = i4_u4{one2, one2, one2, one2};
  unsigned char* const stages = lds_raw + wave * (NG * 1024);
  unsigned char* const zeros = lds_raw + NW * NG * 1024 + wave * 16;
  // group of step J in round r; requests past the wavefront's last group repeat group G - 1 and are multiplied by zero
  auto group_of = [&](int r, int J) { return min(wave + NW * (r * NG + J), G - 1); };

  // ---- round 0: every request, activations first
  i4_u4 xall[NG];
#pragma unroll
  for (int J = 0; J < NG; ++J) xall[J] = __builtin_amdgcn_raw_buffer_load_b128(x_rsrc, xg_off, group_of(0, J) * (kGroup * 2), 0);
  __builtin_amdgcn_sched_barrier(0);
  uint32_t szq[2];
#pragma unroll
  for (int h = 0; h < 2; ++h)
    szq[h] = __builtin_amdgcn_raw_buffer_load_b32(sz_rsrc, ln * 4 + (wofs + group_of(0, min(4 * h + c, NG - 1))) * 64, 0, kStream);
  i4_u2 wall[NG];
#pragma unroll
  for (int J = 0; J < NG; ++J) wall[J] = __builtin_amdgcn_raw_buffer_load_b64(w_rsrc, lane * 8, (wofs + group_of(0, J)) * 512, kStream);
  // what the output stage adds to this thread's element (wavefront m finishes row m, lane group 0 the sixteen columns):
  // requested here, so that the output stage does not end in a round trip of its own
  // (kept as the 16-bit words they are until then: an instruction that touches a loaded value here would wait for every
  // request issued before it; wavefronts without a row repeat the last one)
  const int64_t n_out = (int64_t)tile * 16 + ln;
  // (no branch around a request -- the compiler would wait for every request in flight where the paths join: a tensor
  // that is not there is replaced by the activations' first element)
  const uint32_t bias_pre = (bias ? bias : x)[bias ? n_out : 0];
  const uint32_t res_pre_ld = (residual ? residual : x)[residual ? (int64_t)min(wave, M - 1) * N + n_out : 0];
  uint32_t res_pre = res_pre_ld, bias_pre_v = bias_pre;
  __builtin_amdgcn_sched_barrier(0);
  if (lane == 0) *(i4_u4*)zeros = i4_u4{0u, 0u, 0u, 0u};

  i4_v4f acc = i4_v4f{0.f, 0.f, 0.f, 0.f};
  const int rd0 = ln * 128 + (((2 * c) ^ ln) << 4), rd1 = ln * 128 + (((2 * c + 1) ^ ln) << 4);
  for (int r = 0; r < rounds; ++r) {
    // park this round's activation blocks (the wavefront's own stages: its reads of the last round are behind it)
#pragma unroll
    for (int J = 0; J < NG; ++J) *(i4_u4*)(stages + J * 1024 + prow * 128 + ((ppiece ^ prow) << 4)) = xall[J];
    // the next round's activations and (scale, zero) words, ahead of the weight requests the steps below issue
#pragma unroll
    for (int J = 0; J < NG; ++J) xall[J] = __builtin_amdgcn_raw_buffer_load_b128(x_rsrc, xg_off, group_of(r + 1, J) * (kGroup * 2), 0);
    uint32_t sz_next[2];
#pragma unroll
    for (int h = 0; h < 2; ++h)
      sz_next[h] = __builtin_amdgcn_raw_buffer_load_b32(sz_rsrc, ln * 4 + (wofs + group_of(r + 1, min(4 * h + c, NG - 1))) * 64, 0, kStream);
    __builtin_amdgcn_sched_barrier(0);
    const int live = n_mine - r * NG;                            // steps of this round with a group of their own
#pragma unroll
    for (int J = 0; J < NG; ++J) {
      const i4_u4 xa0 = *(const i4_u4*)(ln < 8 ? stages + J * 1024 + rd0 : zeros);
      const i4_u4 xa1 = *(const i4_u4*)(ln < 8 ? stages + J * 1024 + rd1 : zeros);
      i4_v4f xs = i4_mfma32<DT>(xa0, ones, i4_v4f{0.f, 0.f, 0.f, 0.f});   // the group's activation sums, rows 4c + rr
      xs = i4_mfma32<DT>(xa1, ones, xs);
      const uint32_t w0 = wall[J].x, w1 = wall[J].y;
      const i4_u4 b0 = i4_u4{code_pair(w0, 0, kmagic, kmask), code_pair(w0, 4, kmagic, kmask),
                             code_pair(w0, 8, kmagic, kmask), code_pair(w0, 12, kmagic, kmask)};
      const i4_u4 b1 = i4_u4{code_pair(w1, 0, kmagic, kmask), code_pair(w1, 4, kmagic, kmask),
                             code_pair(w1, 8, kmagic, kmask), code_pair(w1, 12, kmagic, kmask)};
      // the words are spent: the request for the next round goes into the SAME registers (issued while the old words
      // were still wanted it would get others, and the copy back at the end of the round would wait for every request)
      __builtin_amdgcn_sched_barrier(0);
      wall[J] = __builtin_amdgcn_raw_buffer_load_b64(w_rsrc, lane * 8, (wofs + group_of(r + 1, J)) * 512, kStream);
      __builtin_amdgcn_sched_barrier(0);
      const uint32_t szw = (uint32_t)__shfl((int)szq[J >> 2], (J & 3) * 16 + ln, kWave);
      const float sc = J < live ? f16_bits_to_float(szw & 0xffffu) : 0.f;
      const float szo = -sc * (f16_bits_to_float(szw >> 16) + I4<DT>::kOffset);
      i4_v4f raw = i4_mfma32<DT>(xa0, b0, i4_v4f{0.f, 0.f, 0.f, 0.f});
      raw = i4_mfma32<DT>(xa1, b1, raw);
#pragma unroll
      for (int rr = 0; rr < 4; ++rr) acc[rr] = fmaf(sc, raw[rr], fmaf(szo, xs[rr], acc[rr]));
    }
    szq[0] = sz_next[0];
    szq[1] = sz_next[1];
  }

  // ---- output stage: rows 0..7 of every wavefront's accumulators meet in LDS; wavefront m finishes row m
  __syncthreads();                                               // every wavefront is done with its stages
  if (lane < 32) *(i4_v4f*)(&red[(wave * 32 + lane) * 4]) = acc;
  __syncthreads();
  const int m = wave;
  if (m >= M || c != 0) return;
  float v = 0.f;
#pragma unroll
  for (int w = 0; w < NW; ++w) v += red[(w * 32 + (m >> 2) * 16 + ln) * 4 + (m & 3)];
  asm volatile("" : "+v"(bias_pre_v), "+v"(res_pre));
  if (bias) v += I4<DT>::to_float((uint16_t)bias_pre_v);
  if (residual) v = Elem<DT>::round(v) + I4<DT>::to_float((uint16_t)res_pre);   // out = round(round(v) + residual), as store_linear_out
  Elem<DT>::store(y, (int64_t)m * N + n_out, v);
}

template <int DT>
__global__ __launch_bounds__(256) void int4_reduce_kernel(const float* __restrict__ partial,
                                                          const uint16_t* __restrict__ bias, const uint16_t* residual,
                                                          uint16_t* y, int64_t M, int64_t N, int splits) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= M * N) return;
  float v = 0.f;
  for (int s = 0; s < splits; ++s) v += partial[(int64_t)s * M * N + i];
  if (bias) v += I4<DT>::to_float(bias[i % N]);
  store_linear_out<DT>(y, i, v, residual);
}

struct I4Plan { int wgs, row_tiles, splits, groups_per_split; };
// The 8-row kernel takes K ranges (groups per workgroup) long enough that the pipelined loop would pay several round
// trips and short enough for its registers and LDS stages.  Its workgroups hold 63 KB of LDS, two per compute unit.
constexpr int kR8Range = kR8Waves * kR8Groups;
constexpr int kR8MaxRows = 16;                                  // 8 rows per block of the kernel's R parameter
static bool i4_rows8_plain(int64_t M, int G) { return M <= kR8MaxRows && G > 32; }
// Tile pairs per workgroup of a paired 8-row launch, 0 if it should not be one: one pair while that fits the 512
// resident workgroups; beyond that whole compute units' worth -- ceil(pairs / 256) pairs each, 3 to 5, in rounds of
// one pair, so that no compute unit gets a second workgroup while others have one.
static int i4_rows8_pairs(int64_t M, int G, int64_t pairs) {
  if (!(M <= kR8MaxRows && G > 32 && G <= kR8Range)) return 0;
  if (pairs <= 512) return 1;
  const int64_t p = (pairs + 255) / 256;
  return p <= 5 ? (int)std::max<int64_t>(p, 3) : 0;
}

constexpr int kI4MaxRowTiles = 5;
static int i4_row_tile_variant(int64_t need) { return need <= 1 ? 1 : need <= 2 ? 2 : need <= 3 ? 3 : kI4MaxRowTiles; }
// Resident workgroups the launch is balanced for (register use allows 2 per SIMD row for M > 32).
static int i4_slots(int64_t M) { return M > 32 ? 512 : 1024; }
// One workgroup per tile over the whole of K (int4_rows8_long_kernel) instead of K ranges over workgroups: a K that
// needs more than one range, and tiles enough to occupy half the chip.  Up to 8 rows only: every workgroup reads ALL of the
// activations (M x K x 2 bytes: 303 KB at 8 rows, 68 MB from the L2s over 224 workgroups beside 38 MB of weights), and at
// 16 rows that outweighs the saved launch (3584 x 18944: 18.7 us against 13.1 + 3.7 us for K ranges over workgroups).
static bool i4_rows8_long(int64_t M, int64_t N, int G) { return M <= 8 && G > kR8Range && N / 16 >= 128; }
static I4Plan i4_plan(int64_t M, int64_t N, int64_t K) {
  const int G = (int)(K / kGroup);
  const int64_t tiles = N / 16, slots = i4_slots(M);
  if (i4_rows8_long(M, N, G)) return I4Plan{(int)tiles, 1, 1, G};
  if (i4_rows8_plain(M, G)) {
    // The 8-row kernel: K ranges of at most 56 groups, and as many tiles per workgroup (1, 2, 3 in one round; 4, 6, 8, 10
    // in rounds of two) as brings the launch down to one workgroup per compute unit.  (Qwen2.5-7B shapes inside the resident
    // cycle, planned for 256, 400 or 512 resident workgroups: 43.6, 42.9, 42.7 tokens/s.)
    const int splits = (G + kR8Range - 1) / kR8Range;
    const int gps = ((G + splits - 1) / splits + 3) / 4 * 4;
    const int64_t need = (tiles * splits + 255) / 256;
    const int rt = need <= 3 ? (int)std::max<int64_t>(need, 1) : need <= 4 ? 4 : need <= 6 ? 6 : need <= 8 ? 8 : 10;
    return I4Plan{(int)((tiles + rt - 1) / rt), rt, (G + gps - 1) / gps, gps};
  }
  // row tiles per workgroup: the smallest compiled variant that covers all tiles in one resident wave of
  // workgroups; the grid then splits the tiles evenly, so every workgroup has row_tiles or row_tiles - 1
  int row_tiles = i4_row_tile_variant((tiles + slots - 1) / slots);
  // A long K over few tiles (the down projection) is split over workgroups, and every split re-reads its slice of the
  // activations: two tiles per workgroup halve that traffic (3584x18944, 16 rows, five splits; three or
  // five tiles per workgroup and fewer splits were slower)
  if (M <= 16 && row_tiles == 1 && tiles * 4 <= slots && G >= 112) row_tiles = 2;
  const int64_t wgs = (tiles + row_tiles - 1) / row_tiles;
  int splits = (int)std::max<int64_t>(1, (slots + wgs / 2) / wgs);
  // a split costs a second launch (the reduction) and fp32 partials: it pays from about 56 groups
  // (K = 3584) per split upwards -- measured 4608x3584, M = 8: 5.6 us unsplit against 8.2 us in three splits;
  // 3584x18944: 15.5 us in five splits against 22.9 us unsplit
  splits = std::min(splits, std::max(1, G / 56));
  splits = std::min(splits, 32);
  int gps = (G + splits - 1) / splits;
  gps = (gps + 3) / 4 * 4;
  splits = (G + gps - 1) / gps;
  return I4Plan{(int)wgs, row_tiles, splits, gps};
}

// Paired-tile launches: the gate|up projection with the SwiGLU output stage (x [M, K], weights of N = 2F rows, gate rows
// first, act [M, F]) and the q|k|v projection with the rotary / cache-write output stage; either with RMSNorm as prologue.
template <int DT, int EPI>
static int run_int4_paired(const void* x, const uint32_t* wq, const uint32_t* sz, const void* bias, void* out, int64_t M,
                           int64_t N, int64_t K, const I4Fused& fz, hipStream_t st) {
  const int64_t pairs = N / 32, slots = i4_slots(M);
  // one or two pairs per workgroup; two only with few activation rows (the accumulators of four tiles
  // times four row blocks would fill the register file)
  const int rt = (pairs <= slots || M > 32) ? 2 : 4;
  const int64_t wgs = (pairs + rt / 2 - 1) / (rt / 2);
  const dim3 grid((unsigned)wgs, 1);
  const int G = (int)(K / kGroup);
  const bool norm = fz.norm_gain != nullptr;
#define SUBSPEC_I4_PAIRED(MT, RT, NORM)                                                                            \
  if (MT == 1 && M <= 8)                                                                                           \
    hipLaunchKernelGGL((int4_gemm_kernel<DT, 1, RT, EPI, NORM, true>), grid, dim3(kI4Threads), 0, st, (const uint16_t*)x, \
                       (const uint2*)wq, sz, (const uint16_t*)bias, (const uint16_t*)nullptr, (uint16_t*)out, (float*)nullptr, \
                       (int)M, N, (int)K, 1, (G + 3) / 4 * 4, fz);                                                 \
  else                                                                                                             \
  hipLaunchKernelGGL((int4_gemm_kernel<DT, MT, RT, EPI, NORM>), grid, dim3(kI4Threads), 0, st, (const uint16_t*)x, \
                     (const uint2*)wq, sz, (const uint16_t*)bias, (const uint16_t*)nullptr, (uint16_t*)out, (float*)nullptr,   \
                     (int)M, N, (int)K, 1, (G + 3) / 4 * 4, fz)
#define SUBSPEC_I4_PAIRED_RT(MT, NORM) do { if (rt == 2) SUBSPEC_I4_PAIRED(MT, 2, NORM); else SUBSPEC_I4_PAIRED(MT, 4, NORM); } while (0)
  DominantKernelTimer timer(st);
  const int p8_plan = i4_rows8_pairs(M, G, pairs);
  if (const int p8 = (EPI == kEpiRope && p8_plan > 1) ? 0 : p8_plan) {
    const dim3 grid8((unsigned)((pairs + p8 - 1) / p8), 1);
#define SUBSPEC_I4_ROWS8_R(RTR, NR, NORM, R)                                                                       \
  hipLaunchKernelGGL((int4_rows8_kernel<DT, RTR, NR, EPI, NORM, R>), grid8, dim3(kR8Threads), 0, st, (const uint16_t*)x, \
                     (const uint2*)wq, sz, (const uint16_t*)bias, (const uint16_t*)nullptr, (uint16_t*)out, (float*)nullptr,   \
                     (int)M, N, (int)K, 1, kR8Range, fz)
#define SUBSPEC_I4_ROWS8(RTR, NR, NORM)                                                                            \
  do { if (M <= 8) SUBSPEC_I4_ROWS8_R(RTR, NR, NORM, 1); else SUBSPEC_I4_ROWS8_R(RTR, NR, NORM, 2); } while (0)
#define SUBSPEC_I4_ROWS8_P(NORM)                                                                                   \
  do {                                                                                                             \
    if (p8 == 1) SUBSPEC_I4_ROWS8(2, 1, NORM);                                                                     \
    else if constexpr (EPI == kEpiRope) return SUBSPEC_ERR_LIMIT;                                                  \
    else if (p8 == 3) SUBSPEC_I4_ROWS8(2, 3, NORM);                                                                \
    else if (p8 == 4) SUBSPEC_I4_ROWS8(2, 4, NORM);                                                                \
    else SUBSPEC_I4_ROWS8(2, 5, NORM);                                                                             \
  } while (0)
    if (norm) SUBSPEC_I4_ROWS8_P(true); else SUBSPEC_I4_ROWS8_P(false);
#undef SUBSPEC_I4_ROWS8_P
#undef SUBSPEC_I4_ROWS8
#undef SUBSPEC_I4_ROWS8_R
  } else
  if (M <= 16) { if (norm) SUBSPEC_I4_PAIRED_RT(1, true); else SUBSPEC_I4_PAIRED_RT(1, false); }
  else if (M <= 32) { if (norm) SUBSPEC_I4_PAIRED_RT(2, true); else SUBSPEC_I4_PAIRED_RT(2, false); }
  else {
    if (norm) SUBSPEC_FAIL(SUBSPEC_ERR_LIMIT, "int4 projection with the RMSNorm prologue: M=%lld exceeds 32 rows", (long long)M);
    SUBSPEC_I4_PAIRED_RT(4, false);
  }
#undef SUBSPEC_I4_PAIRED_RT
#undef SUBSPEC_I4_PAIRED
  SUBSPEC_CHECK_HIP(hipGetLastError());
  return SUBSPEC_OK;
}

template <int DT>
static int run_int4(const void* x, const uint32_t* wq, const uint32_t* sz, const void* bias, const void* residual, void* y,
                    int64_t M, int64_t N, int64_t K, void* workspace, hipStream_t st) {
  // One row: the GEMV kernel, unless the matrix has few rows and a long K (down projection): then its one workgroup
  // per 16-row tile leaves most of the chip idle and the split-K GEMM path is faster (3584x18944 from HBM: 22 against 32 us).
  if (M == 1 && !i4_rows8_plain(M, (int)(K / kGroup)) && i4_plan(M, N, K).splits == 1) {
    const size_t smem = (size_t)K * 2 + (size_t)(K / 16) * 4 + 64 * 4;
    DominantKernelTimer timer(st);
    hipLaunchKernelGGL((int4_gemv_kernel<DT>), dim3((unsigned)(N / 16)), dim3(kI4Threads), smem, st, (const uint16_t*)x,
                       (const uint2*)wq, sz, (const uint16_t*)bias, (const uint16_t*)residual, (uint16_t*)y, N, K);
  } else {
    const I4Plan pl = i4_plan(M, N, K);
    float* partial = (float*)workspace;
    const dim3 grid((unsigned)pl.wgs, (unsigned)pl.splits);
#define SUBSPEC_I4_LAUNCH(MT, RT)                                                                                  \
  if (MT == 1 && M <= 8)                                                                                           \
    hipLaunchKernelGGL((int4_gemm_kernel<DT, 1, RT, kEpiPlain, false, true>), grid, dim3(kI4Threads), 0, st, (const uint16_t*)x, \
                       (const uint2*)wq, sz, (const uint16_t*)bias, (const uint16_t*)residual, (uint16_t*)y, partial, (int)M, N, (int)K, \
                       pl.splits, pl.groups_per_split, I4Fused{});                                                 \
  else                                                                                                             \
  hipLaunchKernelGGL((int4_gemm_kernel<DT, MT, RT>), grid, dim3(kI4Threads), 0, st, (const uint16_t*)x,            \
                     (const uint2*)wq, sz, (const uint16_t*)bias, (const uint16_t*)residual, (uint16_t*)y, partial, (int)M, N, (int)K, \
                     pl.splits, pl.groups_per_split, I4Fused{})
#define SUBSPEC_I4_ROWS8_R(RTR, NR, R)                                                                             \
  hipLaunchKernelGGL((int4_rows8_kernel<DT, RTR, NR, kEpiPlain, false, R>), grid, dim3(kR8Threads), 0, st, (const uint16_t*)x, \
                     (const uint2*)wq, sz, (const uint16_t*)bias, (const uint16_t*)residual, (uint16_t*)y, partial, (int)M, N, (int)K, \
                     pl.splits, pl.groups_per_split, I4Fused{})
#define SUBSPEC_I4_ROWS8(RTR, NR)                                                                                  \
  do { if (M <= 8) SUBSPEC_I4_ROWS8_R(RTR, NR, 1); else SUBSPEC_I4_ROWS8_R(RTR, NR, 2); } while (0)
#define SUBSPEC_I4_LAUNCH_MT(MT)                                                                                   \
  do {                                                                                                             \
    if (pl.row_tiles == 1) SUBSPEC_I4_LAUNCH(MT, 1);                                                               \
    else if (pl.row_tiles == 2) SUBSPEC_I4_LAUNCH(MT, 2);                                                          \
    else if (pl.row_tiles == 3) SUBSPEC_I4_LAUNCH(MT, 3);                                                          \
    else SUBSPEC_I4_LAUNCH(MT, kI4MaxRowTiles);                                                                    \
  } while (0)
    {
      DominantKernelTimer timer(st);
      if (i4_rows8_long(M, N, (int)(K / kGroup))) {
        hipLaunchKernelGGL((int4_rows8_long_kernel<DT, kR8Waves, 8>), dim3((unsigned)(N / 16)), dim3(kR8Threads), 0, st, (const uint16_t*)x,
                           (const uint2*)wq, sz, (const uint16_t*)bias, (const uint16_t*)residual, (uint16_t*)y, (int)M, N, (int)K);
      } else
      if (i4_rows8_plain(M, (int)(K / kGroup))) {
        switch (pl.row_tiles) {
          case 1: SUBSPEC_I4_ROWS8(1, 1); break;
          case 2: SUBSPEC_I4_ROWS8(2, 1); break;
          case 3: SUBSPEC_I4_ROWS8(3, 1); break;
          case 4: SUBSPEC_I4_ROWS8(2, 2); break;
          case 6: SUBSPEC_I4_ROWS8(2, 3); break;
          case 8: SUBSPEC_I4_ROWS8(2, 4); break;
          default: SUBSPEC_I4_ROWS8(2, 5); break;
        }
      } else
      if (M <= 16) SUBSPEC_I4_LAUNCH_MT(1);
      else if (M <= 32) SUBSPEC_I4_LAUNCH_MT(2);
      else SUBSPEC_I4_LAUNCH_MT(4);
    }
#undef SUBSPEC_I4_ROWS8
#undef SUBSPEC_I4_ROWS8_R
#undef SUBSPEC_I4_LAUNCH_MT
#undef SUBSPEC_I4_LAUNCH
    if (pl.splits > 1)
      hipLaunchKernelGGL((int4_reduce_kernel<DT>), dim3((unsigned)((M * N + 255) / 256)), dim3(256), 0, st, partial,
                         (const uint16_t*)bias, (const uint16_t*)residual, (uint16_t*)y, M, N, pl.splits);
  }
  SUBSPEC_CHECK_HIP(hipGetLastError());
  return SUBSPEC_OK;
}

}  // namespace subspec

using namespace subspec;

extern "C" int subspec_int4_linear(const void* x, const uint32_t* wq, const uint32_t* sz, const void* bias, void* y,
                                   int dtype, int64_t M, int64_t N, int64_t K, int64_t group_size, void* workspace,
                                   size_t workspace_bytes, void* stream) {
  if (M <= 64) return int4_linear_ex(x, wq, sz, bias, nullptr, y, dtype, M, N, K, group_size, workspace, workspace_bytes, stream);
  // more than 64 rows (a whole large tree through the draft): 64 rows per pass over the weights, in stream order
  if (!x || !y) SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "int4_linear: null pointer argument");
  if (dtype != SUBSPEC_BF16 && dtype != SUBSPEC_F16)
    SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "int4_linear: dtype %d not supported (bf16 / fp16 activations only)", dtype);
  if (M > 65536) SUBSPEC_FAIL(SUBSPEC_ERR_LIMIT, "int4_linear: M=%lld too large", (long long)M);
  for (int64_t m0 = 0; m0 < M; m0 += 64) {
    const int64_t m = std::min<int64_t>(64, M - m0);
    const int rc = int4_linear_ex((const uint16_t*)x + m0 * K, wq, sz, bias, nullptr, (uint16_t*)y + m0 * N, dtype, m, N, K,
                                  group_size, workspace, workspace_bytes, stream);
    if (rc) return rc;
  }
  return SUBSPEC_OK;
}

static size_t i4_workspace_one(int64_t M, int64_t N, int64_t K) {
  const I4Plan pl = i4_plan(M, N, K);
  return (pl.splits > 1 ? align_up((size_t)pl.splits * M * N * sizeof(float), 256) : 0) + 256;
}

extern "C" int subspec_int4_gate_up_silu(const void* x, const uint32_t* wq, const uint32_t* sz, const void* bias, void* act,
                                         int dtype, int64_t M, int64_t N, int64_t K, void* stream) {
  return int4_gate_up_silu_ex(x, wq, sz, bias, act, dtype, M, N, K, nullptr, 0.f, stream);
}

extern "C" size_t subspec_int4_linear_workspace(int64_t M, int64_t N, int64_t K) {
  if (M <= 0 || N <= 0 || K <= 0) return 256;
  if (M <= 64) return i4_workspace_one(M, N, K);
  const size_t full = i4_workspace_one(64, N, K);
  return M % 64 ? std::max(full, i4_workspace_one(M % 64, N, K)) : full;
}

static int paired_args_ok(const char* what, const void* x, const uint32_t* wq, const uint32_t* sz, int dtype, int64_t M,
                          int64_t N, int64_t K) {
  if (dtype != SUBSPEC_BF16 && dtype != SUBSPEC_F16)
    SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "%s: dtype %d not supported (bf16 / fp16 activations only)", what, dtype);
  if (!x || !wq || !sz) SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "%s: null pointer argument", what);
  if (M <= 0 || M > 64 || N <= 0 || K <= 0 || N % 32 != 0 || K % kGroup != 0 || K > 65536)
    SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "%s: M=%lld N=%lld K=%lld; 1 <= M <= 64, N a multiple of 32, K of 64", what,
                 (long long)M, (long long)N, (long long)K);
  if (N * K / 2 >= ((int64_t)1 << 31))
    SUBSPEC_FAIL(SUBSPEC_ERR_LIMIT, "%s: N*K/2=%lld bytes of codes exceed the 2 GiB descriptor range", what, (long long)(N * K / 2));
  if (N >= (int64_t)1 << 20) SUBSPEC_FAIL(SUBSPEC_ERR_LIMIT, "%s: N=%lld exceeds the limit of 2^20 - 16 output features", what, (long long)N);
  if ((uintptr_t)x % 16 || (uintptr_t)wq % 16 || (uintptr_t)sz % 16)
    SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "%s: x / wq / sz must be 16-byte aligned", what);
  return SUBSPEC_OK;
}

int subspec::int4_gate_up_silu_ex(const void* x, const uint32_t* wq, const uint32_t* sz, const void* bias, void* act, int dtype,
                                  int64_t M, int64_t N, int64_t K, const void* norm_gain, float norm_eps, void* stream) {
  const int rc = paired_args_ok("int4_gate_up_silu", x, wq, sz, dtype, M, N, K);
  if (rc) return rc;
  if (!act || (uintptr_t)act % 8) SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "int4_gate_up_silu: act must be a non-null, 8-byte aligned pointer");
  if (norm_gain && (uintptr_t)norm_gain % 16) SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "int4_gate_up_silu: the norm gain must be 16-byte aligned");
  I4Fused fz{};
  fz.norm_gain = (const uint16_t*)norm_gain;
  fz.norm_eps = norm_eps;
  if (dtype == SUBSPEC_BF16) return run_int4_paired<SUBSPEC_BF16, kEpiSilu>(x, wq, sz, bias, act, M, N, K, fz, (hipStream_t)stream);
  return run_int4_paired<SUBSPEC_F16, kEpiSilu>(x, wq, sz, bias, act, M, N, K, fz, (hipStream_t)stream);
}

int subspec::int4_qkv_rope_ex(const void* x, const uint32_t* wq, const uint32_t* sz, const void* bias, int dtype, int64_t M,
                              int64_t K, const void* norm_gain, float norm_eps, const int32_t* positions,
                              const int32_t* cache_rows, void* q_out, const KvRowMap& kv, int64_t n_q_heads,
                              float rope_theta, const float* inv_freq, void* stream) {
  const int64_t n_kv_heads = kv.hkv;
  const int64_t N = (n_q_heads + 2 * n_kv_heads) * 128;
  const int rc = paired_args_ok("int4_qkv_rope", x, wq, sz, dtype, M, N, K);
  if (rc) return rc;
  if (!positions || !cache_rows || !q_out || !kv.k_cache || (!kv.page_table && !kv.v_cache))
    SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "int4_qkv_rope: null pointer argument");
  if (norm_gain && (uintptr_t)norm_gain % 16) SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "int4_qkv_rope: the norm gain must be 16-byte aligned");
  I4Fused fz{};
  fz.norm_gain = (const uint16_t*)norm_gain;
  fz.norm_eps = norm_eps;
  fz.positions = positions;
  fz.cache_rows = cache_rows;
  fz.q_out = (uint16_t*)q_out;
  fz.kv = kv;
  fz.inv_freq = inv_freq;
  fz.hq = (int)n_q_heads;
  fz.hkv = (int)n_kv_heads;
  fz.log2_theta = log2f(rope_theta);
  if (dtype == SUBSPEC_BF16) return run_int4_paired<SUBSPEC_BF16, kEpiRope>(x, wq, sz, bias, nullptr, M, N, K, fz, (hipStream_t)stream);
  return run_int4_paired<SUBSPEC_F16, kEpiRope>(x, wq, sz, bias, nullptr, M, N, K, fz, (hipStream_t)stream);
}

int subspec::int4_linear_ex(const void* x, const uint32_t* wq, const uint32_t* sz, const void* bias, const void* residual,
                            void* y, int dtype, int64_t M, int64_t N, int64_t K, int64_t group_size, void* workspace,
                            size_t workspace_bytes, void* stream) {
  if (dtype != SUBSPEC_BF16 && dtype != SUBSPEC_F16)
    SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "int4_linear: dtype %d not supported (bf16 / fp16 activations only)", dtype);
  if (!x || !wq || !sz || !y) SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "int4_linear: null pointer argument");
  if (group_size != kGroup) SUBSPEC_FAIL(SUBSPEC_ERR_LIMIT, "int4_linear: group_size=%lld (built for 64)", (long long)group_size);
  if (M <= 0 || N <= 0 || K <= 0 || N % 16 != 0 || K % kGroup != 0)
    SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "int4_linear: M=%lld N=%lld K=%lld; N must be a multiple of 16 and K of 64",
                 (long long)M, (long long)N, (long long)K);
  if (M > 64) SUBSPEC_FAIL(SUBSPEC_ERR_LIMIT, "int4_linear: M=%lld exceeds the 64 rows of one pass", (long long)M);
  if (K > 65536) SUBSPEC_FAIL(SUBSPEC_ERR_LIMIT, "int4_linear: K=%lld too large", (long long)K);
  if (N * K / 2 >= ((int64_t)1 << 31))
    SUBSPEC_FAIL(SUBSPEC_ERR_LIMIT, "int4_linear: N*K/2=%lld bytes of codes exceed the 2 GiB descriptor range", (long long)(N * K / 2));
  if (N >= (int64_t)1 << 20) SUBSPEC_FAIL(SUBSPEC_ERR_LIMIT, "int4_linear: N=%lld exceeds the limit of 2^20 - 16 output features", (long long)N);
  if ((uintptr_t)x % 16 || (uintptr_t)wq % 16 || (uintptr_t)sz % 16 || (uintptr_t)y % 8)
    SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "int4_linear: x / wq / sz must be 16-byte aligned, y 8-byte aligned");
  {
    const size_t need = subspec_int4_linear_workspace(M, N, K);
    if (!workspace || workspace_bytes < need)
      SUBSPEC_FAIL(SUBSPEC_ERR_WORKSPACE, "int4_linear: workspace of %zu bytes is smaller than the %zu required",
                   workspace_bytes, need);
    if ((uintptr_t)workspace % 16) SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "int4_linear: workspace must be 16-byte aligned");
  }
  if (dtype == SUBSPEC_BF16) return run_int4<SUBSPEC_BF16>(x, wq, sz, bias, residual, y, M, N, K, workspace, (hipStream_t)stream);
  return run_int4<SUBSPEC_F16>(x, wq, sz, bias, residual, y, M, N, K, workspace, (hipStream_t)stream);
}
