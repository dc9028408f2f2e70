// Dense 16-bit linear layers for few activation rows on gfx950:
//   y[M, N] = x[M, K] * W[N, K]^T (+ bias),   1 <= M <= 384,   W row-major bf16 / fp16
//
// Replaces the nn.Linear modules of the target model's decoder layers in the tree-decoding forward
// (ClassicSDGeneratorBase._tree_decoding -> self.target_model(...),
// specdecodes/models/generators/classic_sd.py:75-109): the tree nodes of a speculation (64 with the default
// max_verify_tokens, 1 + 48 * 6 = 289 in configs/exp_offloading/subspec_sd_qwen_7b.yaml:16-19) go through the layer at
// once.  Up to 64 rows every projection streams its whole weight matrix for a handful of rows and is bound by HBM
// (algorithmic bytes = N*K*2 + (M*K + M*N)*2); a library GEMM tiled for large M leaves more than half of that bandwidth
// unused at this shape.  Three kernels: 1 to 32 rows the 16 x 16 x 32 kernel below, 33 to 384 rows the 32 x 32 x 16
// kernel behind it.
//
// Same skeleton as the int4 kernel next door: the activations are the MFMA A operand, a 16-row
// weight tile the B operand (v_mfma_f32_16x16x32, k permutation "step s, lane group c, element e ->
// k = 16c + 8s + e" on both operands), a workgroup owns up to RT consecutive tiles, its four
// wavefronts split K in groups of 64 and run as independent software pipelines (weights two groups
// ahead in registers, activation block through a wavefront-private LDS stage), partial sums are
// added in wavefront order at the end and split-K partials in split order by a second launch.
// The weights are requested as whole 128-byte lines (rows 0..7 of a tile's 64-k block in one request, rows 8..15 in
// the next), as streaming data, and pass through a wavefront-private LDS stage into the operand layout.
#include "common.h"
#include <algorithm>
#include <type_traits>

namespace subspec {

constexpr int kDnThreads = 256;
constexpr int kDnGroup = 64;
constexpr int kDnXlStride = kDnGroup + 8;                      // LDS row stride (elements) of a parked activation block

typedef float dn_v4f __attribute__((ext_vector_type(4)));
typedef uint32_t dn_u4 __attribute__((ext_vector_type(4)));
typedef __bf16 dn_v8bf __attribute__((ext_vector_type(8)));
typedef _Float16 dn_v8h __attribute__((ext_vector_type(8)));

template <int DT>
__device__ __forceinline__ dn_v4f dn_mfma32(dn_u4 a, dn_u4 b, dn_v4f c) {
  if constexpr (DT == SUBSPEC_BF16)
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(dn_v8bf, a), __builtin_bit_cast(dn_v8bf, b), c, 0, 0, 0);
  else
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(dn_v8h, a), __builtin_bit_cast(dn_v8h, b), c, 0, 0, 0);
}

// SILU (the gate|up projection of a SwiGLU MLP, N = 2F rows: gate rows first, up rows behind them): a workgroup
// owns PAIRS of tiles, (gate tile p, up tile p + F/16), and its output stage writes act[m, f] =
// round(silu(round(gate))) * round(up) to y[M, F] instead of the 2F projections.
template <int DT, int MT, int RT, bool SILU = false>
__global__ __launch_bounds__(kDnThreads) void dense_gemm_kernel(
    const uint16_t* __restrict__ x, const uint16_t* __restrict__ w, const uint16_t* __restrict__ bias,
    const uint16_t* residual, uint16_t* y, float* __restrict__ partial, int M, int64_t N, int K, int splits,
    int groups_per_split) {
  // 4 wavefronts x 2 stages of a [16*MT][64] activation block; reused for the final reduction
  constexpr int kStageBytes = 4 * 2 * MT * 16 * kDnXlStride * 2, kRedBytes = 2 * 4 * MT * 256 * 4;
  __shared__ __attribute__((aligned(16))) unsigned char lds_raw[kStageBytes > kRedBytes ? kStageBytes : kRedBytes];
  uint16_t* const xstage = (uint16_t*)lds_raw;
  float* const red = (float*)lds_raw;
  // a wavefront's weight block (16 rows x 128 bytes) on its way from the whole-line layout of the requests to the
  // MFMA operand layout; 16-byte piece p of row r sits at p ^ (r / 2) % 8, which makes writes and reads conflict-free
  __shared__ __attribute__((aligned(16))) uint16_t wstage_raw[4 * 1024];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int ln = lane & 15, c = lane >> 4;
  uint16_t* const wst = wstage_raw + wave * 1024;
  const int G = K / kDnGroup;
  const int n_tiles = (int)(N / 16);
  const int ks = blockIdx.y;
  const int g_begin = ks * groups_per_split, g_end = min(G, g_begin + groups_per_split);
  const int g_first = g_begin + wave;                            // this wavefront's groups: g_first + 4j
  const int nj = g_first < g_end ? (g_end - g_first + 3) / 4 : 0;

  // tiles [tile0, tile0 + ntl) of this workgroup: an even split of all tiles (SILU: of all tile pairs) over the grid
  const int n_units = SILU ? n_tiles / 2 : n_tiles;
  const int tile0 = (int)((int64_t)blockIdx.x * n_units / gridDim.x);                  // SILU: first pair = first gate tile
  const int n_own = (int)((int64_t)(blockIdx.x + 1) * n_units / gridDim.x) - tile0;
  const int ntl = SILU ? 2 * n_own : n_own;                                            // 1 .. RT
  // tile t of this workgroup, counted from its first tile
  auto tile_rel = [&](int t) { return SILU ? (t >> 1) + (t & 1) * (n_tiles / 2) : t; };

  dn_v4f acc[RT][MT];
#pragma unroll
  for (int t = 0; t < RT; ++t)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[t][mt] = dn_v4f{0.f, 0.f, 0.f, 0.f};

  // Buffer-descriptor loads keep their place in the program (plain loads that feed a loop-carried
  // value are merged into one load at the loop head, which would undo the prefetch distance) and
  // return zeros outside the tensor.  The weight descriptor starts at this workgroup's first tile,
  // so its offsets stay far below the 2 GiB range whatever the size of the matrix.
  const __amdgpu_buffer_rsrc_t x_rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)x, 0, M * K * 2, 0x00027000);
  const int64_t w_bytes = (int64_t)(tile_rel(ntl - 1) + 1) * 16 * K * 2;            // up to the last tile it touches
  const __amdgpu_buffer_rsrc_t w_rsrc =
      __builtin_amdgcn_make_buffer_rsrc((void*)(w + (int64_t)tile0 * 16 * K), 0, (int)w_bytes, 0x00027000);
  constexpr int kXg = MT * 2;                                    // 16-byte pieces per lane of one group block
  const int xg_off = ((lane >> 3) * K + (lane & 7) * 8) * 2;     // byte offset of piece 0; piece i is 8 rows further
  uint16_t* const xl = xstage + wave * (2 * MT * 16 * kDnXlStride);  // this wavefront's two stages
  const int xl_write = (lane >> 3) * kDnXlStride + (lane & 7) * 8;
  const int xl_read = ln * kDnXlStride + c * 16;
  // Weight requests cover whole 128-byte lines: one request fetches rows 0..7 of a tile's 64-k block (lane -> row
  // lane / 8, 16-byte piece lane % 8), a second one rows 8..15, both as streaming data (every weight byte is read once
  // per launch).  The MFMA B operand wants lane (ln, c) to hold pieces 2c and 2c + 1 of row ln, so a block passes
  // through a wavefront-private LDS stage on its way to the matrix core.  Requests of 32 bytes per lane straight in
  // operand layout (two half-line requests per line) cannot stream -- the line does not wait in the first-level cache
  // for its second half -- and were 13 to 24 % slower (152064 x 3584 at 8 rows: 195 -> 169 us; 37888 x 3584 at 64
  // rows with the SwiGLU output stage: 71.4 -> 63.0 us).
  const int w_lane = ((lane >> 3) * K + (lane & 7) * 8) * 2;     // byte offset of this lane's piece of rows 0..7 inside a tile
  const int w_lane2 = w_lane + 8 * K * 2;                        // ... of rows 8..15
  const int wst_w0 = (lane >> 3) * 64 + (((lane & 7) ^ ((lane >> 4) & 7)) << 3);               // stage positions (elements)
  const int wst_w1 = ((lane >> 3) + 8) * 64 + (((lane & 7) ^ ((((lane >> 3) + 8) >> 1) & 7)) << 3);
  const int wst_r0 = ln * 64 + (((2 * c) ^ ((ln >> 1) & 7)) << 3), wst_r1 = ln * 64 + (((2 * c + 1) ^ ((ln >> 1) & 7)) << 3);
  constexpr int kWAux = 2;                                       // cache policy of the weight requests: bit 1 = non-temporal
  int wofs[RT];                                                  // byte offset of (tile t, k = 0) from the first tile
#pragma unroll
  for (int t = 0; t < RT; ++t) wofs[t] = tile_rel(min(t, ntl - 1)) * 16 * K * 2;

  // Activation blocks on their way from global memory to LDS: requested kXSlots steps before they are parked (a
  // block that is parked one step after its request makes every step wait for a whole round trip to L2).
  constexpr int kXSlots = MT == 4 ? 1 : 2;   // 64 rows: one (with two the compiler waits for every request at the top of the loop body)
  dn_u4 xg[kXSlots][kXg];
  // Weights on their way, two groups ahead.  With one tile per workgroup they rotate through three register slots, so
  // that a request never targets the slot the current step multiplies from (the compiler would issue it first, into
  // other registers, and copy at the end of the loop body behind a wait for every request in flight).
  constexpr int kWSlots = RT == 1 ? 3 : 2;
  dn_u4 wbuf[kWSlots][RT][2];

#define SUBSPEC_DN_FETCH_X(XS, J)                                                                       \
  {                                                                                                     \
    const int kc = min(g_first + 4 * (J), G - 1) * (kDnGroup * 2);                                      \
    _Pragma("unroll") for (int i = 0; i < kXg; ++i)                                                     \
      xg[XS][i] = __builtin_amdgcn_raw_buffer_load_b128(x_rsrc, xg_off + i * 16 * K, kc, 0);            \
  }
#define SUBSPEC_DN_PARK_X(SLOT)                                                                         \
  _Pragma("unroll") for (int i = 0; i < kXg; ++i)                                                       \
    *(dn_u4*)(&xl[(SLOT) * (MT * 16 * kDnXlStride) + i * 8 * kDnXlStride + xl_write]) = xg[(SLOT) % kXSlots][i];
#define SUBSPEC_DN_FETCH_W(SLOT, J, T)                                                                  \
  {                                                                                                     \
    const int kc = wofs[T] + min(g_first + 4 * (J), G - 1) * (kDnGroup * 2);                            \
    wbuf[SLOT][T][0] = __builtin_amdgcn_raw_buffer_load_b128(w_rsrc, w_lane, kc, kWAux);                \
    wbuf[SLOT][T][1] = __builtin_amdgcn_raw_buffer_load_b128(w_rsrc, w_lane2, kc, kWAux);               \
  }
  // Step J works on LDS stage SLOT = J & 1.  Once its operands are in registers the stage is free:
  // the block of group J + 2 (requested kXSlots steps ago) is parked there and group J + 2 + kXSlots requested.
  // A step past the wavefront's last group multiplies activations that were replaced by zeros.
#define SUBSPEC_DN_STEP(SLOT, WS, WNEXT, J)                                                             \
  {                                                                                                     \
    const bool step_live = (J) < nj;                                                                    \
    dn_u4 xa[MT][2];                                                                                    \
    _Pragma("unroll") for (int mt = 0; mt < MT; ++mt) {                                                 \
      const uint16_t* xr = &xl[(SLOT) * (MT * 16 * kDnXlStride) + mt * 16 * kDnXlStride + xl_read];     \
      const dn_u4 a0 = *(const dn_u4*)xr, a1 = *(const dn_u4*)(xr + 8);                                 \
      xa[mt][0] = step_live ? a0 : dn_u4{0u, 0u, 0u, 0u};                                               \
      xa[mt][1] = step_live ? a1 : dn_u4{0u, 0u, 0u, 0u};                                               \
    }                                                                                                   \
    SUBSPEC_DN_PARK_X(SLOT);                                                                            \
    SUBSPEC_DN_FETCH_X((SLOT) % kXSlots, (J) + 2 + kXSlots);                                            \
    __builtin_amdgcn_sched_barrier(0);              /* keep the requests here: a full step ahead of their use */ \
    /* The request for group J + 2 follows the last product of the tile whose registers it reuses: requested     */ \
    /* earlier, the new weights get registers of their own and a copy at the end of the loop body, which waits   */ \
    /* for EVERY request in flight.  (One tile per workgroup: a third slot instead, see wbuf.)                   */ \
    _Pragma("unroll") for (int t = 0; t < RT; ++t) {                                                    \
      *(dn_u4*)(wst + wst_w0) = wbuf[WS][t][0];       /* whole-line layout -> operand layout */            \
      *(dn_u4*)(wst + wst_w1) = wbuf[WS][t][1];                                                         \
      const dn_u4 wb0 = *(const dn_u4*)(wst + wst_r0), wb1 = *(const dn_u4*)(wst + wst_r1);             \
      _Pragma("unroll") for (int mt = 0; mt < MT; ++mt) {                                               \
        acc[t][mt] = dn_mfma32<DT>(xa[mt][0], wb0, acc[t][mt]);                                         \
        acc[t][mt] = dn_mfma32<DT>(xa[mt][1], wb1, acc[t][mt]);                                         \
      }                                                                                                 \
      __builtin_amdgcn_sched_barrier(0);                                                                \
      SUBSPEC_DN_FETCH_W(WNEXT, (J) + 2, t);                                                            \
    }                                                                                                   \
    __builtin_amdgcn_sched_barrier(0);                                                                  \
  }

  SUBSPEC_DN_FETCH_X(0, 0);
#pragma unroll
  for (int t = 0; t < RT; ++t) SUBSPEC_DN_FETCH_W(0, 0, t);
  SUBSPEC_DN_PARK_X(0);
  SUBSPEC_DN_FETCH_X(1 % kXSlots, 1);
#pragma unroll
  for (int t = 0; t < RT; ++t) SUBSPEC_DN_FETCH_W(1, 1, t);
  SUBSPEC_DN_PARK_X(1);
  SUBSPEC_DN_FETCH_X(0, 2);
  if constexpr (kXSlots == 2) SUBSPEC_DN_FETCH_X(1, 3);
  if constexpr (RT == 1) {
    // step J: LDS stage J % 2, weight slot J % 3, request for group J + 2 into slot (J + 2) % 3
    for (int j = 0; j < nj; j += 6) {
      SUBSPEC_DN_STEP(0, 0, 2, j);
      SUBSPEC_DN_STEP(1, 1, 0, j + 1);
      SUBSPEC_DN_STEP(0, 2, 1, j + 2);
      SUBSPEC_DN_STEP(1, 0, 2, j + 3);
      SUBSPEC_DN_STEP(0, 1, 0, j + 4);
      SUBSPEC_DN_STEP(1, 2, 1, j + 5);
    }
  } else {
    for (int j = 0; j < nj; j += 2) {
      SUBSPEC_DN_STEP(0, 0, 0, j);
      SUBSPEC_DN_STEP(1, 1, 1, j + 1);
    }
  }
  __syncthreads();                                               // the stages are reused for the reduction below
#undef SUBSPEC_DN_PARK_X
#undef SUBSPEC_DN_FETCH_X
#undef SUBSPEC_DN_FETCH_W
#undef SUBSPEC_DN_STEP

  // ---- sum the four wavefronts' partial accumulators in wavefront order (0, 1, 2, 3), one tile per
  // round.  LDS holds two rounds, so a round needs one barrier; wavefront w finishes the activation
  // row blocks mt = w, w + 4, ... of the tile.  Accumulator layout: rows m = 16*mt + 4*c + rr,
  // column n = 16*tile + ln.
  float gate_held[MT][4];                                        // SILU: the rounded gate values between two rounds
  (void)gate_held;
#pragma unroll
  for (int t = 0; t < RT; ++t) {
    if (t >= ntl) break;                                         // uniform
    float* stage = red + (t & 1) * (4 * MT * 256);
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) *(dn_v4f*)(&stage[((wave * MT + mt) * 64 + lane) * 4]) = acc[t][mt];
    __syncthreads();                                             // round t written; round t - 1 fully read
    const int64_t n = (int64_t)(tile0 + tile_rel(t)) * 16 + ln;
    const float bv = (splits == 1 && bias) ? Elem<DT>::load(bias, n) : 0.f;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      if ((mt & 3) != wave) continue;                            // uniform
      dn_v4f v = *(const dn_v4f*)(&stage[((0 * MT + mt) * 64 + lane) * 4]);
#pragma unroll
      for (int wv = 1; wv < 4; ++wv) {
        const dn_v4f o = *(const dn_v4f*)(&stage[((wv * MT + mt) * 64 + lane) * 4]);
#pragma unroll
        for (int rr = 0; rr < 4; ++rr) v[rr] += o[rr];
      }
      if constexpr (SILU) {
        // even round: the gate tile, kept in registers; odd round: its up tile, same wavefront, same lanes
        if ((t & 1) == 0) {
#pragma unroll
          for (int rr = 0; rr < 4; ++rr) gate_held[mt][rr] = Elem<DT>::round(v[rr] + bv);
        } else {
          const int64_t f = (int64_t)(tile0 + (t >> 1)) * 16 + ln;
#pragma unroll
          for (int rr = 0; rr < 4; ++rr) {
            const int m = mt * 16 + c * 4 + rr;
            if (m >= M) continue;
            const float g = gate_held[mt][rr], u = Elem<DT>::round(v[rr] + bv);
            Elem<DT>::store(y, (int64_t)m * (N / 2) + f, Elem<DT>::round(g / (1.f + __expf(-g))) * u);
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

template <int DT>
__global__ __launch_bounds__(256) void dense_reduce_kernel(const float* __restrict__ partial, const uint16_t* __restrict__ bias,
                                                           const uint16_t* residual, uint16_t* y, int64_t M, int64_t N,
                                                           int splits) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= M * N) return;
  float v = 0.f;
  for (int s = 0; s < splits; ++s) v += partial[(int64_t)s * M * N + i];
  if (bias) v += Elem<DT>::load(bias, i % N);
  store_linear_out<DT>(y, i, v, residual);
}

// ------------------------------------------------------------------ 33 <= M <= 384
// The same product for more activation rows, where the weight bytes no longer dominate: v_mfma_f32_32x32x16 with a
// 32-row WEIGHT tile as A operand and 32 activation rows as B operand -- both operands are k-contiguous 16-byte
// pieces of row-major rows, so nothing is transposed.  A workgroup of eight wavefronts owns up to NTMAX weight tiles
// and ALL activation rows (every weight byte is fetched from HBM once, whatever M), and walks K in chunks of 64:
// the chunk of its weight tiles (32 rows x 128 bytes each) and the chunk of the activations (M rows x 128 bytes, from
// the L2) are copied straight into LDS ring slots (global_load_lds_dwordx4, 1 KB = 8 rows x 128 bytes = whole cache
// lines per request), a few wavefronts doing the weight copies and the others the activation copies, so that each
// wavefront's request counter (in-order) tracks one ring and a deep weight ring does not wait behind the shallow
// activation ring.  16-byte piece p of row r sits at position p ^ (r / 2) % 8 of the row: operand reads (lane -> row
// lane % 32, pieces 2 s + lane / 32 of 16-k step s) are conflict-free without padding.  Accumulator layout of the
// instruction: lane -> activation row 32 t + lane % 32, register r -> weight row 8 (r / 4) + 4 (lane / 32) + r % 4.
// SwiGLU pairs: a "tile" is 16 gate rows + 16 up rows of the same 16 output columns, so gate and up of an element are
// registers r and r + 8 of one lane.
// Measured on the four projections of a 7B layer, weights from HBM: M = 64 16.8 / 14.6 / 50.8 / 34.6 us (q|k|v, o,
// gate|up with SwiGLU, down with its reduction; the 16 x 16 x 32 kernel above: 16.2 / 14.8 / 64.2 / 37.6); M = 289
// 33 / 29 / 97 / 70 us.  At 289 rows the kernel is bound by the activation copies: a chunk is 40 KB per workgroup, LDS
// holds two of them beside three weight chunks, and one chunk in flight does not cover the L2 latency (M = 256 with
// three activation slots: 79 us against 94 us with two).
typedef float wd_v16f __attribute__((ext_vector_type(16)));
typedef uint32_t wd_u4 __attribute__((ext_vector_type(4)));
typedef uint32_t wd_u2 __attribute__((ext_vector_type(2)));
typedef __bf16 wd_v8bf __attribute__((ext_vector_type(8)));
typedef _Float16 wd_v8h __attribute__((ext_vector_type(8)));

template <int DT>
__device__ __forceinline__ wd_v16f wd_mfma(wd_u4 a, wd_u4 b, wd_v16f c) {
  if constexpr (DT == SUBSPEC_BF16)
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(wd_v8bf, a), __builtin_bit_cast(wd_v8bf, b), c, 0, 0, 0);
  else
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(wd_v8h, a), __builtin_bit_cast(wd_v8h, b), c, 0, 0, 0);
}
template <int DT> __device__ __forceinline__ uint32_t wd_pack2(float a, float b) {
  if constexpr (DT == SUBSPEC_BF16) {
    typedef __bf16 v2 __attribute__((ext_vector_type(2)));
    v2 r; r[0] = (__bf16)a; r[1] = (__bf16)b;
    return __builtin_bit_cast(uint32_t, r);
  } else {
    typedef _Float16 v2 __attribute__((ext_vector_type(2)));
    v2 r; r[0] = (_Float16)a; r[1] = (_Float16)b;
    return __builtin_bit_cast(uint32_t, r);
  }
}

__device__ __forceinline__ void wd_dma16(uint32_t lds_base, const uint16_t* src) {
  asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(lds_base), "v"(src) : "memory", "m0");
}
template <int N> __device__ __forceinline__ void wd_wait_vmcnt() { asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory"); }

struct WideParams {
  const uint16_t* x; const uint16_t* w; const uint16_t* bias; const uint16_t* residual; uint16_t* y; float* partial;
  int M, K; int64_t N;     // N: rows of w (SILU: 2 F)
  int n_tiles;             // 32-row weight tiles (SILU: tiles of 16 gate + 16 up rows)
  int splits, stages_per_split;   // K ranges and their length in chunks of 64
};

// WM x WN = 8 wavefronts: wavefront (wm, wn) multiplies row tiles wm, wm + WM, ... (at most MG) by weight tiles
// wn, wn + WN, ... (at most NH) of the workgroup.  K advances in chunks of 64: a chunk of the weights (NTMAX x 32 rows x
// 128 bytes) and of the activations (MT x 32 rows x 128 bytes) sits in a ring slot each; a request moves 1 KB = 8 rows x
// 128 bytes, whole cache lines.  Copies: wavefronts [0, NWW) bring the weight chunks (WPER requests each per chunk),
// wavefronts [NWW, NWW + NXW) the activation chunks (ceil(4 MT / NXW) each, at most XPER).
template <int DT, int WM, int MG, int NTMAX, int SW, int SX, int NWW, int WPER, int NXW, int XPER, bool SILU>
__global__ __launch_bounds__(512) void dense_wide_kernel(WideParams p) {
  constexpr int MTMAX = WM * MG;
  __shared__ __attribute__((aligned(16))) uint8_t wd_lds[(SW * NTMAX + SX * MTMAX) * 4096];
  constexpr int WN = 8 / WM, NH = (NTMAX + WN - 1) / WN;
  static_assert(NWW + NXW <= 8 && NWW * WPER >= 4 * NTMAX, "copy plan");
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lr = lane & 31, g = lane >> 5;
  const int M = p.M, K = p.K;
  const int MT = (M + 31) >> 5;
  const int tile0 = (int)((int64_t)blockIdx.x * p.n_tiles / gridDim.x);
  const int ntl = (int)((int64_t)(blockIdx.x + 1) * p.n_tiles / gridDim.x) - tile0;      // 1 .. NTMAX
  const int n_chunks = K >> 6;
  const int st0 = blockIdx.y * p.stages_per_split, st1 = min(n_chunks, st0 + p.stages_per_split);
  const int nst = st1 - st0;

  const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)wd_lds;
  constexpr uint32_t kWStride = NTMAX * 4096;
  constexpr uint32_t xstride = MTMAX * 4096, xring = SW * kWStride;

  // ---- copy plan of this wavefront: lane -> row lane / 8 of the request's eight, position lane % 8, which holds the
  // 16-byte piece (position ^ (row / 2) % 8) of the row's 64 k (conflict-free operand reads)
  const bool w_wave = wave < NWW, x_wave = wave >= NWW && wave < NWW + NXW;
  constexpr int kPer = WPER > XPER ? WPER : XPER;
  // with two activation slots every activation request has landed at each wait, whatever their number; with more the
  // count is fixed at XPER (surplus requests repeat earlier ones)
  const int xper = SX == 2 ? (4 * MT + NXW - 1) / NXW : XPER;
  const int per = w_wave ? WPER : xper;
  const uint16_t* src[kPer];
  uint32_t dst[kPer];
#pragma unroll
  for (int i = 0; i < kPer; ++i) {
    if (w_wave) {
      const int slot = (wave * WPER + i) % (4 * NTMAX);
      const int r = slot * 8 + (lane >> 3), j = min(r >> 5, ntl - 1), rr = r & 31;
      const int pc = (lane & 7) ^ ((r >> 1) & 7);
      int64_t row;
      if constexpr (SILU) row = rr < 16 ? (int64_t)(tile0 + j) * 16 + rr : (p.N >> 1) + (int64_t)(tile0 + j) * 16 + (rr - 16);
      else row = (int64_t)(tile0 + j) * 32 + rr;
      src[i] = p.w + row * K + (int64_t)st0 * 64 + pc * 8;
      dst[i] = lds0 + slot * 1024;
    } else {
      const int slot = ((wave - NWW) * xper + i) % (4 * MT);
      const int r = slot * 8 + (lane >> 3);
      const int pc = (lane & 7) ^ ((r >> 1) & 7);
      src[i] = p.x + (int64_t)min(r, M - 1) * K + (int64_t)st0 * 64 + pc * 8;
      dst[i] = lds0 + xring + slot * 1024;
    }
  }
  const uint32_t cstride = w_wave ? kWStride : xstride;
  constexpr int kWWait = (SW - 2) * WPER, kXWait = (SX - 2) * XPER;
  // chunk s (relative to st0) of this wavefront's ring -> slot
#define SUBSPEC_WD_ISSUE(S, SLOT)                                                                          \
  do {                                                                                             \
    const int s_ = min((S), nst - 1);                                                              \
    _Pragma("unroll") for (int i_ = 0; i_ < kPer; ++i_)                                            \
      if (i_ < per) wd_dma16(__builtin_amdgcn_readfirstlane(dst[i_] + (SLOT) * cstride), src[i_] + s_ * 64); \
  } while (0)

  if (w_wave) {
#pragma unroll
    for (int s = 0; s < SW - 1; ++s) SUBSPEC_WD_ISSUE(s, s);
  } else if (x_wave) {
#pragma unroll
    for (int s = 0; s < SX - 1; ++s) SUBSPEC_WD_ISSUE(s, s);
  }

  // ---- this wavefront's tiles
  const int wn = wave / WM;
  const int wm = WM == 4 ? (wave + 2 * wn) & 3 : wave % WM;      // the two wavefronts of a SIMD take unlike shares
  wd_v16f acc[NH][MG];
#pragma unroll
  for (int i = 0; i < NH; ++i)
#pragma unroll
    for (int k = 0; k < MG; ++k)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][k][r] = 0.f;
  const uint32_t sw = (uint32_t)((lr >> 1) & 7);
  uint32_t opoff[4];
#pragma unroll
  for (int s = 0; s < 4; ++s) opoff[s] = (uint32_t)lr * 128 + (((uint32_t)(2 * s + g) ^ sw) << 4);

  // The K loop, instantiated for the number of weight tiles (NI) and row tiles (NK) this wavefront really has: a test
  // around every matrix instruction would make the accumulators cross basic blocks (register copies at every join).
  const int ni = wn >= ntl ? 0 : min((ntl - wn + WN - 1) / WN, NH), nk = wm >= MT ? 0 : min((MT - wm + WM - 1) / WM, MG);
  auto k_loop = [&](auto ni_c, auto nk_c) {
    constexpr int NI = decltype(ni_c)::value, NK = decltype(nk_c)::value;
    // Operands of the next 16-k step are read while the current step multiplies; the first step of the next chunk is
    // read right behind the barrier that publishes it, in front of the last products of this chunk.
    wd_u4 a0[NI ? NI : 1], b0[NK ? NK : 1], a1[NI ? NI : 1], b1[NK ? NK : 1];
    int wslot = 0, xslot = 0, wnext = SW - 1, xnext = SX - 1;
#define SUBSPEC_WD_READ(A, B, S)                                                                             \
    do {                                                                                             \
      const uint8_t* wst_ = wd_lds + wslot * kWStride + wn * 4096 + opoff[S];                        \
      const uint8_t* xst_ = wd_lds + xring + xslot * xstride + wm * 4096 + opoff[S];                 \
      _Pragma("unroll") for (int i = 0; i < NI; ++i) A[i] = *(const wd_u4*)(wst_ + WN * i * 4096);   \
      _Pragma("unroll") for (int k = 0; k < NK; ++k) B[k] = *(const wd_u4*)(xst_ + WM * k * 4096);   \
    } while (0)
#define SUBSPEC_WD_MUL(A, B)                                                                                 \
    _Pragma("unroll") for (int i = 0; i < NI; ++i)                                                   \
      _Pragma("unroll") for (int k = 0; k < NK; ++k) acc[i][k] = wd_mfma<DT>(A[i], B[k], acc[i][k])
    if (w_wave) wd_wait_vmcnt<kWWait>();
    else if (x_wave) wd_wait_vmcnt<kXWait>();
    __syncthreads();
    if (w_wave) SUBSPEC_WD_ISSUE(SW - 1, wnext);
    else if (x_wave) SUBSPEC_WD_ISSUE(SX - 1, xnext);
    SUBSPEC_WD_READ(a0, b0, 0);
    for (int it = 0; it < nst; ++it) {
      SUBSPEC_WD_READ(a1, b1, 1);
      __builtin_amdgcn_sched_barrier(0);
      SUBSPEC_WD_MUL(a0, b0);
      __builtin_amdgcn_sched_barrier(0);
      SUBSPEC_WD_READ(a0, b0, 2);
      __builtin_amdgcn_sched_barrier(0);
      SUBSPEC_WD_MUL(a1, b1);
      __builtin_amdgcn_sched_barrier(0);
      SUBSPEC_WD_READ(a1, b1, 3);
      __builtin_amdgcn_sched_barrier(0);
      SUBSPEC_WD_MUL(a0, b0);
      __builtin_amdgcn_sched_barrier(0);
      wslot = wslot + 1 == SW ? 0 : wslot + 1;
      xslot = xslot + 1 == SX ? 0 : xslot + 1;
      wnext = wnext + 1 == SW ? 0 : wnext + 1;
      xnext = xnext + 1 == SX ? 0 : xnext + 1;
      if (it + 1 < nst) {
        // the last operands of this chunk are in registers (the wait), so its slots may be overwritten behind the barrier
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        if (w_wave) wd_wait_vmcnt<kWWait>();
        else if (x_wave) wd_wait_vmcnt<kXWait>();
        __syncthreads();
        if (w_wave) SUBSPEC_WD_ISSUE(it + SW, wnext);
        else if (x_wave) SUBSPEC_WD_ISSUE(it + SX, xnext);
        SUBSPEC_WD_READ(a0, b0, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
      SUBSPEC_WD_MUL(a1, b1);
      __builtin_amdgcn_sched_barrier(0);
    }
#undef SUBSPEC_WD_READ
#undef SUBSPEC_WD_MUL
  };
  bool done = false;
  auto try_shape = [&](auto ni_c, auto nk_c) {
    if (!done && ni == decltype(ni_c)::value && nk == decltype(nk_c)::value) { k_loop(ni_c, nk_c); done = true; }
  };
  if (ni == 0 || nk == 0) { k_loop(std::integral_constant<int, 0>{}, std::integral_constant<int, 0>{}); done = true; }
  try_shape(std::integral_constant<int, 1>{}, std::integral_constant<int, 1>{});
  if constexpr (NH >= 2) try_shape(std::integral_constant<int, 2>{}, std::integral_constant<int, 1>{});
  if constexpr (NH >= 3) try_shape(std::integral_constant<int, 3>{}, std::integral_constant<int, 1>{});
  if constexpr (MG >= 2) {
    try_shape(std::integral_constant<int, 1>{}, std::integral_constant<int, 2>{});
    if constexpr (NH >= 2) try_shape(std::integral_constant<int, 2>{}, std::integral_constant<int, 2>{});
    if constexpr (NH >= 3) try_shape(std::integral_constant<int, 3>{}, std::integral_constant<int, 2>{});
  }
  if constexpr (MG >= 3) {
    try_shape(std::integral_constant<int, 1>{}, std::integral_constant<int, 3>{});
    if constexpr (NH >= 2) try_shape(std::integral_constant<int, 2>{}, std::integral_constant<int, 3>{});
    if constexpr (NH >= 3) try_shape(std::integral_constant<int, 3>{}, std::integral_constant<int, 3>{});
  }
  static_assert(NH <= 3 && MG <= 3, "instantiated shapes");
#undef SUBSPEC_WD_ISSUE

  // ---- output: lane -> row m = 32 t + lr; register r -> column 8 (r / 4) + 4 g + r % 4 of the weight tile
  const int ks = blockIdx.y;
#pragma unroll
  for (int i = 0; i < NH; ++i) {
    const int j = wn + WN * i;
    if (j >= ntl) continue;
#pragma unroll
    for (int k = 0; k < MG; ++k) {
      const int t = wm + WM * k;
      if (t >= MT) continue;
      const int m = t * 32 + lr;
      if (m >= M) continue;
      if constexpr (SILU) {
        const int64_t F = p.N >> 1;
#pragma unroll
        for (int q = 0; q < 2; ++q) {
          const int64_t f = (int64_t)(tile0 + j) * 16 + 8 * q + 4 * g;
          float o[4];
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const float bg = p.bias ? Elem<DT>::load(p.bias, f + e) : 0.f, bu = p.bias ? Elem<DT>::load(p.bias, F + f + e) : 0.f;
            const float gate = Elem<DT>::round(acc[i][k][4 * q + e] + bg), up = Elem<DT>::round(acc[i][k][8 + 4 * q + e] + bu);
            o[e] = Elem<DT>::round(gate / (1.f + __expf(-gate))) * up;
          }
          *(wd_u2*)(p.y + (int64_t)m * F + f) = wd_u2{wd_pack2<DT>(o[0], o[1]), wd_pack2<DT>(o[2], o[3])};
        }
      } else {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int64_t n = (int64_t)(tile0 + j) * 32 + 8 * q + 4 * g;
          if (p.splits > 1) {
            *(float4*)(p.partial + ((int64_t)ks * M + m) * p.N + n) =
                make_float4(acc[i][k][4 * q], acc[i][k][4 * q + 1], acc[i][k][4 * q + 2], acc[i][k][4 * q + 3]);
          } else {
            float o[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              float v = acc[i][k][4 * q + e] + (p.bias ? Elem<DT>::load(p.bias, n + e) : 0.f);
              if (p.residual) v = Elem<DT>::round(v) + Elem<DT>::load(p.residual, (int64_t)m * p.N + n + e);
              o[e] = v;
            }
            *(wd_u2*)(p.y + (int64_t)m * p.N + n) = wd_u2{wd_pack2<DT>(o[0], o[1]), wd_pack2<DT>(o[2], o[3])};
          }
        }
      }
    }
  }
}


constexpr int kWideMaxRows = 384;
// Launch shape of the kernel above.  A workgroup takes an even share of the weight tiles, at most five; short N is
// spread over the chip by splitting K (partials in fp32, summed in split order by dense_reduce_kernel): two tiles per
// workgroup for K of a few thousand, four for the long K of a down projection, as many K ranges as keep about 256
// workgroups, each at least six chunks long.
struct WidePlan { int wgs, splits, chunks_per_split; };
static WidePlan wide_plan(int64_t N, int64_t K, bool silu) {
  const int n_tiles = (int)(N / 32), chunks = (int)(K / 64);
  const int nt = (silu || n_tiles >= 5 * 192) ? 5 : chunks > 128 ? 4 : 2;
  WidePlan pl;
  pl.wgs = (n_tiles + nt - 1) / nt;
  int splits = silu ? 1 : std::max(1, std::min(8, 256 / pl.wgs));
  splits = std::min(splits, std::max(1, chunks / 6));
  pl.chunks_per_split = (chunks + splits - 1) / splits;
  pl.splits = (chunks + pl.chunks_per_split - 1) / pl.chunks_per_split;
  return pl;
}
static bool wide_applies(int64_t M, int64_t N) { return M > 32 && M <= kWideMaxRows && N % 32 == 0; }

template <int DT, bool SILU>
static void launch_wide(const WideParams& p, const WidePlan& pl, hipStream_t st) {
  const dim3 grid((unsigned)pl.wgs, (unsigned)pl.splits);
  // rows <= 64: five wavefronts copy weights four chunks deep (the kernel streams); <= 256: three activation slots;
  // <= 384: two (LDS holds no more beside the weights)
  if (p.M <= 64)
    hipLaunchKernelGGL((dense_wide_kernel<DT, 2, 1, 5, 4, 4, 5, 4, 2, 4, SILU>), grid, dim3(512), 0, st, p);
  else if (p.M <= 256)
    hipLaunchKernelGGL((dense_wide_kernel<DT, 4, 2, 5, 3, 3, 2, 10, 4, 8, SILU>), grid, dim3(512), 0, st, p);
  else
    hipLaunchKernelGGL((dense_wide_kernel<DT, 4, 3, 5, 3, 2, 2, 10, 6, 8, SILU>), grid, dim3(512), 0, st, p);
}

struct DnPlan { int wgs, row_tiles, splits, groups_per_split; };
// Tiles per workgroup, measured with weights streamed from HBM (a different matrix every call): with few rows the
// kernel mostly streams weights and small workgroups win -- one tile, or two from 1024 tiles on, where a wavefront's
// activation block is worth sharing (M = 8: 37888x3584 52.9 / 45.0 / 49.5 us at one / two / four tiles, 152064x3584
// 197.9 / 167.3 / 170.0 us, 3584x3584 8.2 / 10.5 / 14.8 us); at M = 64 every wavefront also fetches a [64 x 64]
// activation block per 64 k, which more tiles per workgroup amortise (4608x3584, M = 64: 16.1 us at two tiles, 25.4 us
// at one; 37888x3584: 66.8 us at four, 77.1 at two, 120 at one).
static DnPlan dn_plan(int64_t M, int64_t N, int64_t K) {
  const int G = (int)(K / kDnGroup);
  const int64_t tiles = N / 16, slots = M <= 16 ? 4096 : M <= 32 ? 1024 : 256;
  const int64_t want = (tiles + slots - 1) / slots;
  int row_tiles = want <= 1 ? 1 : want <= 2 ? 2 : 4;
  if (M <= 16) row_tiles = tiles >= 1024 ? 2 : 1;
  // More than 32 rows over a long K (the down projection, 3584 x 18944): one tile per workgroup fetches four bytes
  // of activations for every byte of weights; four tiles and four K ranges keep as many workgroups with a quarter of
  // that (M = 64: 46.7 us with the reduction against 61.5 us).
  const bool long_k = M > 32 && G >= 224;
  if (long_k) row_tiles = 4;
  const int64_t wgs = (tiles + row_tiles - 1) / row_tiles;
  int splits = (int)std::max<int64_t>(1, (slots + wgs / 2) / wgs);
  splits = std::min(splits, std::max(1, G / 112));             // a split costs a second launch: only for long K (two at K = 18944)
  if (long_k) splits = 4;
  splits = std::min(splits, 16);
  int gps = (G + splits - 1) / splits;
  gps = (gps + 3) / 4 * 4;
  splits = (G + gps - 1) / gps;
  return DnPlan{(int)wgs, row_tiles, splits, gps};
}

// gate|up projection with the SwiGLU output stage: x [M, K], W [2F, K] (gate rows first), act [M, F]
template <int DT>
static int run_dense_silu(const void* x, const void* w, const void* bias, void* act, int64_t M, int64_t N, int64_t K,
                          hipStream_t st) {
  if (wide_applies(M, N)) {
    const WidePlan pl = wide_plan(N, K, true);
    const WideParams p{(const uint16_t*)x, (const uint16_t*)w, (const uint16_t*)bias, nullptr, (uint16_t*)act, nullptr,
                       (int)M, (int)K, N, (int)(N / 32), 1, pl.chunks_per_split};
    {
      DominantKernelTimer timer(st);
      launch_wide<DT, true>(p, pl, st);
    }
    SUBSPEC_CHECK_HIP(hipGetLastError());
    return SUBSPEC_OK;
  }
  const int64_t pairs = N / 32;
  // tile pairs per workgroup: one with few activation rows (more, smaller workgroups stream weights faster), three
  // above 32 rows, where a workgroup's activation blocks are amortised over more tiles (37888 x 3584, M = 64: 79.9 us
  // against 87.1 us at two pairs)
  const int rt = M <= 32 ? 2 : 6;
  const int64_t wgs = (pairs + rt / 2 - 1) / (rt / 2);
  const dim3 grid((unsigned)wgs, 1);
  const int G = (int)(K / kDnGroup);
#define SUBSPEC_DN_SILU(MT, RT)                                                                                    \
  hipLaunchKernelGGL((dense_gemm_kernel<DT, MT, RT, true>), grid, dim3(kDnThreads), 0, st, (const uint16_t*)x,    \
                     (const uint16_t*)w, (const uint16_t*)bias, (const uint16_t*)nullptr, (uint16_t*)act, (float*)nullptr,     \
                     (int)M, N, (int)K, 1, (G + 3) / 4 * 4)
  DominantKernelTimer timer(st);
  if (M <= 16) SUBSPEC_DN_SILU(1, 2);
  else if (M <= 32) SUBSPEC_DN_SILU(2, 2);
  else SUBSPEC_DN_SILU(4, 6);
#undef SUBSPEC_DN_SILU
  SUBSPEC_CHECK_HIP(hipGetLastError());
  return SUBSPEC_OK;
}

template <int DT>
static int run_dense(const void* x, const void* w, const void* bias, const void* residual, void* y, int64_t M, int64_t N,
                     int64_t K, void* workspace, hipStream_t st, int* pending_splits) {
  if (pending_splits) *pending_splits = 1;
  if (wide_applies(M, N)) {
    const WidePlan pl = wide_plan(N, K, false);
    const WideParams p{(const uint16_t*)x, (const uint16_t*)w, (const uint16_t*)bias, (const uint16_t*)residual, (uint16_t*)y,
                       (float*)workspace, (int)M, (int)K, N, (int)(N / 32), pl.splits, pl.chunks_per_split};
    {
      DominantKernelTimer timer(st);
      launch_wide<DT, false>(p, pl, st);
    }
    if (pl.splits > 1 && pending_splits) *pending_splits = pl.splits;
    else if (pl.splits > 1)
      hipLaunchKernelGGL((dense_reduce_kernel<DT>), dim3((unsigned)((M * N + 255) / 256)), dim3(256), 0, st, (const float*)workspace,
                         (const uint16_t*)bias, (const uint16_t*)residual, (uint16_t*)y, M, N, pl.splits);
    SUBSPEC_CHECK_HIP(hipGetLastError());
    return SUBSPEC_OK;
  }
  const DnPlan pl = dn_plan(M, N, K);
  float* partial = (float*)workspace;
  const dim3 grid((unsigned)pl.wgs, (unsigned)pl.splits);
#define SUBSPEC_DN_LAUNCH(MT, RT)                                                                                  \
  hipLaunchKernelGGL((dense_gemm_kernel<DT, MT, RT>), grid, dim3(kDnThreads), 0, st, (const uint16_t*)x,           \
                     (const uint16_t*)w, (const uint16_t*)bias, (const uint16_t*)residual, (uint16_t*)y, partial, (int)M, N, (int)K, \
                     pl.splits, pl.groups_per_split)
#define SUBSPEC_DN_LAUNCH_MT(MT)                                                                                   \
  do {                                                                                                             \
    if (pl.row_tiles == 1) SUBSPEC_DN_LAUNCH(MT, 1);                                                               \
    else if (pl.row_tiles == 2) SUBSPEC_DN_LAUNCH(MT, 2);                                                          \
    else SUBSPEC_DN_LAUNCH(MT, 4);                                                                                 \
  } while (0)
  {
    DominantKernelTimer timer(st);
    if (M <= 16) SUBSPEC_DN_LAUNCH_MT(1);
    else if (M <= 32) SUBSPEC_DN_LAUNCH_MT(2);
    else SUBSPEC_DN_LAUNCH_MT(4);
  }
#undef SUBSPEC_DN_LAUNCH_MT
#undef SUBSPEC_DN_LAUNCH
  if (pl.splits > 1 && pending_splits) *pending_splits = pl.splits;
  else if (pl.splits > 1)
    hipLaunchKernelGGL((dense_reduce_kernel<DT>), dim3((unsigned)((M * N + 255) / 256)), dim3(256), 0, st, partial,
                       (const uint16_t*)bias, (const uint16_t*)residual, (uint16_t*)y, M, N, pl.splits);
  SUBSPEC_CHECK_HIP(hipGetLastError());
  return SUBSPEC_OK;
}

}  // namespace subspec

using namespace subspec;

extern "C" size_t subspec_dense_linear_workspace(int64_t M, int64_t N, int64_t K) {
  if (M <= 0 || N <= 0 || K <= 0) return 256;
  if (wide_applies(M, N)) {
    const WidePlan wp = wide_plan(N, K, false);
    return (wp.splits > 1 ? align_up((size_t)wp.splits * M * N * sizeof(float), 256) : 0) + 256;
  }
  const DnPlan pl = dn_plan(M, N, K);
  return (pl.splits > 1 ? align_up((size_t)pl.splits * M * N * sizeof(float), 256) : 0) + 256;
}

extern "C" int subspec_dense_linear(const void* x, const void* w, const void* bias, void* y, int dtype, int64_t M,
                                    int64_t N, int64_t K, void* workspace, size_t workspace_bytes, void* stream) {
  return dense_linear_ex(x, w, bias, nullptr, y, dtype, M, N, K, workspace, workspace_bytes, stream);
}

int subspec::dense_gate_up_silu_ex(const void* x, const void* w, const void* bias, void* act, int dtype, int64_t M, int64_t N,
                                   int64_t K, void* stream) {
  if (dtype != SUBSPEC_BF16 && dtype != SUBSPEC_F16)
    SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "dense_gate_up_silu: dtype %d not supported (bf16 / fp16 only)", dtype);
  if (!x || !w || !act) SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "dense_gate_up_silu: null pointer argument");
  if (M <= 0 || M > kWideMaxRows || N <= 0 || K <= 0 || N % 32 != 0 || K % kDnGroup != 0 || K > 65536)
    SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "dense_gate_up_silu: M=%lld N=%lld K=%lld; 1 <= M <= %d, N a multiple of 32, K of 64",
                 (long long)M, (long long)N, (long long)K, kWideMaxRows);
  // up to 32 rows: a workgroup's weight descriptor spans from its gate tiles to its up tiles, more than half the matrix
  if (M <= 32 && N * K * 2 >= ((int64_t)1 << 31))
    SUBSPEC_FAIL(SUBSPEC_ERR_LIMIT, "dense_gate_up_silu: N*K*2=%lld bytes exceed the 2 GiB descriptor range", (long long)(N * K * 2));
  if ((uintptr_t)x % 16 || (uintptr_t)w % 16 || (uintptr_t)act % 2)
    SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "dense_gate_up_silu: x and w must be 16-byte aligned");
  hipStream_t st = (hipStream_t)stream;
  if (dtype == SUBSPEC_BF16) return run_dense_silu<SUBSPEC_BF16>(x, w, bias, act, M, N, K, st);
  return run_dense_silu<SUBSPEC_F16>(x, w, bias, act, M, N, K, st);
}

extern "C" int subspec_dense_gate_up_silu(const void* x, const void* w, const void* bias, void* act, int dtype, int64_t M,
                                          int64_t N, int64_t K, void* stream) {
  return subspec::dense_gate_up_silu_ex(x, w, bias, act, dtype, M, N, K, stream);
}

int subspec::dense_linear_ex(const void* x, const void* w, const void* bias, const void* residual, void* y, int dtype, int64_t M,
                             int64_t N, int64_t K, void* workspace, size_t workspace_bytes, void* stream, int* pending_splits) {
  if (dtype != SUBSPEC_BF16 && dtype != SUBSPEC_F16)
    SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "dense_linear: dtype %d not supported (bf16 / fp16 only)", dtype);
  if (!x || !w || !y) SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "dense_linear: null pointer argument");
  if (M <= 0 || N <= 0 || K <= 0 || N % 16 != 0 || K % kDnGroup != 0)
    SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "dense_linear: M=%lld N=%lld K=%lld; N must be a multiple of 16 and K of 64",
                 (long long)M, (long long)N, (long long)K);
  if (M > kWideMaxRows) SUBSPEC_FAIL(SUBSPEC_ERR_LIMIT, "dense_linear: M=%lld exceeds the %d-row limit", (long long)M, kWideMaxRows);
  if (M > 64 && N % 32 != 0)
    SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "dense_linear: N=%lld must be a multiple of 32 for more than 64 rows", (long long)N);
  if (K > 65536) SUBSPEC_FAIL(SUBSPEC_ERR_LIMIT, "dense_linear: K=%lld too large", (long long)K);
  if ((uintptr_t)x % 16 || (uintptr_t)w % 16 || (uintptr_t)y % 2)
    SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "dense_linear: x and w must be 16-byte aligned");
  const size_t need = subspec_dense_linear_workspace(M, N, K);
  if (need > 256) {
    if (!workspace || workspace_bytes < need)
      SUBSPEC_FAIL(SUBSPEC_ERR_WORKSPACE, "dense_linear: workspace of %zu bytes is smaller than the %zu required",
                   workspace_bytes, need);
    if ((uintptr_t)workspace % 16) SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "dense_linear: workspace must be 16-byte aligned");
  }
  hipStream_t st = (hipStream_t)stream;
  if (dtype == SUBSPEC_BF16) return run_dense<SUBSPEC_BF16>(x, w, bias, residual, y, M, N, K, workspace, st, pending_splits);
  return run_dense<SUBSPEC_F16>(x, w, bias, residual, y, M, N, K, workspace, st, pending_splits);
}
