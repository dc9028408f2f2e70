// Tree-masked GQA attention of the draft tree against the static KV cache, for gfx950.
//
// Replaces the reference's HF sdpa_attention_forward forced to the math backend with an additive
// finfo.min mask over the whole static cache plus repeat_kv (run/pipelines/run_test.py:64;
// specdecodes/models/generators/classic_sd.py:57-109; mask from cpu_tree.py:263-286 and
// utils/utils.py:4-6): O = softmax(Q K^T * scale + M) V, where tree row i sees the whole prefix and,
// among the tree slots, only node i and its ancestors.
//
// Layout and mapping
//   q        [B, Hq, n, D]            (D = 128; a launch takes 64 query rows, more rows are more launches)
//   k, v     [B, Hkv, S, D]           static cache; rows [0, prefix) are the prompt, rows
//                                     [prefix, prefix + slots) hold the tree nodes (slots <= 512)
//   anc      [B or 1, n, words] u64   bit j of row i (word j / 64): query row i may attend to tree slot j
//                                     (the node in slot j is the row's node or one of its ancestors);
//                                     words = ceil(slots / 64), at most 8
//   out      [B, n, Hq, D]
// One workgroup owns several query heads of one KV head and one chunk of the keys, so a staged K/V block feeds
// several heads' worth of matrix work; workgroups that share a KV chunk get consecutive slots on the same XCD (linear
// id modulo 8), so the chunk is fetched from HBM once and served from that XCD's L2.  Scores are produced TRANSPOSED,
// S^T = K Q^T: the accumulator then holds, per lane, keys of ONE query, the row maximum / sum need one or two cross-lane
// steps, and packed accumulator registers are the B operand of the second product O^T = V^T P^T (with the matching key
// permutation applied to the V^T operand, read from row-major V by transposing LDS reads), so probabilities go from one
// MFMA to the next without leaving registers.  Prefix keys need no mask at all.  Three kernels, chosen by attn_plan:
//   * tree_attention_kernel: windows of up to 16 rows (a level of the draft tree).  v_mfma_f32_16x16x32, a wavefront
//     is a whole head (one 16-row tile), eight heads (a whole 7:1 GQA group) share the staged keys.
//   * tree_attention32_kernel: 17 to 64 rows, one sequence or few (sequence, head) pairs, and every paged call.
//     v_mfma_f32_32x32x16, a wavefront owns 32 rows of a head; K / V blocks travel through two register sets into two
//     padded LDS stages, two blocks' requests in flight.
//   * tree_attention_pp_kernel: 17 to 64 rows, several sequences with at least 128 (sequence, head) pairs (config 3,
//     B = 8).  The same tiles; the two wavefronts of a SIMD alternate between a matrix phase and a softmax phase, K / V
//     blocks are copied from memory straight into a ring of four LDS stages.
// When the keys are split over several workgroups the per-chunk results are merged by a second launch.
// Algorithmic bytes per batch element = K+V rows actually attended + Q + O; at config 3 the arithmetic intensity
// (405 FLOP/B) is above the chip's ridge, so the bound that applies is the matrix pipe, not HBM.
#include "common.h"
#include <algorithm>

namespace subspec {

constexpr int kAttnThreads = 512;         // 256 for the one-head shape
constexpr int kAttnRows = 64;          // query rows per head
constexpr int kAttnD = 128;
constexpr int kKeyBlock = 64;
constexpr int kKStride = kAttnD + 8;   // LDS row stride (elements) of the K tile
constexpr int kVStride = kAttnD + 16;  // LDS row stride (elements) of the V tile: 8-dword rows of the transposing reads tile the banks
constexpr int kXcds = 8;

typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef float v4f __attribute__((ext_vector_type(4)));

template <int DT>
__device__ __forceinline__ v4f mfma32(uint4 a, uint4 b, v4f c) {
  if constexpr (DT == SUBSPEC_BF16) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf, a), __builtin_bit_cast(v8bf, b), c, 0, 0, 0);
  } else {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(v8h, a), __builtin_bit_cast(v8h, b), c, 0, 0, 0);
  }
}

typedef __bf16 v2bf_t __attribute__((ext_vector_type(2)));
typedef _Float16 v2h_t __attribute__((ext_vector_type(2)));
typedef float v2f_t __attribute__((ext_vector_type(2)));


// Transposing LDS read of 16-bit elements (ds_read_b64_tr_b16): within each group of 16 lanes,
// lane i receives element i%4 of the four 8-byte rows addressed by lanes i/4, i/4 + 4, i/4 + 8,
// i/4 + 12 of the group.
typedef short v4s_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ uint2 lds_read_tr16(const uint16_t* p) {
  const v4s_t v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) v4s_t*)p);
  return __builtin_bit_cast(uint2, v);
}

struct AttnParams {
  int64_t batch, hq, hkv, n_rows, n_slots, seq_stride, prefix, anc_batch_stride;
  int mask_words;              // 64-bit words per ancestor bitset: ceil(n_slots / 64)
  int row0, win_rows;          // this launch covers query rows row0 .. row0 + win_rows - 1 (win_rows <= 64) of n_rows ...
  int windows;                 // ... or `windows` > 1 windows of 64 rows from row0 on (32-row kernels): see attn_window
  int chunks;
  int64_t chunk_keys;          // multiple of kKeyBlock
  int pairs_per_kv;            // workgroups (groups of 4 or 8 query heads) per KV head
  int64_t units;               // batch * hkv * chunks
  float scale_log2;            // softmax scale * log2(e)
  // paged cache (one request): row p of K lives at page_table[p >> page_shift], token p & (page_len - 1) of
  // a pool layer [max_pages][2 (K, V)][page_len][hkv][128]; V is v_delta elements behind K
  // when not null, the prefix length is read here by the kernel and `prefix` above is only the upper bound the grid
  // and the key chunks were laid out for (a captured launch replayed while the prefix grows)
  const int64_t* prefix_dev;
  const int32_t* page_table;
  int page_shift, max_pages;
  int64_t page_stride, tok_stride, v_delta;   // elements
};

// Several windows of 64 query rows in one launch (a tree of more than 64 rows in the target): the windows of a sequence
// read the same keys, so they are laid out as further batch entries -- virtual entry vb = window * batch + b -- that share
// the cache of sequence b; split-KV partials are kept per virtual entry.
struct AttnWindow { int b, row0, win_rows; };
__device__ __forceinline__ AttnWindow attn_window(const AttnParams& ap, int vb) {
  const int w = vb / (int)ap.batch;
  const int row0 = ap.row0 + w * kAttnRows;
  return AttnWindow{vb - w * (int)ap.batch, row0, ap.windows > 1 ? min((int)ap.n_rows - row0, kAttnRows) : ap.win_rows};
}

// THREADS = 512: eight wavefronts; 256: four wavefronts, each 16 rows of ONE head (ROWT = 1, WPH = 4) -- with 33 to 64
// query rows and few sequences this shape gets its workgroups from the heads instead of from key chunks, so the
// split-KV partials (fp32, rows x 128 per head and chunk) stay below the K / V bytes themselves.
template <int DT, bool PAGED, int ROWT, int WPH, int THREADS = kAttnThreads>
__global__ __launch_bounds__(THREADS) __attribute__((amdgpu_waves_per_eu(2, 2))) void tree_attention_kernel(
    const uint16_t* __restrict__ q, const uint16_t* __restrict__ kc, const uint16_t* __restrict__ vc,
    const uint64_t* __restrict__ anc, AttnParams ap, uint16_t* __restrict__ out, float* __restrict__ part_o,
    float* __restrict__ part_ml) {
  // two stages of (K, V), both row-major [key][d]: block i+1 is written while block i is multiplied
  __shared__ __attribute__((aligned(16))) uint16_t Ks2[2][kKeyBlock * kKStride];
  __shared__ __attribute__((aligned(16))) uint16_t Vs2[2][kKeyBlock * kVStride];

  // workgroups of one (batch, kv head, chunk) unit sit in consecutive slots of one XCD
  // Every kernel argument is wanted in a scalar register HERE: left alone, the compiler fetches the fields of the
  // parameter block where they are first used, in six batches with a wait each -- six dependent round trips to the
  // scalar cache (cold at every launch) before the first key is requested.
  asm volatile("" ::"s"(ap.batch), "s"(ap.hq), "s"(ap.hkv), "s"(ap.n_rows), "s"(ap.n_slots), "s"(ap.seq_stride), "s"(ap.prefix),
               "s"(ap.anc_batch_stride), "s"(ap.mask_words), "s"(ap.row0), "s"(ap.win_rows), "s"(ap.chunks), "s"(ap.chunk_keys),
               "s"(ap.pairs_per_kv), "s"(ap.units), "s"(ap.scale_log2), "s"(ap.prefix_dev), "s"(ap.page_table),
               "s"(ap.page_shift), "s"(ap.max_pages), "s"(ap.page_stride), "s"(ap.tok_stride), "s"(ap.v_delta));
  asm volatile("" ::"s"(q), "s"(kc), "s"(vc), "s"(anc), "s"(out), "s"(part_o), "s"(part_ml));
  const uint32_t lin = blockIdx.x;
  const int xcd = (int)(lin % (uint32_t)kXcds);
  const uint32_t slot = lin / (uint32_t)kXcds;
  const int pair = (int)(slot % (uint32_t)ap.pairs_per_kv);
  const uint32_t unit = (slot / (uint32_t)ap.pairs_per_kv) * (uint32_t)kXcds + (uint32_t)xcd;
  if ((int64_t)unit >= ap.units) return;
  const int chunk = (int)(unit % (uint32_t)ap.chunks);
  const uint32_t bkv = unit / (uint32_t)ap.chunks;
  const int kvh = (int)(bkv % (uint32_t)ap.hkv), b = (int)(bkv / (uint32_t)ap.hkv);
  const int group = (int)((uint32_t)ap.hq / (uint32_t)ap.hkv);

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int lq = lane & 15, lg = lane >> 4;            // query column of the lane, lane group
  constexpr int kHeadsPerWG = (THREADS / 64) / WPH;    // heads of one KV head that share a workgroup's K / V stages
  const int head_in_group = pair * kHeadsPerWG + wave / WPH;
  const bool head_ok = head_in_group < group;
  const int qh = kvh * group + (head_ok ? head_in_group : 0);
  const int bh = b * (int)ap.hq + qh;
  const int n = (int)ap.n_rows;
  const int64_t prefix = ap.prefix_dev ? min(max(*ap.prefix_dev, (int64_t)0), ap.prefix) : ap.prefix;
  const int64_t kv_len = prefix + ap.n_slots;

  // ---- Q^T operands of the wave's two 16-row tiles: Q[row][32*ks + 8*lg .. +7]
  int row[ROWT];
  bool row_ok[ROWT];
  uint4 qreg[ROWT][kAttnD / 32];
  const uint64_t* row_bits[ROWT];                          // the row's ancestor bitset (mask_words words)
#pragma unroll
  for (int nt = 0; nt < ROWT; ++nt) {
    row[nt] = (wave % WPH) * (16 * ROWT) + nt * 16 + lq;   // row inside this launch's window
    row_ok[nt] = head_ok && row[nt] < ap.win_rows;
    const int grow = ap.row0 + (row_ok[nt] ? row[nt] : 0);
    const uint16_t* qp = q + ((int64_t)bh * n + grow) * kAttnD;
#pragma unroll
    for (int ks = 0; ks < kAttnD / 32; ++ks)
      qreg[nt][ks] = row_ok[nt] ? *(const uint4*)(qp + ks * 32 + lg * 8) : make_uint4(0, 0, 0, 0);
    row_bits[nt] = anc + ((int64_t)b * ap.anc_batch_stride + grow) * ap.mask_words;
  }

  v4f oacc[ROWT][kAttnD / 16];
  float m_run[ROWT], l_run[ROWT];
#pragma unroll
  for (int nt = 0; nt < ROWT; ++nt) {
    m_run[nt] = -INFINITY;
    l_run[nt] = 0.f;
#pragma unroll
    for (int mt = 0; mt < kAttnD / 16; ++mt) oacc[nt][mt] = v4f{0.f, 0.f, 0.f, 0.f};
  }

  // contiguous cache [B, Hkv, S, 128]: row p of this head at base + p * 128.  Paged pool: see AttnParams.
  const uint16_t* kbase = PAGED ? kc + (int64_t)kvh * kAttnD : kc + ((int64_t)b * ap.hkv + kvh) * ap.seq_stride * kAttnD;
  const uint16_t* vbase = PAGED ? kbase + ap.v_delta : vc + ((int64_t)b * ap.hkv + kvh) * ap.seq_stride * kAttnD;
  auto row_offset = [&](int64_t p) -> int64_t {          // element offset of cache row p from kbase / vbase
    if constexpr (PAGED) {
      const int page = min(max(ap.page_table[p >> ap.page_shift], 0), ap.max_pages - 1);   // a bad table must not fault
      return (int64_t)page * ap.page_stride + (p & ((1 << ap.page_shift) - 1)) * ap.tok_stride;
    } else {
      return p * kAttnD;
    }
  };
  const int64_t key0 = (int64_t)chunk * ap.chunk_keys;
  const int64_t key1 = min(key0 + ap.chunk_keys, kv_len);

  // staging registers: this thread's share (2 x 16 bytes of K, 2 x 16 bytes of V) of one 64-key
  // block; the next block is requested as soon as the current one sits in LDS, so the request
  // travels while the current block is multiplied.  Plain scalars on purpose: arrays captured by
  // a lambda end up in memory and every prefetch would be waited for at once.
  constexpr int KPT = 1024 / THREADS;                  // keys of a block per thread: 2 (512 threads) or 4 (256)
  constexpr int KSTEP = 64 / KPT;
  uint4 k0, k1, k2, k3, v0, v1, v2, v3;
  (void)k2; (void)k3; (void)v2; (void)v3;
  const int skey = tid >> 4, sdc = tid & 15;           // this thread stages keys skey + KSTEP * i, d-chunk sdc
#define SUBSPEC_ATTN_FETCH(KB)                                                                   \
  do {                                                                                           \
    const int64_t p0_ = row_offset(min((KB) + skey, kv_len - 1));                                \
    const int64_t p1_ = row_offset(min((KB) + KSTEP + skey, kv_len - 1));                        \
    k0 = *(const uint4*)(kbase + p0_ + sdc * 8);                                                 \
    k1 = *(const uint4*)(kbase + p1_ + sdc * 8);                                                 \
    v0 = *(const uint4*)(vbase + p0_ + sdc * 8);                                                 \
    v1 = *(const uint4*)(vbase + p1_ + sdc * 8);                                                 \
    if constexpr (KPT == 4) {                                                                    \
      const int64_t p2_ = row_offset(min((KB) + 2 * KSTEP + skey, kv_len - 1));                  \
      const int64_t p3_ = row_offset(min((KB) + 3 * KSTEP + skey, kv_len - 1));                  \
      k2 = *(const uint4*)(kbase + p2_ + sdc * 8);                                               \
      k3 = *(const uint4*)(kbase + p3_ + sdc * 8);                                               \
      v2 = *(const uint4*)(vbase + p2_ + sdc * 8);                                               \
      v3 = *(const uint4*)(vbase + p3_ + sdc * 8);                                               \
    }                                                                                            \
  } while (0)
#define SUBSPEC_ATTN_STAGE(BUF)                                                                  \
  do {                                                                                           \
    uint16_t* ksw_ = Ks2[BUF];                                                                   \
    uint16_t* vsw_ = Vs2[BUF];                                                                   \
    *(uint4*)(ksw_ + skey * kKStride + sdc * 8) = k0;                                            \
    *(uint4*)(ksw_ + (skey + KSTEP) * kKStride + sdc * 8) = k1;                                  \
    *(uint4*)(vsw_ + skey * kVStride + sdc * 8) = v0;                                            \
    *(uint4*)(vsw_ + (skey + KSTEP) * kVStride + sdc * 8) = v1;                                  \
    if constexpr (KPT == 4) {                                                                    \
      *(uint4*)(ksw_ + (skey + 2 * KSTEP) * kKStride + sdc * 8) = k2;                            \
      *(uint4*)(ksw_ + (skey + 3 * KSTEP) * kKStride + sdc * 8) = k3;                            \
      *(uint4*)(vsw_ + (skey + 2 * KSTEP) * kVStride + sdc * 8) = v2;                            \
      *(uint4*)(vsw_ + (skey + 3 * KSTEP) * kVStride + sdc * 8) = v3;                            \
    }                                                                                            \
  } while (0)

  // mask words of the first block of this chunk that reaches into the tree (none does: the loads are harmless)
  uint64_t bits[ROWT][2];
  auto load_bits = [&](int w) {
#pragma unroll
    for (int nt = 0; nt < ROWT; ++nt) {
      bits[nt][0] = (row_ok[nt] && w < ap.mask_words) ? row_bits[nt][w] : 0ull;
      bits[nt][1] = (row_ok[nt] && w + 1 < ap.mask_words) ? row_bits[nt][w + 1] : 0ull;
    }
  };
  int held_word = (int)(max(max(key0, prefix / kKeyBlock * kKeyBlock) - prefix, (int64_t)0) >> 6);
  load_bits(held_word);

  SUBSPEC_ATTN_FETCH(key0);
  SUBSPEC_ATTN_STAGE(0);
  if (key0 + kKeyBlock < key1) SUBSPEC_ATTN_FETCH(key0 + kKeyBlock);

  int buf = 0;
  for (int64_t kb = key0; kb < key1; kb += kKeyBlock, buf ^= 1) {
    // one barrier per block: stage `buf` is complete, and everyone has left the other stage
    __syncthreads();
    if (kb + kKeyBlock < key1) {
      SUBSPEC_ATTN_STAGE(buf ^ 1);                     // next block -> the stage nobody reads now
      if (kb + 2 * kKeyBlock < key1) SUBSPEC_ATTN_FETCH(kb + 2 * kKeyBlock);
    }
    const uint16_t* Ks = Ks2[buf];
    const uint16_t* Vs = Vs2[buf];

    // ---- S^T tiles: 4 x (16 keys x 16 queries) per row tile; lane holds keys 16*kt + 4*lg + r of query lq.
    //      Scores stay unscaled; the softmax scale is folded into the exp2 argument.
    float s[ROWT][4][4];
    float mloc[ROWT];
#pragma unroll
    for (int nt = 0; nt < ROWT; ++nt) mloc[nt] = -INFINITY;
    const bool plain = kb + kKeyBlock <= prefix;    // block lies entirely in the prefix: no mask (uniform)
    // a 64-key block touches at most two consecutive words of the bitsets: word0 and word0 + 1.  They were
    // fetched before the loop for the first masked block; trees beyond 128 slots fetch again as the blocks move on.
    const int word0 = (int)(max(kb - prefix, (int64_t)0) >> 6);
    if (!plain && word0 != held_word) {                // uniform
      held_word = word0;
      load_bits(word0);
    }
    v4f acc[4][ROWT];
#pragma unroll
    for (int kt = 0; kt < 4; ++kt)
#pragma unroll
      for (int nt = 0; nt < ROWT; ++nt) acc[kt][nt] = v4f{0.f, 0.f, 0.f, 0.f};
    // eight independent accumulator chains (4 key tiles x 2 row tiles) keep the matrix pipe busy
#pragma unroll
    for (int ks = 0; ks < kAttnD / 32; ++ks) {
#pragma unroll
      for (int kt = 0; kt < 4; ++kt) {
        const uint4 a = *(const uint4*)(Ks + (kt * 16 + lq) * kKStride + ks * 32 + lg * 8);
#pragma unroll
        for (int nt = 0; nt < ROWT; ++nt) acc[kt][nt] = mfma32<DT>(a, qreg[nt][ks], acc[kt][nt]);
      }
    }
#pragma unroll
    for (int kt = 0; kt < 4; ++kt) {
      if (plain) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
#pragma unroll
          for (int nt = 0; nt < ROWT; ++nt) {
            s[nt][kt][r] = acc[kt][nt][r];
            mloc[nt] = fmaxf(mloc[nt], acc[kt][nt][r]);
          }
        }
      } else {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int64_t pos = kb + kt * 16 + lg * 4 + r;
          const bool in_range = pos < kv_len;
          const bool tree = pos >= prefix;
          const int rel = tree ? (int)(pos - prefix) : 0;   // tree slot, < 64 * mask_words when in range
          const int sh = rel & 63;
          const bool first_word = (rel >> 6) == word0;
#pragma unroll
          for (int nt = 0; nt < ROWT; ++nt) {
            const uint64_t word = first_word ? bits[nt][0] : bits[nt][1];
            const bool ok = in_range && (!tree || ((word >> sh) & 1ull));
            const float t = ok ? acc[kt][nt][r] : -INFINITY;
            s[nt][kt][r] = t;
            mloc[nt] = fmaxf(mloc[nt], t);
          }
        }
      }
    }
    // running maximum in units of raw scores (the scale is positive, so the order is the same)
    float mneg[ROWT];                                     // -max * scale_log2, the additive term of the exp2 argument
#pragma unroll
    for (int nt = 0; nt < ROWT; ++nt) {
      float mx = mloc[nt];
      mx = fmaxf(mx, __shfl_xor(mx, 16, kWave));
      mx = fmaxf(mx, __shfl_xor(mx, 32, kWave));
      const float m_new = fmaxf(m_run[nt], mx);
      const float m_use = m_new == -INFINITY ? 0.f : m_new;
      const float alpha = __builtin_amdgcn_exp2f((m_run[nt] - m_use) * ap.scale_log2);   // m_run = -inf -> 0
      m_run[nt] = m_new;
      mneg[nt] = -m_use * ap.scale_log2;
      if (__any(alpha != 1.0f)) {                      // the maximum settles after a few blocks
        l_run[nt] *= alpha;
#pragma unroll
        for (int mt = 0; mt < kAttnD / 16; ++mt) oacc[nt][mt] *= alpha;
      }
    }
    // ---- P^T as B operands straight from the accumulators: k index 8*lg + e of step j is key
    //      32*j + 16*(e/4) + 4*lg + e%4, i.e. registers of score tiles 2j and 2j+1
    uint4 pb[ROWT][2];
#pragma unroll
    for (int nt = 0; nt < ROWT; ++nt) {
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        float p[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          p[e] = __builtin_amdgcn_exp2f(fmaf(s[nt][2 * j + (e >> 2)][e & 3], ap.scale_log2, mneg[nt]));
          l_run[nt] += p[e];
        }
        pb[nt][j] = make_uint4(pack2<DT>(p[0], p[1]), pack2<DT>(p[2], p[3]), pack2<DT>(p[4], p[5]), pack2<DT>(p[6], p[7]));
      }
    }
    // ---- O^T += V^T P^T : 8 tiles of 16 head-dims, two 32-key steps, the same V^T operand for both row tiles.
    //      V sits row-major in LDS; the transposing LDS read hands lane (lq, lg) the values
    //      V[key_e][16*mt + lq], e = 0..3, when lane r of the 16-lane group supplies the address of
    //      V[key_{r/4}][16*mt + 4*(r%4)].  Two such reads (keys 32j + 4lg + e and 32j + 16 + 4lg + e)
    //      give the eight keys of the lane's k indices, in the order the P^T operand uses.
    const uint16_t* vlane = Vs + (lg * 4 + (lq >> 2)) * kVStride + (lq & 3) * 4;
#pragma unroll
    for (int mt = 0; mt < kAttnD / 16; ++mt) {
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const uint16_t* vp = vlane + (j * 32) * kVStride + mt * 16;
        const uint2 lo = lds_read_tr16(vp), hi = lds_read_tr16(vp + 16 * kVStride);
        const uint4 a = make_uint4(lo.x, lo.y, hi.x, hi.y);
#pragma unroll
        for (int nt = 0; nt < ROWT; ++nt) oacc[nt][mt] = mfma32<DT>(a, pb[nt][j], oacc[nt][mt]);
      }
    }
  }

#pragma unroll
  for (int nt = 0; nt < ROWT; ++nt) {
    // the four lane groups hold disjoint keys of the same query
    float l = l_run[nt];
    l += __shfl_xor(l, 16, kWave);
    l += __shfl_xor(l, 32, kWave);
    if (!row_ok[nt]) continue;
    if (ap.chunks == 1) {
      const float inv = l > 0.f ? 1.0f / l : 0.f;
      uint16_t* op = out + (((int64_t)b * n + ap.row0 + row[nt]) * ap.hq + qh) * kAttnD;
#pragma unroll
      for (int mt = 0; mt < kAttnD / 16; ++mt) {
        const v4f o = oacc[nt][mt];
        *(uint2*)(op + mt * 16 + lg * 4) = make_uint2(pack2<DT>(o[0] * inv, o[1] * inv), pack2<DT>(o[2] * inv, o[3] * inv));
      }
    } else {
      const int64_t pslot = ((int64_t)bh * ap.chunks + chunk) * kAttnRows + row[nt];
      float* po = part_o + pslot * kAttnD;
#pragma unroll
      for (int mt = 0; mt < kAttnD / 16; ++mt) {
        // The one-head shape (one sequence, 64 rows) writes twice the K / V bytes in partials over many chunks: as
        // streaming stores they drain while the kernel runs instead of at its end (config 3, B = 1: 20.7 -> 18.9 us).
        // With eight sequences (four chunks) the same stores cost 3 us: the merge then misses the L2.
        if constexpr (THREADS == 256) __builtin_nontemporal_store(oacc[nt][mt], (v4f*)(po + mt * 16 + lg * 4));
        else *(v4f*)(po + mt * 16 + lg * 4) = oacc[nt][mt];
      }
      if (lg == 0) { part_ml[pslot * 2] = m_run[nt] * ap.scale_log2; part_ml[pslot * 2 + 1] = l; }
    }
  }
}

// Merge of the per-chunk (O, max, sum) triples: 32 lanes x float4 cover the 128 dims of one
// (head, row); a workgroup takes blockDim.x / 32 rows (8, or 2 when the launch would otherwise be
// too small to fill the chip).  Slot of (bh, chunk c, row) = (bh * chunks + c) * 64 + row; maxima
// are stored already multiplied by scale * log2(e).
template <int DT>
__global__ __launch_bounds__(256) void tree_attention_merge_kernel(
    const float* __restrict__ part_o, const float* __restrict__ part_ml, AttnParams ap, uint16_t* __restrict__ out) {
  const int row = blockIdx.x * (blockDim.x >> 5) + (threadIdx.x >> 5), bh = blockIdx.y;
  if (row >= ap.win_rows) return;
  const int b = bh / (int)ap.hq, qh = bh % (int)ap.hq;
  const int d4 = threadIdx.x & 31;
  const int64_t slot0 = (int64_t)bh * ap.chunks * kAttnRows + row;     // chunk c: slot0 + c * kAttnRows
  float m = -INFINITY;
  v4f num = {0.f, 0.f, 0.f, 0.f};
  float den = 0.f;
  constexpr int kUpFront = 24;
  if (ap.chunks <= kUpFront) {
    // the usual case (a draft level has 12 to 18 chunks at prefixes of 2000 to 2400): every load of the launch is issued before the
    // first wait -- one round trip instead of two (the maxima first, then the rows); the sums run in the same order
    v2f_t ml[kUpFront];
    v4f oc[kUpFront];
#pragma unroll
    for (int c = 0; c < kUpFront; ++c) {
      const int64_t slot = slot0 + (int64_t)min(c, (int)ap.chunks - 1) * kAttnRows;
      ml[c] = *(const v2f_t*)(&part_ml[slot * 2]);
      oc[c] = *(const v4f*)(&part_o[slot * kAttnD + d4 * 4]);
    }
#pragma unroll
    for (int c = 0; c < kUpFront; ++c) m = fmaxf(m, ml[c][0]);         // slots past the last chunk repeat it
#pragma unroll
    for (int c = 0; c < kUpFront; ++c) {
      const float w = (c >= ap.chunks || ml[c][0] == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(ml[c][0] - m);
#pragma unroll
      for (int i = 0; i < 4; ++i) num[i] = fmaf(w, oc[c][i], num[i]);
      den = fmaf(w, ml[c][1], den);
    }
  } else {
#pragma unroll 8
    for (int c = 0; c < ap.chunks; ++c) m = fmaxf(m, part_ml[(slot0 + (int64_t)c * kAttnRows) * 2]);
#pragma unroll 8
    for (int c = 0; c < ap.chunks; ++c) {
      const int64_t slot = slot0 + (int64_t)c * kAttnRows;
      const v2f_t ml = *(const v2f_t*)(&part_ml[slot * 2]);
      const v4f oc = *(const v4f*)(&part_o[slot * kAttnD + d4 * 4]);
      const float w = ml[0] == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(ml[0] - m);
#pragma unroll
      for (int i = 0; i < 4; ++i) num[i] = fmaf(w, oc[i], num[i]);
      den = fmaf(w, ml[1], den);
    }
  }
  const float inv = den > 0.f ? 1.f / den : 0.f;
  uint2 packed;
  packed.x = pack2<DT>(num[0] * inv, num[1] * inv);
  packed.y = pack2<DT>(num[2] * inv, num[3] * inv);
  *(uint2*)(out + (((int64_t)b * ap.n_rows + ap.row0 + row) * ap.hq + qh) * kAttnD + d4 * 4) = packed;
}


// ---------------------------------------------------------------------------------------------------------------
// Windows of 17 to 64 query rows: the same algorithm on 32x32x16 matrix instructions.  A wavefront owns 32 rows of one
// head.  S^T = K Q^T is two 32 x 32 accumulators per 64-key block (lane: query row lane % 32, sixteen keys
// 32 t + 8 (r / 4) + 4 (lane / 32) + r % 4), so a row maximum is fifteen in-lane steps and ONE cross-lane step, and
// registers 8 s .. 8 s + 7 of tile t are, packed, the B operand of the 16-key step (t, s) of O^T = V^T P^T.  A
// 32 x 32 x 16 instruction occupies the matrix pipe for 32 cycles but the issue port for about 8 (the 16 x 16 x 32
// form: 16 and 8), which leaves room for the softmax's vector instructions and the LDS operand reads of the other
// wavefront of the SIMD: measured on this chip, one such instruction hides three fused multiply-adds, an exponential
// and a 16-byte LDS read per lane, the 16 x 16 x 32 form only two multiply-adds.
typedef float v16f __attribute__((ext_vector_type(16)));
template <int DT>
__device__ __forceinline__ v16f mfma32x32(uint4 a, uint4 b, v16f c) {
  if constexpr (DT == SUBSPEC_BF16) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, a), __builtin_bit_cast(v8bf, b), c, 0, 0, 0);
  } else {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(v8h, a), __builtin_bit_cast(v8h, b), c, 0, 0, 0);
  }
}
constexpr int kKStride32 = kAttnD + 8;    // 272-byte rows: the 16-byte reads of 16 consecutive keys tile the 64 banks
constexpr int kVStride32 = kAttnD + 32;   // 320-byte rows: a transposing read takes 64 bytes of each of 4 keys per 32 lanes
constexpr int kTileElems = 32 * kAttnD;   // partial O of one 32-row tile, 16-bit, stored [16 (d-tile, quad)][64 lanes][4]

// WPH wavefronts per head (1: up to 32 rows, 2: up to 64), THREADS / 64 / WPH heads of one KV head per workgroup.
template <int DT, bool PAGED, int WPH, int THREADS>
__global__ __launch_bounds__(THREADS) __attribute__((amdgpu_waves_per_eu(2, 2))) void tree_attention32_kernel(
    const uint16_t* __restrict__ q, const uint16_t* __restrict__ kc, const uint16_t* __restrict__ vc,
    const uint64_t* __restrict__ anc, AttnParams ap, uint16_t* __restrict__ out, float* __restrict__ part_o,
    float* __restrict__ part_ml) {
  __shared__ __attribute__((aligned(16))) uint16_t Ks2[2][kKeyBlock * kKStride32];
  __shared__ __attribute__((aligned(16))) uint16_t Vs2[2][kKeyBlock * kVStride32];
  // ancestor bitsets of the window's rows (the heads of a workgroup share them).  Read from LDS inside the loop: a
  // global load there would make the loop wait for EVERY request in flight, the prefetched keys included.
  __shared__ uint64_t mask_s[kAttnRows][SUBSPEC_MAX_TREE_NODES / 64 + 1];
  asm volatile("" ::"s"(ap.batch), "s"(ap.hq), "s"(ap.hkv), "s"(ap.n_rows), "s"(ap.n_slots), "s"(ap.seq_stride), "s"(ap.prefix),
               "s"(ap.anc_batch_stride), "s"(ap.mask_words), "s"(ap.row0), "s"(ap.win_rows), "s"(ap.chunks), "s"(ap.chunk_keys),
               "s"(ap.pairs_per_kv), "s"(ap.units), "s"(ap.scale_log2), "s"(ap.prefix_dev), "s"(ap.page_table),
               "s"(ap.page_shift), "s"(ap.max_pages), "s"(ap.page_stride), "s"(ap.tok_stride), "s"(ap.v_delta));
  asm volatile("" ::"s"(q), "s"(kc), "s"(vc), "s"(anc), "s"(out), "s"(part_o), "s"(part_ml));
  const uint32_t lin = blockIdx.x;
  const int xcd = (int)(lin % (uint32_t)kXcds);
  const uint32_t slot = lin / (uint32_t)kXcds;
  const int pair = (int)(slot % (uint32_t)ap.pairs_per_kv);
  const uint32_t unit = (slot / (uint32_t)ap.pairs_per_kv) * (uint32_t)kXcds + (uint32_t)xcd;
  if ((int64_t)unit >= ap.units) return;
  const int chunk = (int)(unit % (uint32_t)ap.chunks);
  const uint32_t bkv = unit / (uint32_t)ap.chunks;
  const int kvh = (int)(bkv % (uint32_t)ap.hkv), vb = (int)(bkv / (uint32_t)ap.hkv);
  const AttnWindow aw = attn_window(ap, vb);          // (sequence, window of 64 query rows) of this unit
  const int b = aw.b;
  const int group = (int)((uint32_t)ap.hq / (uint32_t)ap.hkv);

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int lr = lane & 31, g = lane >> 5;              // query row of the lane inside its tile, half of the k range
  constexpr int kHeadsPerWG = (THREADS / 64) / WPH;
  const int head_in_group = pair * kHeadsPerWG + wave / WPH;
  const bool head_ok = head_in_group < group;
  const int qh = kvh * group + (head_ok ? head_in_group : 0);
  const int bh = b * (int)ap.hq + qh, vbh = vb * (int)ap.hq + qh;   // q / out rows; partial slots
  const int n = (int)ap.n_rows;
  const int64_t prefix = ap.prefix_dev ? min(max(*ap.prefix_dev, (int64_t)0), ap.prefix) : ap.prefix;
  const int64_t kv_len = prefix + ap.n_slots;
  const int tile = wave % WPH;
  const int row = tile * 32 + lr;                       // row inside this launch's window
  const bool row_ok = head_ok && row < aw.win_rows;
  const int grow = aw.row0 + (row_ok ? row : 0);

  v16f oacc[kAttnD / 32];
#pragma unroll
  for (int dt = 0; dt < kAttnD / 32; ++dt)
#pragma unroll
    for (int r = 0; r < 16; ++r) oacc[dt][r] = 0.f;
  float m_run = -INFINITY, l_run = 0.f;

  const uint16_t* kbase = PAGED ? kc + (int64_t)kvh * kAttnD : kc + ((int64_t)b * ap.hkv + kvh) * ap.seq_stride * kAttnD;
  const uint16_t* vbase = PAGED ? kbase + ap.v_delta : vc + ((int64_t)b * ap.hkv + kvh) * ap.seq_stride * kAttnD;
  auto row_offset = [&](int64_t p) -> int64_t {
    if constexpr (PAGED) {
      const int page = min(max(ap.page_table[p >> ap.page_shift], 0), ap.max_pages - 1);
      return (int64_t)page * ap.page_stride + (p & ((1 << ap.page_shift) - 1)) * ap.tok_stride;
    } else {
      return p * kAttnD;
    }
  };
  const int64_t key0 = (int64_t)chunk * ap.chunk_keys;
  const int64_t key1 = min(key0 + ap.chunk_keys, kv_len);

  constexpr int KPT = 1024 / THREADS;                  // keys of a block per thread: 2 (512 threads), 4 (256), 8 (128)
  constexpr int KSTEP = 64 / KPT;
  // Two register sets: block j travels in set j % 2 and is written to LDS stage j % 2 one block ahead of its use, so the
  // requests of TWO blocks are in flight while a block is multiplied (one block's worth per compute unit does not cover
  // the memory latency).  Native vectors: arrays of HIP's uint4 struct would live in memory.
  dec_u4 kst[2][KPT], vst[2][KPT];
  const int skey = tid >> 4, sdc = tid & 15;
#define SUBSPEC_ATTN32_FETCH(SET, KB)                                                            \
  do {                                                                                           \
    _Pragma("unroll") for (int i_ = 0; i_ < KPT; ++i_) {                                         \
      const int64_t p_ = row_offset(min((KB) + i_ * KSTEP + skey, key1 - 1));                    \
      kst[SET][i_] = *(const dec_u4*)(kbase + p_ + sdc * 8);                                     \
      vst[SET][i_] = *(const dec_u4*)(vbase + p_ + sdc * 8);                                     \
    }                                                                                            \
  } while (0)
#define SUBSPEC_ATTN32_STAGE(SET)                                                                \
  do {                                                                                           \
    _Pragma("unroll") for (int i_ = 0; i_ < KPT; ++i_) {                                         \
      *(dec_u4*)(Ks2[SET] + (skey + i_ * KSTEP) * kKStride32 + sdc * 8) = kst[SET][i_];          \
      *(dec_u4*)(Vs2[SET] + (skey + i_ * KSTEP) * kVStride32 + sdc * 8) = vst[SET][i_];          \
    }                                                                                            \
  } while (0)

  // Every fetch and every stage is unconditional (rows beyond the chunk repeat its last row and are never multiplied):
  // the counter that a wait names is fixed at compile time, and a request that is issued on one path only makes the
  // compiler wait for ALL requests in flight wherever the paths join.
  // The longest transfer first, and nothing waits before everything is on its way: the first two key blocks, the Q rows
  // (B operands: B[k = 8 g + e][row] = Q[row][16 ks + 8 g + e]), the mask words -- the latter only in chunks that reach the tree.
  SUBSPEC_ATTN32_FETCH(0, key0);
  SUBSPEC_ATTN32_FETCH(1, key0 + kKeyBlock);
  uint4 qreg[kAttnD / 16];
  {
    const uint16_t* qp = q + ((int64_t)bh * n + grow) * kAttnD + g * 8;
#pragma unroll
    for (int ks = 0; ks < kAttnD / 16; ++ks) qreg[ks] = row_ok ? *(const uint4*)(qp + ks * 16) : make_uint4(0, 0, 0, 0);
  }
  constexpr int kMaskWords = SUBSPEC_MAX_TREE_NODES / 64 + 1, kMaskPerThread = (kAttnRows * kMaskWords + THREADS - 1) / THREADS;
  uint64_t mword[kMaskPerThread];
  const bool reaches_tree = key1 > prefix;             // (uniform)
#pragma unroll
  for (int u = 0; u < kMaskPerThread; ++u) {
    const int i = tid + u * THREADS, r = i / kMaskWords, w = i % kMaskWords;
    mword[u] = (reaches_tree && i < kAttnRows * kMaskWords && r < aw.win_rows && w < ap.mask_words)
                   ? anc[((int64_t)b * ap.anc_batch_stride + aw.row0 + r) * ap.mask_words + w] : 0ull;
  }
  SUBSPEC_ATTN32_STAGE(0);
  SUBSPEC_ATTN32_FETCH(0, key0 + 2 * kKeyBlock);
  if (reaches_tree) {
#pragma unroll
    for (int u = 0; u < kMaskPerThread; ++u)
      if (tid + u * THREADS < kAttnRows * kMaskWords) (&mask_s[0][0])[tid + u * THREADS] = mword[u];
  }

  // LDS addresses of the lane's operands.  K: key 32 t + lr, pieces of 16 bytes at 16 ks + 8 g.  V^T (transposing read,
  // per 16 lanes: lane r supplies the 8 bytes of key r / 4 at d = 4 (r % 4) and receives four keys of d = r): keys
  // 4 g + r / 4 of the 16-key step, d = 32 dt + 16 (lr / 16) + ...
  const int koff = lr * kKStride32 + g * 8;
  const int voff = (4 * g + ((lane & 15) >> 2)) * kVStride32 + (lr & 16) + 4 * (lane & 3);

  for (int64_t kb2 = key0; kb2 < key1; kb2 += 2 * kKeyBlock) {
#pragma unroll
   for (int buf = 0; buf < 2; ++buf) {
    const int64_t kb = kb2 + buf * kKeyBlock;
    __syncthreads();                                   // stage `buf` is complete, and everyone has left the other stage
    SUBSPEC_ATTN32_STAGE(buf ^ 1);
    SUBSPEC_ATTN32_FETCH(buf ^ 1, kb + 3 * kKeyBlock);
    if (kb >= key1) continue;                          // (uniform) odd number of blocks: the requests above keep every path's count equal
    if (!(head_ok && tile * 32 < aw.win_rows)) continue; // (wave-uniform) a head slot or row tile with nothing in it only helps with the staging
    const uint16_t* Ks = Ks2[buf] + koff;
    const uint16_t* Vs = Vs2[buf] + voff;

    v16f sacc[2];
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int r = 0; r < 16; ++r) sacc[t][r] = 0.f;
#pragma unroll
    for (int ks = 0; ks < kAttnD / 16; ++ks) {
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        const uint4 a = *(const uint4*)(Ks + t * 32 * kKStride32 + ks * 16);
        sacc[t] = mfma32x32<DT>(a, qreg[ks], sacc[t]);
      }
    }
    const bool plain = kb + kKeyBlock <= prefix;
    float mloc = -INFINITY;
    if (plain) {
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int r = 0; r < 16; r += 2) mloc = fmaxf(fmaxf(sacc[t][r], sacc[t][r + 1]), mloc);
    } else {
      // a 64-key block touches at most two consecutive words of the row's bitset (a zero word follows the last)
      const int word0 = min((int)(max(kb - prefix, (int64_t)0) >> 6), SUBSPEC_MAX_TREE_NODES / 64 - 1);
      const uint64_t bits0 = row_ok ? mask_s[row][word0] : 0ull, bits1 = row_ok ? mask_s[row][word0 + 1] : 0ull;
#pragma unroll
      for (int t = 0; t < 2; ++t) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int64_t pos = kb + t * 32 + (r >> 2) * 8 + g * 4 + (r & 3);
          const bool in_range = pos < kv_len;
          const bool tree = pos >= prefix;
          const int rel = tree ? (int)(pos - prefix) : 0;
          const uint64_t word = (rel >> 6) == word0 ? bits0 : bits1;
          const bool ok = in_range && (!tree || ((word >> (rel & 63)) & 1ull));
          const float tv = ok ? sacc[t][r] : -INFINITY;
          sacc[t][r] = tv;
          mloc = fmaxf(mloc, tv);
        }
      }
    }
    mloc = fmaxf(mloc, __shfl_xor(mloc, 32, kWave));
    const float m_new = fmaxf(m_run, mloc);
    const float m_use = m_new == -INFINITY ? 0.f : m_new;
    const float alpha = __builtin_amdgcn_exp2f((m_run - m_use) * ap.scale_log2);
    m_run = m_new;
    const float mneg = -m_use * ap.scale_log2;
    if (__any(alpha != 1.0f)) {
      l_run *= alpha;
#pragma unroll
      for (int dt = 0; dt < kAttnD / 32; ++dt) oacc[dt] *= alpha;
    }
    uint4 pb[2][2];
#pragma unroll
    for (int t = 0; t < 2; ++t) {
#pragma unroll
      for (int s = 0; s < 2; ++s) {
        float p[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          p[e] = __builtin_amdgcn_exp2f(fmaf(sacc[t][8 * s + e], ap.scale_log2, mneg));
          l_run += p[e];
        }
        pb[t][s] = make_uint4(pack2<DT>(p[0], p[1]), pack2<DT>(p[2], p[3]), pack2<DT>(p[4], p[5]), pack2<DT>(p[6], p[7]));
      }
    }
    // O^T += V^T P^T: four 32-wide d tiles, four 16-key steps; the A operand of step (t, s) holds, for the lane's d, the keys
    // 32 t + 16 s + 4 g + {0..3} and 32 t + 16 s + 8 + 4 g + {0..3}, in the order the accumulator registers of S^T hold them
#pragma unroll
    for (int t = 0; t < 2; ++t) {
#pragma unroll
      for (int s = 0; s < 2; ++s) {
#pragma unroll
        for (int dt = 0; dt < kAttnD / 32; ++dt) {
          const uint16_t* vp = Vs + (t * 32 + s * 16) * kVStride32 + dt * 32;
          const uint2 lo = lds_read_tr16(vp), hi = lds_read_tr16(vp + 8 * kVStride32);
          oacc[dt] = mfma32x32<DT>(make_uint4(lo.x, lo.y, hi.x, hi.y), pb[t][s], oacc[dt]);
        }
      }
    }
   }
  }
#undef SUBSPEC_ATTN32_FETCH
#undef SUBSPEC_ATTN32_STAGE

  float l = l_run + __shfl_xor(l_run, 32, kWave);
  if (!head_ok || tile * 32 >= aw.win_rows) return;      // (wave-uniform) nothing of this tile is wanted
  if (ap.chunks == 1) {
    if (!row_ok) return;
    const float inv = l > 0.f ? 1.0f / l : 0.f;
    uint16_t* op = out + (((int64_t)b * n + aw.row0 + row) * ap.hq + qh) * kAttnD + g * 4;
#pragma unroll
    for (int dt = 0; dt < kAttnD / 32; ++dt)
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4)
        *(uint2*)(op + dt * 32 + q4 * 8) = make_uint2(pack2<DT>(oacc[dt][4 * q4] * inv, oacc[dt][4 * q4 + 1] * inv),
                                                      pack2<DT>(oacc[dt][4 * q4 + 2] * inv, oacc[dt][4 * q4 + 3] * inv));
  } else {
    // the chunk's own softmax-weighted average of V, in the 16-bit dtype (a convex combination of such averages is what the
    // merge forms, so their rounding error does not grow); every store instruction writes 512 consecutive bytes
    const float inv = l > 0.f ? 1.0f / l : 0.f;
    uint16_t* po = (uint16_t*)part_o + (((int64_t)vbh * ap.chunks + chunk) * 2 + tile) * kTileElems + lane * 4;
#pragma unroll
    for (int dt = 0; dt < kAttnD / 32; ++dt)
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4)
        *(uint2*)(po + (dt * 4 + q4) * 256) = make_uint2(pack2<DT>(oacc[dt][4 * q4] * inv, oacc[dt][4 * q4 + 1] * inv),
                                                         pack2<DT>(oacc[dt][4 * q4 + 2] * inv, oacc[dt][4 * q4 + 3] * inv));
    if (g == 0) {
      const int64_t pslot = ((int64_t)vbh * ap.chunks + chunk) * kAttnRows + row;
      *(v2f_t*)(part_ml + pslot * 2) = v2f_t{m_run * ap.scale_log2, l};
    }
  }
}

// ---------------------------------------------------------------------------------------------------------------
// The same tiles with the two wavefronts of every SIMD half a block apart ("ping-pong").  Left to themselves the eight
// wavefronts of a workgroup run in step (they start together and meet at a barrier per block): all of them multiply,
// then all of them evaluate the softmax, and the matrix pipe idles while the vector ALU works and the other way round
// -- measured: 1.76 us per 64-key block and workgroup for 1.0 us of matrix work, vector and matrix time simply added.
// Here a block is two phases separated by workgroup barriers, M (O^T += V^T P^T of the previous block, then S^T = K Q^T
// of this one: matrix instructions and their LDS operand reads) and V (softmax of S^T: vector ALU only); wavefronts
// 4..7 (group B, the second wavefront of each SIMD) enter the loop one barrier later than wavefronts 0..3 (group A), so
// whenever one wavefront of a SIMD is in M the other is in V.
// K / V blocks travel from memory straight into LDS (global_load_lds_dwordx4: no staging registers, no LDS write
// instructions) through a ring of four stages; a wavefront issues its share of block i + 2 inside the M phase of block i.  The copies are
// inline assembly ON PURPOSE: a wait names a count fixed at compile time, and for LDS-DMA requests it knows about the
// compiler waits for all of them before every LDS read; the waits for these are placed by hand (group A at the end of
// V, group B at the end of M: every odd global phase).  A stage's rows are unpadded (a DMA instruction writes 1 KB of
// consecutive LDS, four rows); the 16-byte pieces of a row are XOR-swizzled instead, by choosing which piece of the
// row each lane fetches: K piece p of row r sits at p ^ (r % 16) (the operand read of 16 consecutive rows then covers
// all 64 banks), V piece p at p ^ 4 (r % 4) (the transposing read takes 64 bytes of each of 4 consecutive rows).
constexpr int kPPStages = 4;
constexpr int kPPStageBytes = kKeyBlock * kAttnD * 2;                 // 16 KB
constexpr int kPPVOff = kPPStages * kPPStageBytes;                    // V ring behind the K ring
constexpr int kPPMaskOff = 2 * kPPStages * kPPStageBytes;             // 128 KB
constexpr int kPPMaskWords = SUBSPEC_MAX_TREE_NODES / 64 + 1;         // a zero word follows the last
constexpr int kPPLdsBytes = kPPMaskOff + kAttnRows * kPPMaskWords * 8;

__device__ __forceinline__ void pp_wait_vmcnt4() { asm volatile("s_waitcnt vmcnt(4)" ::: "memory"); }
__device__ __forceinline__ void pp_dma16(uint32_t lds_base, const uint16_t* src) {
  asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(lds_base), "v"(src) : "memory", "m0");
}

// The matrix work of an M phase as steps of one matrix instruction each.  MODE 2 (the steady state) alternates the two
// products: even steps are O^T += V^T P^T of the previous block ((t, s) major, the four d tiles minor), odd steps
// S^T = K Q^T of this one (d step major, the two key tiles minor), so an accumulator comes up again only every fourth
// (S^T) or eighth (O^T) step -- two S^T accumulators used alternately wait for each other (measured: 43 cycles per
// instruction instead of 33).  MODE 0 is S^T alone (the first block), MODE 1 O^T alone (after the last).  The LDS operand of
// step k + kAhead is requested right after the instruction of step k has been issued, through a ring of operand registers;
// scheduling fences keep the compiler from undoing the distance (left alone it requests every operand immediately before
// its use and waits for it, with the matrix pipe idle meanwhile).  With `copy`, the wavefront's four K / V copy instructions
// of the block two ahead are issued a quarter of the steps apart instead of in a row: a copy instruction waits for room in the
// compute unit's memory pipeline, and that wait then falls into the shadow of a matrix instruction.
// A wavefront on its own issues an instruction every five to six cycles, so the phase is as much a count of instructions
// as of matrix cycles: the twelve operand addresses (8 d steps of K, 4 d tiles of V^T; the XOR swizzle keeps them from
// being immediates) are formed once per phase, the key offsets are immediates.
// The S^T accumulators do not start at zero but at -ref, the row's reference score (PPRef below), so the softmax does not
// subtract.  (Q scaled by scale * log2(e) beforehand would save the multiplication as well, but rounds Q a second time:
// 3 % error in the probabilities of rows whose scores reach the hundreds.  Not done.)
struct PPAddr { uint32_t vst, kst, vx, kx; };
// a wavefront's four copy instructions of one block: K rows 0..3, K rows 4..7, V rows 0..3, V rows 4..7 of its share
struct PPCopy {
  const uint16_t *k0, *k1, *v0, *v1;     // lane addresses less the row offsets
  int r0, r1;                            // element offsets of the two row groups inside the chunk
  uint32_t kdst, vdst;                   // LDS addresses of the wavefront's rows in the stage
};
__device__ __forceinline__ void pp_copy_issue(const PPCopy& cp, int c) {
  if (c == 0) pp_dma16(cp.kdst, cp.k0 + cp.r0);
  else if (c == 1) pp_dma16(cp.kdst + 1024, cp.k1 + cp.r1);
  else if (c == 2) pp_dma16(cp.vdst, cp.v0 + cp.r0);
  else pp_dma16(cp.vdst + 1024, cp.v1 + cp.r1);
}
template <int MODE> __device__ __forceinline__ constexpr bool pp_step_is_pv(int k) { return MODE == 1 || (MODE == 2 && (k & 1) == 0); }
template <int MODE> __device__ __forceinline__ constexpr int pp_step_index(int k) { return MODE == 2 ? k >> 1 : k; }
template <int DT, int MODE>
__device__ __forceinline__ dec_u4 pp_load_step(int k, const uint32_t (&kaddr)[8], const uint32_t (&vaddr)[4]) {
  const int j = pp_step_index<MODE>(k);
  if (pp_step_is_pv<MODE>(k)) {
    const int ts = j >> 2, dt = j & 3;                   // ts = 2 t + s: keys 16 ts .. 16 ts + 15 of the block
    const uint32_t va = vaddr[dt] + (uint32_t)(ts * 16 * 256);
    const uint2 lo = lds_read_tr16((const uint16_t*)(__attribute__((address_space(3))) uint16_t*)(uintptr_t)va);
    const uint2 hi = lds_read_tr16((const uint16_t*)(__attribute__((address_space(3))) uint16_t*)(uintptr_t)(va + 8 * 256));
    return dec_u4{lo.x, lo.y, hi.x, hi.y};
  } else {
    const int ks = j >> 1, t = j & 1;
    const uint32_t ka = kaddr[ks] + (uint32_t)(t * 32 * 256);
    return *(const dec_u4*)(__attribute__((address_space(3))) dec_u4*)(uintptr_t)ka;
  }
}
template <int DT, int MODE>
__device__ __forceinline__ void pp_matrix_phase(const PPAddr& ad, const PPCopy& cp, bool copy, v16f (&oacc)[4], v16f (&sacc)[2],
                                                const v16f& cinit, const uint4 (&pb)[2][2], const uint4 (&qreg)[8]) {
  constexpr int kSteps = MODE == 2 ? 32 : 16;
  constexpr int kAhead = 4;
  // the wavefront that multiplies goes first: between two wavefronts of a SIMD the older one wins every issue slot, and
  // without this group B's matrix phases take a third longer than group A's
  __builtin_amdgcn_s_setprio(1);
  uint32_t kaddr[8], vaddr[4];
  if (MODE != 1) {
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) kaddr[ks] = ad.kst + (ad.kx ^ (uint32_t)(ks << 5));
  }
  if (MODE != 0) {
#pragma unroll
    for (int dt = 0; dt < 4; ++dt) vaddr[dt] = ad.vst + (ad.vx ^ (uint32_t)(dt << 6));
  }
  dec_u4 ring[kAhead];
#pragma unroll
  for (int k = 0; k < kAhead; ++k) ring[k] = pp_load_step<DT, MODE>(k, kaddr, vaddr);
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int k = 0; k < kSteps; ++k) {
    const uint4 a = __builtin_bit_cast(uint4, ring[k % kAhead]);
    const int j = pp_step_index<MODE>(k);
    if (pp_step_is_pv<MODE>(k)) {
      const int ts = j >> 2, dt = j & 3;
      oacc[dt] = mfma32x32<DT>(a, pb[ts >> 1][ts & 1], oacc[dt]);
    } else {
      const int ks = j >> 1, t = j & 1;
      sacc[t] = mfma32x32<DT>(a, qreg[ks], ks == 0 ? cinit : sacc[t]);
    }
    __builtin_amdgcn_sched_barrier(0);
    if (k + kAhead < kSteps) ring[k % kAhead] = pp_load_step<DT, MODE>(k + kAhead, kaddr, vaddr);
    if (k % (kSteps / 4) == 1 && copy) pp_copy_issue(cp, k / (kSteps / 4));       // (uniform)
    __builtin_amdgcn_sched_barrier(0);
  }
  __builtin_amdgcn_s_setprio(0);
}

// Online-softmax step of one 64-key block on the S^T accumulators (vector ALU only).  The accumulators hold raw scores
// relative to the row's REFERENCE score `ref`, which is not the running maximum but something within kPPSlack (in exp2
// units) of it from below: the first block that shows the row a key sets it to that block's maximum, a later block moves it only when its
// maximum exceeds it by more than kPPSlack (then O, the running sum and this block's arguments are rescaled -- rare once
// the first blocks are through).  Probabilities are therefore at most 2^kPPSlack instead of at most 1, which costs neither
// range nor precision in bf16 / fp16 x fp32, and the common case is 16 three-way maxima, 32 exponentials, 16 packed
// conversions and 16 two-element dot products against ones for the row sum, besides the 32 multiplications by the scale.
constexpr float kPPSlack = 8.0f;
struct PPRow { int64_t prefix, kv_len; const uint64_t* mask_row; float scale_log2; int g; bool row_ok; };
struct PPRef { float ref, l; bool have; };
template <int DT>
__device__ __forceinline__ float pp_pair_sum(uint32_t packed, float acc) {
  if constexpr (DT == SUBSPEC_BF16) return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(v2bf_t, packed), __builtin_bit_cast(v2bf_t, 0x3f803f80u), acc, false);
  else return __builtin_amdgcn_fdot2(__builtin_bit_cast(v2h_t, packed), __builtin_bit_cast(v2h_t, 0x3c003c00u), acc, false);
}
__device__ __forceinline__ float pp_max_halves(float x) {          // maximum of lanes i and i ^ 32, in both
  const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
template <int DT>
__device__ __forceinline__ void pp_softmax_phase(int64_t kb, const PPRow& rw, v16f (&sacc)[2], v16f (&oacc)[4], v16f& cinit,
                                                 uint4 (&pb)[2][2], PPRef& rf) {
  const bool plain = kb + kKeyBlock <= rw.prefix;
  if (!plain) {
    // a 64-key block touches at most two consecutive words of the row's bitset (a zero word follows the last)
    const int word0 = min((int)(max(kb - rw.prefix, (int64_t)0) >> 6), SUBSPEC_MAX_TREE_NODES / 64 - 1);
    const uint64_t bits0 = rw.row_ok ? rw.mask_row[word0] : 0ull, bits1 = rw.row_ok ? rw.mask_row[word0 + 1] : 0ull;
#pragma unroll
    for (int t = 0; t < 2; ++t) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int64_t pos = kb + t * 32 + (r >> 2) * 8 + rw.g * 4 + (r & 3);
        const bool in_range = pos < rw.kv_len;
        const bool tree = pos >= rw.prefix;
        const int rel = tree ? (int)(pos - rw.prefix) : 0;
        const uint64_t word = (rel >> 6) == word0 ? bits0 : bits1;
        const bool ok = in_range && (!tree || ((word >> (rel & 63)) & 1ull));
        sacc[t][r] = ok ? sacc[t][r] : -INFINITY;
      }
    }
  }
  float mt[2] = {-INFINITY, -INFINITY};
#pragma unroll
  for (int t = 0; t < 2; ++t)
#pragma unroll
    for (int r = 0; r < 16; r += 2) mt[t] = fmaxf(fmaxf(sacc[t][r], sacc[t][r + 1]), mt[t]);
  const float mloc = pp_max_halves(fmaxf(mt[0], mt[1]));           // raw score units, relative to ref
  const bool move = mloc > -INFINITY && (!rf.have || mloc * rw.scale_log2 > kPPSlack);
  if (__any(move)) {
    const float d = move ? mloc : 0.f;                              // the row's reference goes up (first time: anywhere) by d
    const float alpha = __builtin_amdgcn_exp2f(-d * rw.scale_log2);
    rf.ref += d;
    rf.l *= alpha;
#pragma unroll
    for (int dt = 0; dt < kAttnD / 32; ++dt) oacc[dt] *= alpha;
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int r = 0; r < 16; ++r) sacc[t][r] -= d;
#pragma unroll
    for (int r = 0; r < 16; ++r) cinit[r] = -rf.ref;
  }
  rf.have = rf.have || mloc > -INFINITY;
  float lsum[2][2];
#pragma unroll
  for (int t = 0; t < 2; ++t) {
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      float p[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) p[e] = __builtin_amdgcn_exp2f(sacc[t][8 * s + e] * rw.scale_log2);
      pb[t][s] = make_uint4(pack2<DT>(p[0], p[1]), pack2<DT>(p[2], p[3]), pack2<DT>(p[4], p[5]), pack2<DT>(p[6], p[7]));
      lsum[t][s] = pp_pair_sum<DT>(pb[t][s].w, pp_pair_sum<DT>(pb[t][s].z, pp_pair_sum<DT>(pb[t][s].y, pp_pair_sum<DT>(pb[t][s].x, 0.f))));
    }
  }
  rf.l += (lsum[0][0] + lsum[0][1]) + (lsum[1][0] + lsum[1][1]);
}

template <int DT, int WPH>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2))) void tree_attention_pp_kernel(
    const uint16_t* __restrict__ q, const uint16_t* __restrict__ kc, const uint16_t* __restrict__ vc,
    const uint64_t* __restrict__ anc, AttnParams ap, uint16_t* __restrict__ out, float* __restrict__ part_o,
    float* __restrict__ part_ml) {
  __shared__ __attribute__((aligned(1024))) uint8_t lds[kPPLdsBytes];
  asm volatile("" ::"s"(ap.batch), "s"(ap.hq), "s"(ap.hkv), "s"(ap.n_rows), "s"(ap.n_slots), "s"(ap.seq_stride), "s"(ap.prefix),
               "s"(ap.anc_batch_stride), "s"(ap.mask_words), "s"(ap.row0), "s"(ap.win_rows), "s"(ap.chunks), "s"(ap.chunk_keys),
               "s"(ap.pairs_per_kv), "s"(ap.units), "s"(ap.scale_log2), "s"(ap.prefix_dev));
  asm volatile("" ::"s"(q), "s"(kc), "s"(vc), "s"(anc), "s"(out), "s"(part_o), "s"(part_ml));
  const uint32_t lin = blockIdx.x;
  const int xcd = (int)(lin % (uint32_t)kXcds);
  const uint32_t slot = lin / (uint32_t)kXcds;
  const int pair = (int)(slot % (uint32_t)ap.pairs_per_kv);
  const uint32_t unit = (slot / (uint32_t)ap.pairs_per_kv) * (uint32_t)kXcds + (uint32_t)xcd;
  if ((int64_t)unit >= ap.units) return;
  const int chunk = (int)(unit % (uint32_t)ap.chunks);
  const uint32_t bkv = unit / (uint32_t)ap.chunks;
  const int kvh = (int)(bkv % (uint32_t)ap.hkv), vb = (int)(bkv / (uint32_t)ap.hkv);
  const AttnWindow aw = attn_window(ap, vb);          // (sequence, window of 64 query rows) of this unit
  const int b = aw.b;
  const int group = (int)((uint32_t)ap.hq / (uint32_t)ap.hkv);

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lr = lane & 31, g = lane >> 5;
  constexpr int kHeadsPerWG = 8 / WPH;
  const int head_in_group = pair * kHeadsPerWG + wave / WPH;
  const bool head_ok = head_in_group < group;
  const int qh = kvh * group + (head_ok ? head_in_group : 0);
  const int bh = b * (int)ap.hq + qh, vbh = vb * (int)ap.hq + qh;   // q / out rows; partial slots
  const int n = (int)ap.n_rows;
  const int64_t prefix = ap.prefix_dev ? min(max(*ap.prefix_dev, (int64_t)0), ap.prefix) : ap.prefix;
  const int64_t kv_len = prefix + ap.n_slots;
  const int tile = wave % WPH;
  const int row = tile * 32 + lr;
  const bool live = head_ok && tile * 32 < aw.win_rows;     // (wave-uniform) this wavefront has rows to work on
  const bool row_ok = head_ok && row < aw.win_rows;
  const int grow = aw.row0 + (row_ok ? row : 0);
  const bool grp_b = wave >= 4;                             // the second wavefront of each SIMD (wavefront w runs on SIMD w % 4)

  const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)lds;
  const int64_t key0 = (int64_t)chunk * ap.chunk_keys;
  const int64_t key1 = min(key0 + ap.chunk_keys, kv_len);
  const int nkeys = (int)(key1 - key0);
  const int nb = (nkeys + kKeyBlock - 1) / kKeyBlock;
  const uint16_t* kbase = kc + (((int64_t)b * ap.hkv + kvh) * ap.seq_stride + key0) * kAttnD;
  const uint16_t* vbase = vc + (((int64_t)b * ap.hkv + kvh) * ap.seq_stride + key0) * kAttnD;

  // ---- copies: wavefront w brings rows 8 w .. 8 w + 7 of a block, K and V, two instructions of four rows each
  const int crow = wave * 8 + (lane >> 4);                                       // row of the first instruction; + 4 for the second
  const int kpiece0 = ((lane & 15) ^ (crow & 15)) * 8, kpiece1 = ((lane & 15) ^ ((crow + 4) & 15)) * 8;
  const int vpiece = ((lane & 15) ^ (4 * (crow & 3))) * 8;                       // (crow + 4) % 4 == crow % 4
  const uint32_t kdst = lds0 + wave * 2048, vdst = lds0 + kPPVOff + wave * 2048;
  PPCopy cp;
  cp.k0 = kbase + kpiece0; cp.k1 = kbase + kpiece1; cp.v0 = vbase + vpiece; cp.v1 = cp.v0;
  // block J of the chunk -> stage J % 4 (rows past the chunk repeat its last row)
#define SUBSPEC_PP_PLAN(J)                                                                     \
  do {                                                                                         \
    cp.r0 = min((J) * kKeyBlock + crow, nkeys - 1) * kAttnD;                                   \
    cp.r1 = min((J) * kKeyBlock + crow + 4, nkeys - 1) * kAttnD;                               \
    const uint32_t st_ = (uint32_t)((J) & (kPPStages - 1)) * kPPStageBytes;                    \
    cp.kdst = kdst + st_; cp.vdst = vdst + st_;                                                \
  } while (0)
#define SUBSPEC_PP_ISSUE(J)                                                                    \
  do {                                                                                         \
    SUBSPEC_PP_PLAN(J);                                                                        \
    pp_copy_issue(cp, 0); pp_copy_issue(cp, 1); pp_copy_issue(cp, 2); pp_copy_issue(cp, 3);    \
  } while (0)
  SUBSPEC_PP_ISSUE(0);
  SUBSPEC_PP_ISSUE(1);
  // ---- everything else that has to come out of memory before the first product, requested behind the first two K / V blocks
  //      (the longest transfer first); one wait covers all of it
  uint4 qreg[kAttnD / 16];
  {
    const uint16_t* qp = q + ((int64_t)bh * n + grow) * kAttnD + g * 8;
#pragma unroll
    for (int ks = 0; ks < kAttnD / 16; ++ks) qreg[ks] = row_ok ? *(const uint4*)(qp + ks * 16) : make_uint4(0, 0, 0, 0);
  }
  uint64_t* mask_s = (uint64_t*)(lds + kPPMaskOff);
  uint64_t mword[2];
#pragma unroll
  for (int u = 0; u < 2; ++u) {
    const int i = tid + u * 512, r = i / kPPMaskWords, w = i % kPPMaskWords;
    mword[u] = (i < kAttnRows * kPPMaskWords && r < aw.win_rows && w < ap.mask_words)
                   ? anc[((int64_t)b * ap.anc_batch_stride + aw.row0 + r) * ap.mask_words + w] : 0ull;
  }


  v16f oacc[kAttnD / 32], sacc[2];
#pragma unroll
  for (int dt = 0; dt < kAttnD / 32; ++dt)
#pragma unroll
    for (int r = 0; r < 16; ++r) oacc[dt][r] = 0.f;
#pragma unroll
  for (int t = 0; t < 2; ++t)
#pragma unroll
    for (int r = 0; r < 16; ++r) sacc[t][r] = 0.f;
  uint4 pb[2][2] = {};
  v16f cinit;                                          // -ref in every register: what an S^T accumulator starts from
#pragma unroll
  for (int r = 0; r < 16; ++r) cinit[r] = 0.f;
  PPRef rf{0.f, 0.f, false};

  // operand addresses inside a stage (bytes).  K: key 32 t + lr, logical piece 2 ks + g.  V^T: the lane of a 16-lane group
  // with index r supplies the 8 bytes of key 4 g + r / 4 (of the 16-key step's half) at d = 32 dt + 16 h + 4 (r % 4).
  const int r16 = lane & 15, hh = (lane >> 4) & 1;
  const uint32_t klane = lds0 + lr * 256;
  const uint32_t vlane = lds0 + kPPVOff + (4 * g + (r16 >> 2)) * 256 + (2 * hh + ((r16 & 3) >> 1)) * 16 + (r16 & 1) * 8;
  PPAddr ad;
  ad.kx = (uint32_t)((g ^ (lr & 15)) << 4);
  ad.vx = (uint32_t)((r16 >> 2) << 6);
  PPRow rw{prefix, kv_len, mask_s + row * kPPMaskWords, ap.scale_log2, g, row_ok};
#define SUBSPEC_PP_STAGES(I)                                                                   \
  ad.vst = vlane + (uint32_t)(((I) - 1) & (kPPStages - 1)) * kPPStageBytes;                     \
  ad.kst = klane + (uint32_t)((I) & (kPPStages - 1)) * kPPStageBytes

  __builtin_amdgcn_s_waitcnt(0x0F70);                // the Q rows and mask words (and with them blocks 0 and 1)
#pragma unroll
  for (int u = 0; u < 2; ++u)
    if (tid + u * 512 < kAttnRows * kPPMaskWords) mask_s[tid + u * 512] = mword[u];
  __syncthreads();
  if (grp_b) __syncthreads();
  // ---- block 0: M is S^T only
  SUBSPEC_PP_PLAN(2);
  if (live) {
    SUBSPEC_PP_STAGES(0);
    pp_matrix_phase<DT, 0>(ad, cp, true, oacc, sacc, cinit, pb, qreg);
  } else {
    pp_copy_issue(cp, 0); pp_copy_issue(cp, 1); pp_copy_issue(cp, 2); pp_copy_issue(cp, 3);
  }
  if (grp_b) pp_wait_vmcnt4();
  __syncthreads();
  if (live) pp_softmax_phase<DT>(key0, rw, sacc, oacc, cinit, pb, rf);
  if (!grp_b) pp_wait_vmcnt4();
  __syncthreads();
  for (int i = 1; i < nb; ++i) {
    SUBSPEC_PP_PLAN(i + 2);
    if (live) {
      SUBSPEC_PP_STAGES(i);
      pp_matrix_phase<DT, 2>(ad, cp, true, oacc, sacc, cinit, pb, qreg);
    } else {
      pp_copy_issue(cp, 0); pp_copy_issue(cp, 1); pp_copy_issue(cp, 2); pp_copy_issue(cp, 3);
    }
    if (grp_b) pp_wait_vmcnt4();
    __syncthreads();
    if (live) pp_softmax_phase<DT>(key0 + (int64_t)i * kKeyBlock, rw, sacc, oacc, cinit, pb, rf);
    if (!grp_b) pp_wait_vmcnt4();
    __syncthreads();
  }
  // ---- after the last block: M is O^T += V^T P^T only
  if (live) {
    SUBSPEC_PP_STAGES(nb);
    pp_matrix_phase<DT, 1>(ad, cp, false, oacc, sacc, cinit, pb, qreg);
  }
  __syncthreads();
  if (!grp_b) __syncthreads();
#undef SUBSPEC_PP_STAGES
#undef SUBSPEC_PP_PLAN
#undef SUBSPEC_PP_ISSUE
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");     // no copy may still be on its way into LDS when the workgroup ends

  const float l = rf.l + __shfl_xor(rf.l, 32, kWave);
  if (!live) return;
  if (ap.chunks == 1) {
    if (!row_ok) return;
    const float inv = l > 0.f ? 1.0f / l : 0.f;
    uint16_t* op = out + (((int64_t)b * n + aw.row0 + row) * ap.hq + qh) * kAttnD + g * 4;
#pragma unroll
    for (int dt = 0; dt < kAttnD / 32; ++dt)
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4)
        *(uint2*)(op + dt * 32 + q4 * 8) = make_uint2(pack2<DT>(oacc[dt][4 * q4] * inv, oacc[dt][4 * q4 + 1] * inv),
                                                      pack2<DT>(oacc[dt][4 * q4 + 2] * inv, oacc[dt][4 * q4 + 3] * inv));
  } else {
    // the chunk's own softmax-weighted average of V, in the 16-bit dtype (a convex combination of such averages is what the
    // merge forms, so their rounding error does not grow); every store instruction writes 512 consecutive bytes
    const float inv = l > 0.f ? 1.0f / l : 0.f;
    uint16_t* po = (uint16_t*)part_o + (((int64_t)vbh * ap.chunks + chunk) * 2 + tile) * kTileElems + lane * 4;
#pragma unroll
    for (int dt = 0; dt < kAttnD / 32; ++dt)
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4)
        *(uint2*)(po + (dt * 4 + q4) * 256) = make_uint2(pack2<DT>(oacc[dt][4 * q4] * inv, oacc[dt][4 * q4 + 1] * inv),
                                                         pack2<DT>(oacc[dt][4 * q4 + 2] * inv, oacc[dt][4 * q4 + 3] * inv));
    if (g == 0) {
      const int64_t pslot = ((int64_t)vbh * ap.chunks + chunk) * kAttnRows + row;
      *(v2f_t*)(part_ml + pslot * 2) = v2f_t{rf.have ? rf.ref * ap.scale_log2 : -INFINITY, l};
    }
  }
}

// Merge for the tile layout above: one thread per four consecutive head dims of a row; blockIdx.x = (b, head, tile),
// blockIdx.y = quarter of the tile's sixteen register quads.  A chunk's tile is its normalised output, its weight
// exp2(ref_c - max ref) * sum_c.
// With up to eight chunks (CMAX = 4 or 8, the compiled bound) every load of a thread -- the reference and sum of its row
// and its four elements, of every chunk -- is issued before the first is used, so the launch pays ONE round trip to
// memory instead of one for the maximum and one for the sums (config 3, B = 8: 6.1 -> 5.3 us); CMAX = 0 is the two-pass
// form for more chunks, where that many loads up front cost more than they save.
template <int DT, int CMAX>
__global__ __launch_bounds__(256) void tree_attention32_merge_kernel(
    const float* __restrict__ part_o, const float* __restrict__ part_ml, AttnParams ap, uint16_t* __restrict__ out) {
  const int tile = blockIdx.x & 1, vbh = blockIdx.x >> 1;
  const int lane = threadIdx.x & 63, idx16 = blockIdx.y * 4 + (threadIdx.x >> 6);
  const int row = tile * 32 + (lane & 31), g = lane >> 5;
  const int vb = vbh / (int)ap.hq, qh = vbh % (int)ap.hq;
  const AttnWindow aw = attn_window(ap, vb);
  const int b = aw.b;
  if (row >= aw.win_rows) return;
  const int64_t slot0 = (int64_t)vbh * ap.chunks * kAttnRows + row;
  const uint16_t* po = (const uint16_t*)part_o + ((int64_t)vbh * ap.chunks * 2 + tile) * kTileElems + (idx16 * 64 + lane) * 4;
  auto unpack4 = [](uint2 o, float* f) {
    if constexpr (DT == SUBSPEC_BF16) {
      f[0] = bf16_bits_to_float(o.x & 0xffffu); f[1] = bf16_bits_to_float(o.x >> 16);
      f[2] = bf16_bits_to_float(o.y & 0xffffu); f[3] = bf16_bits_to_float(o.y >> 16);
    } else {
      f[0] = f16_bits_to_float(o.x & 0xffffu); f[1] = f16_bits_to_float(o.x >> 16);
      f[2] = f16_bits_to_float(o.y & 0xffffu); f[3] = f16_bits_to_float(o.y >> 16);
    }
  };
  float m = -INFINITY, den = 0.f;
  float num[4] = {0.f, 0.f, 0.f, 0.f};
  if constexpr (CMAX > 0) {
    v2f_t ml[CMAX];
    uint2 oc[CMAX];
#pragma unroll
    for (int c = 0; c < CMAX; ++c) {
      const int cc = min(c, ap.chunks - 1);              // chunks past the count repeat the last one and get no weight
      ml[c] = *(const v2f_t*)(&part_ml[(slot0 + (int64_t)cc * kAttnRows) * 2]);
      oc[c] = *(const uint2*)(po + (int64_t)cc * 2 * kTileElems);
    }
#pragma unroll
    for (int c = 0; c < CMAX; ++c) m = fmaxf(m, ml[c][0]);
#pragma unroll
    for (int c = 0; c < CMAX; ++c) {
      // the chunk's share of the row sum
      const float w = (c >= ap.chunks || ml[c][0] == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(ml[c][0] - m) * ml[c][1];
      float f[4];
      unpack4(oc[c], f);
#pragma unroll
      for (int i = 0; i < 4; ++i) num[i] = fmaf(w, f[i], num[i]);
      den += w;
    }
  } else {
    // many chunks (one sequence cut into a dozen or more): two passes, eight chunks' requests in flight in each
#pragma unroll 8
    for (int c = 0; c < ap.chunks; ++c) m = fmaxf(m, part_ml[(slot0 + (int64_t)c * kAttnRows) * 2]);
#pragma unroll 8
    for (int c = 0; c < ap.chunks; ++c) {
      const v2f_t ml = *(const v2f_t*)(&part_ml[(slot0 + (int64_t)c * kAttnRows) * 2]);
      const uint2 o = *(const uint2*)(po + (int64_t)c * 2 * kTileElems);
      const float w = ml[0] == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(ml[0] - m) * ml[1];
      float f[4];
      unpack4(o, f);
#pragma unroll
      for (int i = 0; i < 4; ++i) num[i] = fmaf(w, f[i], num[i]);
      den += w;
    }
  }
  const float inv = den > 0.f ? 1.f / den : 0.f;
  const int d0 = (idx16 >> 2) * 32 + (idx16 & 3) * 8 + g * 4;
  *(uint2*)(out + (((int64_t)b * ap.n_rows + aw.row0 + row) * ap.hq + qh) * kAttnD + d0) =
      make_uint2(pack2<DT>(num[0] * inv, num[1] * inv), pack2<DT>(num[2] * inv, num[3] * inv));
}

// Launch shape of one window of query rows.
struct AttnPlan { int threads, rowt, wph, heads_per_wg, chunks; bool mfma32, pingpong; };
static AttnPlan attn_plan(int64_t batch, int64_t hq, int64_t hkv, int64_t win_rows, int64_t kv_len, bool one_sequence) {
  AttnPlan pl;
  const int group = (int)(hq / hkv);
  const int64_t blocks = (kv_len + kKeyBlock - 1) / kKeyBlock;
  pl.mfma32 = win_rows > 16;
  // the ping-pong kernel pays for its set-up over many blocks: (sequence, head) pairs enough to fill the chip with few key
  // chunks.  One sequence never takes it, so that a request's attention over pages equals the contiguous one bit for bit.
  pl.pingpong = pl.mfma32 && !one_sequence && batch * hq >= 128;
  if (win_rows <= 16) {
    // a draft level: a wavefront is a whole head (one 16-row tile), eight heads share the staged keys
    pl.threads = 512; pl.rowt = 1; pl.wph = 1;
  } else if (win_rows <= 32) {
    // one 32-row tile per head, eight heads share the staged keys
    pl.threads = 512; pl.rowt = 2; pl.wph = 1;
  } else if (batch * hq >= 128) {
    // 33 to 64 rows, many (sequence, head) pairs: four heads share the staged keys (two wavefronts of 32 rows per head)
    pl.threads = 512; pl.rowt = 2; pl.wph = 2;
  } else {
    // 33 to 64 rows, few sequences: two heads per 256-thread workgroup, so that the workgroups come from the heads
    // and not from key chunks whose partial results would outweigh the keys
    pl.threads = 256; pl.rowt = 2; pl.wph = 2;
  }
  pl.heads_per_wg = (pl.threads / 64) / pl.wph;
  const int64_t wgs_per_chunk = batch * hkv * ((group + pl.heads_per_wg - 1) / pl.heads_per_wg);
  // enough workgroups to cover the chip once (twice with the small workgroups, two of which share a compute unit),
  // at least two key blocks per chunk ...
  const int64_t target_wgs = pl.threads == 256 ? 512 : 256;
  int64_t chunks = std::max<int64_t>(1, (target_wgs + wgs_per_chunk - 1) / wgs_per_chunk);
  if (win_rows <= 32) chunks = std::max<int64_t>(chunks, 1024 / std::max<int64_t>(1, batch * hq));   // few rows: short chunks, latency first
  chunks = std::min<int64_t>(chunks, std::max<int64_t>(1, blocks / 2));
  // ... and the partial results (fp32 rows x 128 per head and chunk) are priced against the K / V bytes (16-bit,
  // 2 x kv_len x 128 per KV head): at most twice as many
  const int64_t by_bytes = std::max<int64_t>(1, 2 * (kv_len * hkv) / std::max<int64_t>(1, hq * win_rows));
  chunks = std::min<int64_t>(chunks, by_bytes);
  pl.chunks = (int)std::min<int64_t>(chunks, 64);
  return pl;
}
// One call = one launch (pair): up to 64 query rows are one window; more rows are ceil(n_rows / 64) windows laid out as
// further batch entries (attn_window), planned like that many sequences of 64 rows.
struct AttnLaunch { int windows, win_rows; int64_t vbatch; AttnPlan pl; };
static AttnLaunch attn_launch(int64_t batch, int64_t hq, int64_t hkv, int64_t n_rows, int64_t kv_len) {
  AttnLaunch al;
  al.windows = (int)((n_rows + kAttnRows - 1) / kAttnRows);
  al.win_rows = (int)std::min<int64_t>(n_rows, kAttnRows);
  al.vbatch = batch * al.windows;
  al.pl = attn_plan(al.vbatch, hq, hkv, al.win_rows, kv_len, batch == 1);
  return al;
}

}  // namespace subspec

using namespace subspec;

static size_t attn_partial_bytes(int64_t batch, int64_t hq, int chunks, size_t* o_bytes) {
  const size_t slots = (size_t)batch * hq * chunks * kAttnRows;
  *o_bytes = align_up(slots * kAttnD * sizeof(float), 256);
  return *o_bytes + align_up(slots * 2 * sizeof(float), 256);
}

extern "C" size_t subspec_tree_attention_workspace(int64_t batch, int64_t n_q_heads, int64_t n_kv_heads, int64_t n_rows,
                                                   int64_t prefix_len, int64_t n_tree_slots) {
  if (batch <= 0 || n_q_heads <= 0 || n_kv_heads <= 0 || n_q_heads % n_kv_heads != 0 || n_rows <= 0) return 256;
  const AttnLaunch al = attn_launch(batch, n_q_heads, n_kv_heads, n_rows, prefix_len + n_tree_slots);
  if (al.pl.chunks == 1) return 256;
  size_t o_bytes;
  return attn_partial_bytes(al.vbatch, n_q_heads, al.pl.chunks, &o_bytes);
}

static int tree_attention_impl(const char* what, const void* q, const void* k_cache, const void* v_cache, void* out, int dtype,
                               int64_t batch, int64_t n_q_heads, int64_t n_kv_heads, int64_t n_rows, int64_t n_tree_slots,
                               int64_t head_dim, int64_t kv_seq_stride, int64_t prefix_len, const uint64_t* anc_bits,
                               int64_t anc_batch_stride, float scale, const KvPages* paged, const int64_t* prefix_dev,
                               void* workspace, size_t workspace_bytes, void* stream) {
  if (dtype != SUBSPEC_BF16 && dtype != SUBSPEC_F16)
    SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "%s: dtype %d not supported (bf16 / fp16 only)", what, dtype);
  if (!q || !k_cache || !v_cache || !out || !anc_bits) SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "%s: null pointer argument", what);
  if (head_dim != kAttnD) SUBSPEC_FAIL(SUBSPEC_ERR_LIMIT, "%s: head_dim=%lld (built for 128)", what, (long long)head_dim);
  if (batch <= 0 || n_q_heads <= 0 || n_kv_heads <= 0 || n_q_heads % n_kv_heads != 0)
    SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "%s: batch=%lld heads=%lld/%lld", what, (long long)batch, (long long)n_q_heads,
                 (long long)n_kv_heads);
  if (n_rows <= 0 || n_rows > SUBSPEC_MAX_TREE_NODES)
    SUBSPEC_FAIL(SUBSPEC_ERR_LIMIT, "%s: n_rows=%lld outside [1, %d]", what, (long long)n_rows, SUBSPEC_MAX_TREE_NODES);
  if (n_tree_slots < 1 || n_tree_slots > SUBSPEC_MAX_TREE_NODES)
    SUBSPEC_FAIL(SUBSPEC_ERR_LIMIT, "%s: n_tree_slots=%lld outside [1, %d] (at most %d 64-bit mask words per row)", what,
                 (long long)n_tree_slots, SUBSPEC_MAX_TREE_NODES, SUBSPEC_MAX_TREE_NODES / 64);
  if (prefix_len < 0 || prefix_len + n_tree_slots > kv_seq_stride)
    SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "%s: prefix_len=%lld + n_tree_slots=%lld exceeds the cache length %lld", what,
                 (long long)prefix_len, (long long)n_tree_slots, (long long)kv_seq_stride);
  if (batch * n_q_heads * ((n_rows + kAttnRows - 1) / kAttnRows) > 65535)
    SUBSPEC_FAIL(SUBSPEC_ERR_LIMIT, "%s: batch*heads*windows=%lld too large", what,
                 (long long)(batch * n_q_heads * ((n_rows + kAttnRows - 1) / kAttnRows)));
  if ((uintptr_t)q % 8 || (uintptr_t)k_cache % 16 || (uintptr_t)v_cache % 16 || (uintptr_t)out % 8)
    SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "%s: q/out must be 8-byte and k/v 16-byte aligned", what);
  AttnParams ap;
  ap.batch = batch; ap.hq = n_q_heads; ap.hkv = n_kv_heads; ap.n_rows = n_rows; ap.n_slots = n_tree_slots;
  ap.seq_stride = kv_seq_stride;
  ap.prefix = prefix_len; ap.anc_batch_stride = anc_batch_stride;
  ap.mask_words = (int)((n_tree_slots + 63) / 64);
  ap.row0 = 0; ap.win_rows = (int)std::min<int64_t>(n_rows, kAttnRows);
  ap.prefix_dev = prefix_dev;
  ap.page_table = nullptr; ap.page_shift = 0; ap.max_pages = 0; ap.page_stride = ap.tok_stride = ap.v_delta = 0;
  if (paged) {
    int shift = 0;
    while ((1ll << shift) < paged->page_len) ++shift;
    ap.page_table = paged->table;
    ap.page_shift = shift;
    ap.max_pages = (int)paged->max_pages;
    ap.tok_stride = n_kv_heads * kAttnD;
    ap.v_delta = paged->page_len * ap.tok_stride;
    ap.page_stride = 2 * ap.v_delta;
  }
  const int64_t kv_len = prefix_len + n_tree_slots;
  const int64_t blocks = (kv_len + kKeyBlock - 1) / kKeyBlock;
  ap.scale_log2 = scale * kLog2e;
  const int group = (int)(n_q_heads / n_kv_heads);
  float* part_o = nullptr;
  float* part_ml = nullptr;
  const AttnLaunch al = attn_launch(batch, n_q_heads, n_kv_heads, n_rows, kv_len);
  const AttnPlan& pl = al.pl;
  const int64_t vbatch = al.vbatch;
  if (pl.chunks > 1) {
    size_t o_bytes;
    const size_t need = attn_partial_bytes(vbatch, n_q_heads, pl.chunks, &o_bytes);
    if (!workspace || workspace_bytes < need)
      SUBSPEC_FAIL(SUBSPEC_ERR_WORKSPACE, "%s: workspace of %zu bytes is smaller than the %zu required", what,
                   workspace_bytes, need);
    if ((uintptr_t)workspace % 16) SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "%s: workspace must be 16-byte aligned", what);
    part_o = (float*)workspace;
    part_ml = (float*)((char*)workspace + o_bytes);
  }
  hipStream_t st = (hipStream_t)stream;
  {
    ap.row0 = 0;
    ap.win_rows = al.win_rows;
    ap.windows = al.windows;
    ap.chunk_keys = (blocks + pl.chunks - 1) / pl.chunks * kKeyBlock;
    ap.chunks = (int)((kv_len + ap.chunk_keys - 1) / ap.chunk_keys);
    ap.units = vbatch * n_kv_heads * ap.chunks;
    ap.pairs_per_kv = (group + pl.heads_per_wg - 1) / pl.heads_per_wg;
    const dim3 grid((unsigned)((ap.units + kXcds - 1) / kXcds * kXcds * ap.pairs_per_kv));
    const int64_t merge_rows = batch * n_q_heads * ap.win_rows / 8 >= 1024 ? 8 : 2;   // rows per merge workgroup (one window only)
    const dim3 merge_grid((unsigned)((ap.win_rows + merge_rows - 1) / merge_rows), (unsigned)(batch * n_q_heads));
#define SUBSPEC_ATTN_KERNEL(DT, PAGED, ROWT, WPH, THREADS)                                                          \
  hipLaunchKernelGGL((tree_attention_kernel<DT, PAGED, ROWT, WPH, THREADS>), grid, dim3(THREADS), 0, st, (const uint16_t*)q, \
                     (const uint16_t*)k_cache, (const uint16_t*)v_cache, anc_bits, ap, (uint16_t*)out, part_o, part_ml)
#define SUBSPEC_ATTN32_KERNEL(DT, PAGED, WPH, THREADS)                                                             \
  hipLaunchKernelGGL((tree_attention32_kernel<DT, PAGED, WPH, THREADS>), grid, dim3(THREADS), 0, st, (const uint16_t*)q, \
                     (const uint16_t*)k_cache, (const uint16_t*)v_cache, anc_bits, ap, (uint16_t*)out, part_o, part_ml)
#define SUBSPEC_ATTNPP_KERNEL(DT, WPH)                                                                             \
  hipLaunchKernelGGL((tree_attention_pp_kernel<DT, WPH>), grid, dim3(512), 0, st, (const uint16_t*)q,              \
                     (const uint16_t*)k_cache, (const uint16_t*)v_cache, anc_bits, ap, (uint16_t*)out, part_o, part_ml)
#define SUBSPEC_ATTN_LAUNCH(DT, PAGED)                                                                             \
  do {                                                                                                             \
    {                                                                                                              \
      DominantKernelTimer timer(st);                                                                               \
      if (!pl.mfma32) SUBSPEC_ATTN_KERNEL(DT, PAGED, 1, 1, 512);                                                   \
      else if (pl.pingpong && !PAGED) {                                                                            \
        if (pl.wph == 1) SUBSPEC_ATTNPP_KERNEL(DT, 1); else SUBSPEC_ATTNPP_KERNEL(DT, 2);                          \
      }                                                                                                            \
      else if (pl.wph == 1) SUBSPEC_ATTN32_KERNEL(DT, PAGED, 1, 512);                                              \
      else if (pl.threads == 512) SUBSPEC_ATTN32_KERNEL(DT, PAGED, 2, 512);                                        \
      else SUBSPEC_ATTN32_KERNEL(DT, PAGED, 2, 256);                                                               \
    }                                                                                                              \
    if (ap.chunks > 1) {                                                                                           \
      if (pl.mfma32) {                                                                                             \
        const dim3 mg((unsigned)(vbatch * n_q_heads * 2), 4);                                                      \
        if (ap.chunks <= 4) hipLaunchKernelGGL((tree_attention32_merge_kernel<DT, 4>), mg, dim3(256), 0, st, part_o, part_ml, ap, (uint16_t*)out); \
        else if (ap.chunks <= 8) hipLaunchKernelGGL((tree_attention32_merge_kernel<DT, 8>), mg, dim3(256), 0, st, part_o, part_ml, ap, (uint16_t*)out); \
        else hipLaunchKernelGGL((tree_attention32_merge_kernel<DT, 0>), mg, dim3(256), 0, st, part_o, part_ml, ap, (uint16_t*)out); \
      } else                                                                                                         \
        hipLaunchKernelGGL((tree_attention_merge_kernel<DT>), merge_grid, dim3(merge_rows * 32), 0, st, part_o, part_ml, ap, \
                           (uint16_t*)out);                                                                        \
    }                                                                                                              \
  } while (0)
    if (dtype == SUBSPEC_BF16) { if (paged) SUBSPEC_ATTN_LAUNCH(SUBSPEC_BF16, true); else SUBSPEC_ATTN_LAUNCH(SUBSPEC_BF16, false); }
    else { if (paged) SUBSPEC_ATTN_LAUNCH(SUBSPEC_F16, true); else SUBSPEC_ATTN_LAUNCH(SUBSPEC_F16, false); }
#undef SUBSPEC_ATTN_LAUNCH
#undef SUBSPEC_ATTN32_KERNEL
#undef SUBSPEC_ATTN_KERNEL
  }
  SUBSPEC_CHECK_HIP(hipGetLastError());
  return SUBSPEC_OK;
}

extern "C" int subspec_tree_attention(const void* q, const void* k_cache, const void* v_cache, void* out, int dtype,
                                      int64_t batch, int64_t n_q_heads, int64_t n_kv_heads, int64_t n_rows,
                                      int64_t n_tree_slots, int64_t head_dim, int64_t kv_seq_stride, int64_t prefix_len,
                                      const uint64_t* anc_bits, int64_t anc_batch_stride, float scale,
                                      void* workspace, size_t workspace_bytes, void* stream) {
  return tree_attention_impl("tree_attention", q, k_cache, v_cache, out, dtype, batch, n_q_heads, n_kv_heads, n_rows,
                             n_tree_slots, head_dim, kv_seq_stride, prefix_len, anc_bits, anc_batch_stride, scale, nullptr,
                             nullptr, workspace, workspace_bytes, stream);
}

extern "C" int subspec_tree_attention_paged(const void* q, const void* kv_pool_layer, const int32_t* page_indices,
                                            int64_t n_pages, int64_t max_pages, int64_t page_len, void* out, int dtype,
                                            int64_t n_q_heads, int64_t n_kv_heads, int64_t n_rows, int64_t n_tree_slots,
                                            int64_t head_dim, int64_t prefix_len, const uint64_t* anc_bits, float scale,
                                            void* workspace, size_t workspace_bytes, void* stream) {
  if (!page_indices) SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "tree_attention_paged: null page table");
  if (page_len <= 0 || (page_len & (page_len - 1)) != 0 || page_len > 4096)
    SUBSPEC_FAIL(SUBSPEC_ERR_LIMIT, "tree_attention_paged: page_len=%lld must be a power of two up to 4096", (long long)page_len);
  if (n_pages <= 0 || max_pages < n_pages || max_pages > 0x7fffffff)
    SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "tree_attention_paged: n_pages=%lld max_pages=%lld", (long long)n_pages, (long long)max_pages);
  const KvPages pg{page_indices, n_pages, max_pages, page_len};
  // the request's pages play the part of the cache length: rows beyond them do not exist
  return tree_attention_impl("tree_attention_paged", q, kv_pool_layer, kv_pool_layer, out, dtype, 1, n_q_heads, n_kv_heads,
                             n_rows, n_tree_slots, head_dim, n_pages * page_len, prefix_len, anc_bits, 0, scale, &pg, nullptr,
                             workspace, workspace_bytes, stream);
}

int subspec::tree_attention_ex(const void* q, const void* k_cache, const void* v_cache, void* out, int dtype, int64_t n_q_heads,
                               int64_t n_kv_heads, int64_t n_rows, int64_t n_tree_slots, int64_t kv_seq_stride, int64_t prefix_len,
                               const int64_t* prefix_dev, const KvPages* pages, const uint64_t* anc_bits, float scale,
                               void* workspace, size_t workspace_bytes, void* stream) {
  if (pages) {
    if (!pages->table) SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "tree_attention: null page table");
    if (pages->page_len <= 0 || (pages->page_len & (pages->page_len - 1)) != 0 || pages->page_len > 4096)
      SUBSPEC_FAIL(SUBSPEC_ERR_LIMIT, "tree_attention: page_len=%lld must be a power of two up to 4096", (long long)pages->page_len);
    if (pages->n_pages <= 0 || pages->max_pages < pages->n_pages || pages->max_pages > 0x7fffffff)
      SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "tree_attention: n_pages=%lld max_pages=%lld", (long long)pages->n_pages, (long long)pages->max_pages);
    return tree_attention_impl("tree_attention", q, k_cache, k_cache, out, dtype, 1, n_q_heads, n_kv_heads, n_rows, n_tree_slots, kAttnD,
                               pages->n_pages * pages->page_len, prefix_len, anc_bits, 0, scale, pages, prefix_dev, workspace,
                               workspace_bytes, stream);
  }
  return tree_attention_impl("tree_attention", q, k_cache, v_cache, out, dtype, 1, n_q_heads, n_kv_heads, n_rows, n_tree_slots, kAttnD,
                             kv_seq_stride, prefix_len, anc_bits, 0, scale, nullptr, prefix_dev, workspace, workspace_bytes, stream);
}
