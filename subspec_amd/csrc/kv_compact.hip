// KV-cache compaction for gfx950: keep the K/V rows of the accepted tree nodes.
//
// One workgroup per (slab, 256-byte column block): a slab is one [seq, row_bytes] matrix (one
// layer x {K,V} x batch x kv-head).  All source rows are read into registers first, then a
// barrier, then written, so the overlapping source/destination ranges behave exactly like the
// reference's index_select followed by index_copy_ (specdecodes/models/utils/cache_utils.py:199-208).
// Pure data movement: algorithmic bytes = 2 * slabs * count * row_bytes; latency-bound at the
// sizes of one speculative cycle.  The row count may be read from device memory so the kernel can
// be queued right behind the verifier without a host round trip.
//
// Paged pools (one request's pages of a [layers][max_pages][2][page_len][heads * head_dim] pool, the
// layout of KvCachePool in specdecodes/models/utils/flashinfer/cache_manager.py:35-52) use the same
// kernel: a slab is one (layer, K or V) plane, a row is one token (all heads), and row r sits in page
// page_table[r / page_len] at token r % page_len.
#include "common.h"

namespace subspec {

constexpr int kCompactThreads = 256;
constexpr int kSegBytes = 16;
constexpr int kSegsPerBlock = 16;                               // 256-byte column block
constexpr int kRowsPerRound = kCompactThreads / kSegsPerBlock;  // 16 rows in flight per round
constexpr int kMaxRounds = SUBSPEC_MAX_TREE_NODES / kRowsPerRound;

struct PageMap {
  const int32_t* table;      // NULL: rows are contiguous
  int page_shift, max_pages;
  int64_t page_stride;       // bytes between consecutive pages of one slab
  int inner_count;           // slab i = base + (i / inner_count) * slab_stride + (i % inner_count) * inner_stride
  int64_t inner_stride;
};

__global__ __launch_bounds__(kCompactThreads) void kv_compact_kernel(
    char* base, void* const* slab_ptrs, int64_t slab_stride, int64_t seq_len, int64_t row_bytes,
    int64_t offset, const int64_t* __restrict__ ctx, const int32_t* __restrict__ count_dev, int count_host,
    int max_count, PageMap pm) {
  int count = count_dev ? *count_dev : count_host;
  count = min(count, max_count);
  char* slab = slab_ptrs ? (char*)slab_ptrs[blockIdx.x]
                         : base + (int64_t)(blockIdx.x / pm.inner_count) * slab_stride + (int64_t)(blockIdx.x % pm.inner_count) * pm.inner_stride;
  auto row_at = [&](int64_t r) -> char* {
    if (!pm.table) return slab + r * row_bytes;
    const int page = min(max(pm.table[r >> pm.page_shift], 0), pm.max_pages - 1);   // a bad table must not fault
    return slab + (int64_t)page * pm.page_stride + (r & ((1 << pm.page_shift) - 1)) * row_bytes;
  };
  const int seg = threadIdx.x % kSegsPerBlock;
  const int r0 = threadIdx.x / kSegsPerBlock;
  const int64_t col = ((int64_t)blockIdx.y * kSegsPerBlock + seg) * kSegBytes;
  const bool col_ok = col < row_bytes;

  uint4 held[kMaxRounds];
#pragma unroll
  for (int k = 0; k < kMaxRounds; ++k) {
    const int j = k * kRowsPerRound + r0;
    if (col_ok && j < count) {
      const int64_t src = offset + ctx[j];
      // a context outside the cache would be a caller bug; skip it rather than fault
      if (src >= 0 && src < seq_len) held[k] = *(const uint4*)(row_at(src) + col);
      else held[k] = make_uint4(0, 0, 0, 0);
    }
  }
  __syncthreads();
#pragma unroll
  for (int k = 0; k < kMaxRounds; ++k) {
    const int j = k * kRowsPerRound + r0;
    if (col_ok && j < count) {
      const int64_t src = offset + ctx[j];
      const int64_t dst = offset + j;
      if (src >= 0 && src < seq_len && dst < seq_len) *(uint4*)(row_at(dst) + col) = held[k];
    }
  }
}

}  // namespace subspec

using namespace subspec;

extern "C" int subspec_kv_compact(void* base, void* const* slab_ptrs, int64_t n_slabs, int64_t slab_stride_bytes,
                                  int64_t seq_len, int64_t row_bytes, int64_t offset, const int64_t* ctx,
                                  const int32_t* count_dev, int32_t count_host, int32_t max_count, void* stream) {
  if ((!base && !slab_ptrs) || !ctx) SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "kv_compact: null pointer argument");
  if (n_slabs <= 0 || n_slabs > 0x7fffffff) SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "kv_compact: n_slabs=%lld", (long long)n_slabs);
  if (row_bytes <= 0 || row_bytes % kSegBytes != 0)
    SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "kv_compact: row_bytes=%lld must be a positive multiple of 16", (long long)row_bytes);
  if (base && ((uintptr_t)base % kSegBytes != 0 || slab_stride_bytes % kSegBytes != 0))
    SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "kv_compact: base / slab stride must be 16-byte aligned");
  if (offset < 0 || seq_len <= 0 || offset > seq_len)
    SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "kv_compact: offset=%lld seq_len=%lld", (long long)offset, (long long)seq_len);
  if (max_count < 0 || max_count > SUBSPEC_MAX_TREE_NODES)
    SUBSPEC_FAIL(SUBSPEC_ERR_LIMIT, "kv_compact: max_count=%d exceeds %d", max_count, SUBSPEC_MAX_TREE_NODES);
  if (!count_dev && (count_host < 0 || count_host > max_count))
    SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "kv_compact: count=%d outside [0, max_count=%d]", count_host, max_count);
  if (max_count == 0 || (!count_dev && count_host == 0)) return SUBSPEC_OK;
  const int64_t col_blocks = (row_bytes + kSegBytes * kSegsPerBlock - 1) / (kSegBytes * kSegsPerBlock);
  if (col_blocks > 65535) SUBSPEC_FAIL(SUBSPEC_ERR_LIMIT, "kv_compact: row_bytes=%lld too wide", (long long)row_bytes);
  hipLaunchKernelGGL(kv_compact_kernel, dim3((unsigned)n_slabs, (unsigned)col_blocks), dim3(kCompactThreads), 0,
                     (hipStream_t)stream, (char*)base, slab_ptrs, slab_stride_bytes, seq_len, row_bytes, offset, ctx,
                     count_dev, count_host, max_count, PageMap{nullptr, 0, 0, 0, 1, 0});
  SUBSPEC_CHECK_HIP(hipGetLastError());
  return SUBSPEC_OK;
}

extern "C" int subspec_kv_compact_paged(void* pool, int64_t n_layers, int64_t max_pages, int64_t page_len, int64_t token_bytes,
                                        const int32_t* page_indices, int64_t n_pages, int64_t offset, const int64_t* ctx,
                                        const int32_t* count_dev, int32_t count_host, int32_t max_count, void* stream) {
  if (!pool || !page_indices || !ctx) SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "kv_compact_paged: null pointer argument");
  if (n_layers <= 0 || n_layers > (1 << 20)) SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "kv_compact_paged: n_layers=%lld", (long long)n_layers);
  if (page_len <= 0 || (page_len & (page_len - 1)) != 0 || page_len > 4096)
    SUBSPEC_FAIL(SUBSPEC_ERR_LIMIT, "kv_compact_paged: page_len=%lld must be a power of two up to 4096", (long long)page_len);
  if (n_pages <= 0 || max_pages < n_pages || max_pages > 0x7fffffff)
    SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "kv_compact_paged: n_pages=%lld max_pages=%lld", (long long)n_pages, (long long)max_pages);
  if (token_bytes <= 0 || token_bytes % kSegBytes != 0 || (uintptr_t)pool % kSegBytes != 0)
    SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "kv_compact_paged: token_bytes=%lld must be a positive multiple of 16 and the pool 16-byte aligned",
                 (long long)token_bytes);
  const int64_t seq_len = n_pages * page_len;
  if (offset < 0 || offset > seq_len) SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "kv_compact_paged: offset=%lld outside the %lld rows of the request", (long long)offset, (long long)seq_len);
  if (max_count < 0 || max_count > SUBSPEC_MAX_TREE_NODES)
    SUBSPEC_FAIL(SUBSPEC_ERR_LIMIT, "kv_compact_paged: max_count=%d exceeds %d", max_count, SUBSPEC_MAX_TREE_NODES);
  if (!count_dev && (count_host < 0 || count_host > max_count))
    SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "kv_compact_paged: count=%d outside [0, max_count=%d]", count_host, max_count);
  if (max_count == 0 || (!count_dev && count_host == 0)) return SUBSPEC_OK;
  const int64_t col_blocks = (token_bytes + kSegBytes * kSegsPerBlock - 1) / (kSegBytes * kSegsPerBlock);
  if (col_blocks > 65535) SUBSPEC_FAIL(SUBSPEC_ERR_LIMIT, "kv_compact_paged: token_bytes=%lld too wide", (long long)token_bytes);
  int shift = 0;
  while ((1ll << shift) < page_len) ++shift;
  const int64_t plane = page_len * token_bytes;                  // one page's K (or V) rows
  const PageMap pm{page_indices, shift, (int)max_pages, 2 * plane, 2, plane};
  hipLaunchKernelGGL(kv_compact_kernel, dim3((unsigned)(n_layers * 2), (unsigned)col_blocks), dim3(kCompactThreads), 0,
                     (hipStream_t)stream, (char*)pool, (void* const*)nullptr, max_pages * 2 * plane, seq_len, token_bytes, offset,
                     ctx, count_dev, count_host, max_count, pm);
  SUBSPEC_CHECK_HIP(hipGetLastError());
  return SUBSPEC_OK;
}
