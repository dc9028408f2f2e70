/*
 * C ABI of libsubspec_hip.so: hand-written gfx950 (MI355X) kernels for the speculative-decoding
 * hot path of NYCU-EDgeAi/subspec.  Plain pointers and sizes only; every pointer named "device"
 * is device memory owned by the caller, every call is asynchronous on `stream` (a hipStream_t
 * passed as void*, NULL = the default stream) and allocates nothing.
 *
 * Return value: 0 on success, a negative SUBSPEC_ERR_* otherwise; subspec_last_error() then
 * returns a human-readable message (thread-local).
 *
 * Each entry point cites the reference interface it replaces (paths relative to the reference).
 */
#ifndef SUBSPEC_HIP_H
#define SUBSPEC_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SUBSPEC_ABI_VERSION 2

/* element types of logits / probabilities / KV / activations */
#define SUBSPEC_F32 0
#define SUBSPEC_F16 1
#define SUBSPEC_BF16 2

#define SUBSPEC_OK 0
#define SUBSPEC_ERR_ARG (-1)       /* bad shape / dtype / alignment / null pointer */
#define SUBSPEC_ERR_WORKSPACE (-2) /* workspace too small */
#define SUBSPEC_ERR_HIP (-3)       /* a HIP runtime call failed */
#define SUBSPEC_ERR_LIMIT (-4)     /* size beyond what the kernels are built for */

/* verify_method / threshold_method as in generator_kwargs (configs/methods/subspec_sd_lossy.yaml:20-31) */
#define SUBSPEC_VERIFY_EXACT 0
#define SUBSPEC_VERIFY_LOSSY 1
#define SUBSPEC_GATE_ENTROPY 0
#define SUBSPEC_GATE_PROB 1

/* How the normalized entropy of 16-bit rows is evaluated.
 *  GUARD : one fp32 pass; rows whose entropy lies within 2% of the threshold are re-evaluated
 *          with the reference's per-element rounding (p, log p and p*log p each rounded to the
 *          row dtype), so gate decisions match the reference.
 *  ALWAYS: every row uses the per-element rounding; node_entropy is then the value the
 *          reference computes.
 * Bit-exact against the reference's CPU path: bf16 and fp32 rows.  fp16 rows (always evaluated with the
 * per-element rounding) agree except where torch's CPU softmax loses small addends: it accumulates
 * sum exp in 16 fp32 lanes, and the lane that holds a dominant logit drops them, which can move the
 * rounded maximum probability of a peaked fp16 row by one step and its entropy by up to 1 %.  An fp16
 * lossy run therefore takes the reference's gate decisions except for entropies within about 1 % of the
 * threshold; accepted paths, argmax tokens and bf16 / fp32 entropies are exact. */
#define SUBSPEC_ENTROPY_GUARD 0
#define SUBSPEC_ENTROPY_ALWAYS 1

/* Largest tree: nodes the verifier walks, tree slots (and query rows) attention takes, rows one
 * compaction moves.  The reference's offloading configurations draft 1 + 48 * 6 = 289 nodes
 * (configs/exp_offloading/subspec_sd_qwen_7b.yaml:16-19). */
#define SUBSPEC_MAX_TREE_NODES 512

int subspec_abi_version(void);
const char* subspec_last_error(void);

/* Measurement aid (no counterpart in the reference, whose phase timing is CUDA events around Python
 * calls, specdecodes/models/utils/mixin.py:101-224): while enabled, each entry-point call records a pair
 * of events on its launch stream around its dominant kernel (the one pass over the logits /
 * probabilities / KV / weights).  Up to 512 calls are kept since the last enable;
 * subspec_profile_read_ms(i) waits for call i's pair and returns that kernel's duration in
 * milliseconds (-1 if out of range).  Process-wide, not thread-safe. */
int subspec_profile_enable(int on);
int subspec_profile_count(void);
float subspec_profile_read_ms(int index);

/* ------------------------------------------------------------------------------------------
 * Tree verification, fused: softmax statistics, first-index argmax of the rounded probabilities,
 * normalized entropy, p[parent(i), token(i)] for every node, then the greedy walk or the lossy
 * bottom-up DP, longest-path extraction and bonus token -- three kernel launches, no host sync.
 *
 * Replaces  verify_tree            specdecodes/models/utils/tree_verify.py:8-163
 *           lossy_bottom_up_verify specdecodes/models/utils/lossy_tree_verify.py:9-343
 *           _sample_token(return_probs=True) + .cpu()   specdecodes/models/generators/base.py:109-139,
 *                                                       tree_verify.py:51-52,117-118
 *           _verify_step           specdecodes/models/generators/classic_sd.py:111-116
 * for the greedy (do_sample=False) target.
 *
 * logits      device, [batch, rows, vocab] contiguous, element type `dtype`; row r of a tree is
 *             the target distribution at original node r + skip_nodes.
 * token_ids   device int32 [batch, n_nodes]   token of every node of the WHOLE tree
 * parents     device int32 [batch, n_nodes]   parent index, -1 for the root; parent < child
 * root        context node to start from (original indexing)
 * eos_token_id  < 0 : none
 * out_tokens  device int64 [batch, n_nodes + 1]  accepted tokens followed by the bonus token
 * out_ctx     device int64 [batch, n_nodes + 1]  context node (original indexing) of each token
 *                                               = the KV rows to keep
 * out_counts  device int32 [batch, 4]  {emitted, accept_len, total_len, status}; status != 0
 *                                      means the tree broke a precondition (see verify.hip)
 * node_target / node_entropy / node_child_prob   device [batch, rows] (int64 / float / float):
 *             argmax token, normalized entropy and p[parent(i), token(i)] per scored node
 *             (what the reference's diagnostics are computed from); node_entropy is 0 unless
 *             the entropy gate is used.  node_target and node_entropy are written for every row,
 *             node_child_prob for every row that is a node of the tree (the caller need not clear them).
 */
size_t subspec_tree_verify_workspace(int64_t batch, int64_t rows, int64_t vocab, int dtype);

int subspec_tree_verify(const void* logits, int dtype, int64_t batch, int64_t rows, int64_t vocab,
                        const int32_t* token_ids, const int32_t* parents, int64_t n_nodes,
                        int32_t root, int32_t skip_nodes, int64_t eos_token_id,
                        int verify_method, int threshold_method, double threshold, int32_t window_size,
                        int entropy_policy,
                        void* workspace, size_t workspace_bytes,
                        int64_t* out_tokens, int64_t* out_ctx, int32_t* out_counts,
                        int64_t* node_target, float* node_entropy, float* node_child_prob,
                        void* stream);

/* subspec_tree_verify for callers that cannot allocate device memory (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  Same arguments,
 * kernels and results as subspec_tree_verify (greedy target), minus the workspace: the per-slice partial
 * records live in an array built into the library (SUBSPEC_TREE_VERIFY_STATIC_MAX_ROWS * 64 slices * 48
 * bytes = 6 MiB of device memory per GPU, held until the process ends).  The call allocates nothing.
 * batch * rows beyond SUBSPEC_TREE_VERIFY_STATIC_MAX_ROWS is rejected with SUBSPEC_ERR_LIMIT.  All calls
 * on one GPU share that GPU's array: calls that overlap on one GPU (different streams or threads) race;
 * calls in stream order do not.  Nothing in the array needs to start at zero.  The FIRST call on a device looks up the
 * array's address (hipGetSymbolAddress, which may load the code object): make it outside a graph capture; every later
 * call on that device only launches kernels. */
#define SUBSPEC_TREE_VERIFY_STATIC_MAX_ROWS 2048

int subspec_tree_verify_static(const void* logits, int dtype, int64_t batch, int64_t rows, int64_t vocab,
                               const int32_t* token_ids, const int32_t* parents, int64_t n_nodes,
                               int32_t root, int32_t skip_nodes, int64_t eos_token_id,
                               int verify_method, int threshold_method, double threshold, int32_t window_size,
                               int entropy_policy,
                               int64_t* out_tokens, int64_t* out_ctx, int32_t* out_counts,
                               int64_t* node_target, float* node_entropy, float* node_child_prob,
                               void* stream);

/* Tree verification with a SAMPLED target token (do_sample=True).
 *
 * Replaces the same call sites as subspec_tree_verify when the generator samples:
 *   GeneratorBase._sample_token(do_sample=True)   specdecodes/models/generators/base.py:116-132
 *     (TemperatureLogitsWarper, softmax in the logits dtype, torch.multinomial(probs, 1))
 *   ClassicSDGeneratorBase._verify_step            specdecodes/models/generators/classic_sd.py:111-116
 *   lossy_bottom_up_verify target_tokens           specdecodes/models/utils/lossy_tree_verify.py:75-77
 *
 * Every logits row is divided by `temperature` and rounded to its dtype, its probabilities
 * p_i = softmax rounded to the dtype are formed as in subspec_tree_verify, and ONE token per row is
 * drawn by the exponential race  argmax_i p_i / E_i  (first index on equal keys),
 *   E_i = -log(u_i),  u_i = ((w >> 9) + 0.5) * 2^-23,
 *   w   = word (i mod 4) of Philox4x32-10(counter = {i / 4, batch_index * rows + row,
 *                                                    offset low word, offset high word},
 *                                         key = {seed low word, seed high word}).
 * The draw of a row is used wherever the greedy verifier uses the row's argmax: at most one draw
 * per context, as in the reference's walk.  The probability gate, the entropy gate and
 * node_child_prob / node_entropy refer to the warped rows; node_target holds the draws.  Callers
 * advance `offset` between calls to get fresh noise from one seed.  Other arguments, outputs and
 * the workspace are those of subspec_tree_verify.  A one-node tree (n_nodes = 1, rows = 1) returns
 * the draw of a single row in out_tokens[0]: the first token after the prefill.
 */
int subspec_tree_verify_sample(const void* logits, int dtype, int64_t batch, int64_t rows, int64_t vocab,
                               const int32_t* token_ids, const int32_t* parents, int64_t n_nodes,
                               int32_t root, int32_t skip_nodes, int64_t eos_token_id,
                               int verify_method, int threshold_method, double threshold,
                               int32_t window_size, int entropy_policy, float temperature, uint64_t seed,
                               uint64_t offset, void* workspace, size_t workspace_bytes,
                               int64_t* out_tokens, int64_t* out_ctx, int32_t* out_counts,
                               int64_t* node_target, float* node_entropy, float* node_child_prob,
                               void* stream);

/* ------------------------------------------------------------------------------------------
 * KV-cache compaction after verification: for every slab (one [seq, row_bytes] matrix: one
 * layer x {K,V} x batch x kv-head), row offset+j <- row offset+ctx[j] for j < count, with
 * gather-then-scatter semantics; rows outside [offset, offset+count) are untouched.
 *
 * Replaces  KVManager.reorder_cache_with_offset -> TreeStaticCache.reorder_cache_with_offset
 *           specdecodes/models/utils/cache_utils.py:55-56,166-208 (and :85-103 for the dynamic cache).
 *
 * slab_ptrs   device array of n_slabs base pointers, or NULL when the slabs are
 *             base + i * slab_stride_bytes
 * ctx         device int64 [>= count]  (e.g. out_ctx of subspec_tree_verify)
 * count_dev   device int32*, number of rows to move read on the device (e.g. &out_counts[0]);
 *             NULL -> use count_host.  max_count bounds both (<= SUBSPEC_MAX_TREE_NODES).
 */
int subspec_kv_compact(void* base, void* const* slab_ptrs, int64_t n_slabs, int64_t slab_stride_bytes,
                       int64_t seq_len, int64_t row_bytes, int64_t offset,
                       const int64_t* ctx, const int32_t* count_dev, int32_t count_host, int32_t max_count,
                       void* stream);

/* ------------------------------------------------------------------------------------------
 * Top-k draft-tree expansion: per batch item the global top-k over (leaves x vocab) of
 * round_dtype(probs[b, l, v] * parent_probs[b, l]), sorted by value descending and, among equal
 * values, flat index (l * vocab + v) ascending.
 *
 * Replaces  DraftModelBase.topk_sampling -> _topk_flatten   specdecodes/models/draft_models/base.py:268-305
 *           (and its graph twin _topk_flatten_for_graph :307-323): torch.mul into a full-size buffer
 *           followed by torch.topk over the flattened row.
 *
 * probs          device [batch, leaves, vocab] contiguous, element type `dtype`
 * parent_probs   device [batch, leaves], same dtype
 * k              1 <= k <= min(vocab, 64)   (the reference clamps k to vocab on the host)
 * token_ids      device int64 [batch, k]    flat index %  vocab
 * topk_probs     device `dtype` [batch, k]
 * parent_indices device int64 [batch, k]    flat index // vocab
 */
size_t subspec_topk_expand_workspace(int64_t batch, int64_t leaves, int64_t vocab, int32_t k);

int subspec_topk_expand(const void* probs, const void* parent_probs, int dtype, int64_t batch, int64_t leaves,
                        int64_t vocab, int32_t k, void* workspace, size_t workspace_bytes,
                        int64_t* token_ids, void* topk_probs, int64_t* parent_indices, void* stream);

/* ------------------------------------------------------------------------------------------
 * Tree-masked GQA attention of the draft tree against the static KV cache:
 * out = softmax(q k^T * scale + mask) v, where query row i attends to cache rows [0, prefix_len) and
 * to tree slot prefix_len + j (j < n_tree_slots <= SUBSPEC_MAX_TREE_NODES) iff bit j of row i's ancestor bitset is set (the
 * node in slot j is row i's node or one of its ancestors).  The verify forward has one query row per
 * slot; a draft step queries only the newest level (n_rows < n_tree_slots); a tree extended during
 * the target forward (post-speculation) occupies more slots than the tree that is being verified.
 *
 * Replaces  HF sdpa_attention_forward under SDPBackend.MATH with the additive finfo.min mask and
 *           repeat_kv, as reached from _tree_decoding   specdecodes/models/generators/classic_sd.py:57-109
 *           (run/pipelines/run_test.py:64); mask construction Tree.create_attention_mask
 *           specdecodes/models/utils/cpu_tree.py:263-286, _get_tree_mask / invert_mask
 *           generators/classic_sd.py:33-55, utils/utils.py:4-6.  The FlashInfer form is
 *           flashinfer/attention_wrapper.py:116-151,288-316.
 *
 * q          device [batch, n_q_heads, n_rows, head_dim]      bf16 / fp16, head_dim = 128, n_rows <= SUBSPEC_MAX_TREE_NODES
 *            (more than 64 rows: windows of 64 rows in the same launch, which share the keys)
 * k_cache    device [batch, n_kv_heads, kv_seq_stride, head_dim]  (HF static-cache layout); the K/V of
 * v_cache    the tree nodes must already sit in rows prefix_len .. prefix_len + n_tree_slots - 1
 * out        device [batch, n_rows, n_q_heads, head_dim]       (= [batch, n_rows, hidden])
 * anc_bits   device uint64 [*, n_rows, words], words = ceil(n_tree_slots / 64) (bit j of a row is bit
 *            j % 64 of word j / 64); batch element b uses rows from b * anc_batch_stride (0: shared tree)
 * workspace  partial results when the keys are split over workgroups (may be NULL if the size is 256)
 */
size_t subspec_tree_attention_workspace(int64_t batch, int64_t n_q_heads, int64_t n_kv_heads, int64_t n_rows,
                                        int64_t prefix_len, int64_t n_tree_slots);

int subspec_tree_attention(const void* q, const void* k_cache, const void* v_cache, void* out, int dtype,
                           int64_t batch, int64_t n_q_heads, int64_t n_kv_heads, int64_t n_rows,
                           int64_t n_tree_slots, int64_t head_dim,
                           int64_t kv_seq_stride, int64_t prefix_len, const uint64_t* anc_bits,
                           int64_t anc_batch_stride, float scale, void* workspace, size_t workspace_bytes,
                           void* stream);

/* ------------------------------------------------------------------------------------------
 * Paged KV cache (one request): the same attention and compaction over the page pool of the
 * reference's FlashInfer path instead of the contiguous static cache.
 *
 * Pool layout  [layers][max_pages][2 (K, V)][page_len][n_kv_heads][head_dim]   ("NHD" pages):
 *           KvCachePool.cache_data    specdecodes/models/utils/flashinfer/cache_manager.py:35-52
 * page_indices  device int32 [n_pages]: the request's pages in sequence order
 *           RequestKvCache.kv_page_indices / KvCacheBatchPosition.kv_page_indices   cache_manager.py:9-25,218-240,350-372
 * Cache row p lives in page page_indices[p / page_len] at token p % page_len; page_len must be a power
 * of two.  Page numbers are clamped to [0, max_pages) on the device, so a corrupt table reads wrong
 * rows but never leaves the pool.
 *
 * subspec_tree_attention_paged replaces
 *   flashinfer.BatchPrefillWithPagedKVCacheWrapper.run with custom_mask (mode "tree")
 *           specdecodes/models/utils/flashinfer/attention_wrapper.py:104-137 and its forward call
 * kv_pool_layer = one layer of the pool; every other argument as in subspec_tree_attention (batch 1,
 * workspace = subspec_tree_attention_workspace(1, n_q_heads, n_kv_heads, n_rows, prefix_len, n_tree_slots)).
 *
 * subspec_kv_compact_paged replaces
 *   KvCachePool.reorder_cache_with_offset (clone of every layer, index_select / index_copy_, copy back)
 *           cache_manager.py:120-213
 * for all layers, K and V, in one launch: row offset + j <- row offset + ctx[j], j < count, rows
 * addressed through page_indices (the reference indexes the pool as if the request's pages were
 * 0, 1, 2, ...: the identity table).  token_bytes = n_kv_heads * head_dim * sizeof(dtype).
 */
int subspec_tree_attention_paged(const void* q, const void* kv_pool_layer, const int32_t* page_indices, int64_t n_pages,
                                 int64_t max_pages, int64_t page_len, void* out, int dtype, int64_t n_q_heads,
                                 int64_t n_kv_heads, int64_t n_rows, int64_t n_tree_slots, int64_t head_dim,
                                 int64_t prefix_len, const uint64_t* anc_bits, float scale, void* workspace,
                                 size_t workspace_bytes, void* stream);

int subspec_kv_compact_paged(void* pool, int64_t n_layers, int64_t max_pages, int64_t page_len, int64_t token_bytes,
                             const int32_t* page_indices, int64_t n_pages, int64_t offset, const int64_t* ctx,
                             const int32_t* count_dev, int32_t count_host, int32_t max_count, void* stream);

/* ------------------------------------------------------------------------------------------
 * Draft probabilities: out = softmax(round(logits / temperature)) over the last axis, in the logits
 * dtype (the quotient is rounded to the dtype first, the softmax is evaluated in fp32 and each
 * probability rounded once).
 *
 * Replaces  ClassicSDDraftModel.forward(with_softmax=True): torch.softmax(logits / temperature, -1)
 *           specdecodes/models/draft_models/classic_sd.py:10-16
 *
 * logits, out  device [rows, vocab], same dtype (fp32 / fp16 / bf16); out may alias logits.
 * workspace    device, 8-byte aligned, subspec_softmax_temperature_workspace(rows, vocab) bytes, or
 *              NULL.  With few rows (a draft step has 1 to 16) one workgroup per row leaves the chip
 *              idle; given the workspace, rows are cut into slices over two launches.  NULL (or a
 *              size of 0 returned by the query) selects the one-workgroup-per-row kernel.
 */
size_t subspec_softmax_temperature_workspace(int64_t rows, int64_t vocab);

int subspec_softmax_temperature(const void* logits, void* out, int dtype, int64_t rows, int64_t vocab,
                                float temperature, void* workspace, size_t workspace_bytes, void* stream);

/* TemperatureLogitsWarper alone: out[i] = logits[i] / temperature, the IEEE quotient rounded once to
 * the logits dtype (what ``scores / temperature`` gives for a tensor in that dtype).
 *
 * Replaces  logits_processor(None, logits) with a TemperatureLogitsWarper in
 *           GeneratorBase._sample_token   specdecodes/models/generators/base.py:57-58,121-123
 * for callers that want the warped scores themselves; the sampling verifier and
 * subspec_softmax_temperature apply the same quotient internally.  n = number of elements.
 */
int subspec_temperature_warp(const void* logits, void* out, int dtype, int64_t n, float temperature,
                             void* stream);

/* ------------------------------------------------------------------------------------------
 * int4 group-wise (group 64 along the input dimension, fp16 scale and zero per row and group)
 * linear layer of the substitute draft:  y[M, N] = x[M, K] * ((Wq - zero) * scale)^T (+ bias).
 *
 * Replaces  hqq HQQLinear -> gemlite A16W4 GEMV/GEMM as installed by HqqQuantizer.quantize_model
 *           specdecodes/helpers/quantizers/hqq/__init__.py:17-120 (AutoHQQHFModel.quantize_model
 *           quantizers/hqq/hf/base.py:94-230) for BaseQuantizeConfig(nbits=4, group_size=64, axis=1)
 *           specdecodes/helpers/recipes/subspec/hqq_4bit_postspec.py:17-58.
 *
 * x     device [M, K]  bf16 / fp16, K % 64 == 0; one pass over the weights serves 64 rows (a tree window),
 *       more rows are further passes on the same stream
 * wq    device uint32, tiled codes: [N/16][K/64][4][16] entries of 8 bytes; entry (c, r) holds the 16
 *       codes of row 16*nt + r for k = 64*g + 16*c .. +15, word j the codes of k = .. + 8j .. +7
 *       with code(8j + 2i) in bits 4i..4i+3 and code(8j + 2i + 1) in bits 16+4i..16+4i+3
 * sz    device uint32 [N/16][K/64][16]: fp16 scale (low half) and fp16 zero (high half) of
 *       row 16*nt + r, group g
 * bias  device [N] (same dtype as x) or NULL
 * y     device [M, N], same dtype as x;  N % 16 == 0
 */
size_t subspec_int4_linear_workspace(int64_t M, int64_t N, int64_t K);

int subspec_int4_linear(const void* x, const uint32_t* wq, const uint32_t* sz, const void* bias, void* y, int dtype,
                        int64_t M, int64_t N, int64_t K, int64_t group_size, void* workspace, size_t workspace_bytes,
                        void* stream);

/* The SwiGLU MLP's first projection and its activation in one launch:
 *   act[m, f] = round(silu(round(gate[m, f]))) * round(up[m, f]),   gate | up = x * W^T (+ bias),
 * W = the gate projection's F rows followed by the up projection's F rows (N = 2F, same tiled layout as
 * subspec_int4_linear), every intermediate rounded to the activation dtype exactly where the separate
 * projection and activation would round it.  A workgroup owns (gate tile, up tile) pairs, so the 2F
 * projections never travel through memory.
 *
 * Replaces  act_fn(gate_proj(x)) * up_proj(x) of the decoder MLP (HuggingFace Qwen2MLP / LlamaMLP with
 *           HQQLinear projections; the reference's patched form is LigerSwiGLUMLP.forward,
 *           specdecodes/models/utils/flashinfer/rms_norm.py:43-78, with flashinfer.activation.silu_and_mul).
 *
 * x    device [M, K] bf16 / fp16, 1 <= M <= 64;  act  device [M, N / 2];  N % 32 == 0, K % 64 == 0;
 * bias device [N] or NULL.  No workspace.
 */
int subspec_int4_gate_up_silu(const void* x, const uint32_t* wq, const uint32_t* sz, const void* bias, void* act,
                              int dtype, int64_t M, int64_t N, int64_t K, void* stream);

/* The same for a dense 16-bit gate|up weight W [2F, K] row-major (gate rows first), as the target's layers hold it:
 * 1 <= M <= 384; up to 32 rows 2F * K * 2 bytes must stay below 2 GiB. */
int subspec_dense_gate_up_silu(const void* x, const void* w, const void* bias, void* act, int dtype, int64_t M,
                               int64_t N, int64_t K, void* stream);

/* ------------------------------------------------------------------------------------------
 * One int4 decoder layer of the substitute draft over the rows of a tree level, issued as a fixed
 * sequence of launches from one host call (no per-module Python dispatch):
 *   x += o_proj(attn(rope(qkv_proj(rmsnorm(x)))));  x += down_proj(silu(gate) * up),
 *   gate|up = gate_up_proj(rmsnorm(x)).  K and V of the rows are written into the static cache
 *   at cache_rows before attention; attention is subspec_tree_attention with batch 1.
 *
 * Replaces  one HuggingFace Qwen2 / Llama decoder layer of the draft whose q,k,v,o,gate,up,down
 *           projections are the HQQ int4 linears of
 *           specdecodes/helpers/recipes/subspec/hqq_4bit_postspec.py:17-58, as run per tree level by
 *           specdecodes/models/draft_models/classic_sd.py:85-118 (speculate_once); the reference
 *           removes the per-module launch cost with torch.compile / captured graphs
 *           (specdecodes/models/draft_models/subspec_sd_fi.py:65-179).
 *
 * Projections are fused: qkv = q|k|v rows (N = 4608 at the Qwen2.5-7B shape), gate_up = gate|up rows, all in
 * the tiled int4 layout of subspec_int4_linear.  Rotary embedding is the rotate-half form with
 * angle = position * rope_theta^(-2i / head_dim).
 *
 * x           device [n_rows, hidden], updated in place (the residual stream)
 * positions   device int32 [n_rows]   rotary position of each row (prefix_len + node depth)
 * cache_rows  device int32 [n_rows]   cache row each row's K / V is written to (prefix_len + slot); a row outside
 *             [0, kv_seq_stride) is not written (its K / V are dropped), so a bad tensor cannot leave the cache
 * anc_bits    device uint64 [n_rows, words]  as for subspec_tree_attention (words = ceil(n_tree_slots / 64))
 * k_cache, v_cache  device [n_kv_heads, kv_seq_stride, head_dim] of THIS layer (batch 1)
 * Limits: n_rows <= 64, n_tree_slots <= SUBSPEC_MAX_TREE_NODES, head_dim 128, hidden % 64 == 0 and <= 16384,
 *         intermediate % 64 == 0.
 */
typedef struct subspec_decoder_layer_dims {
  int32_t dtype;            /* SUBSPEC_BF16 or SUBSPEC_F16 */
  int32_t reserved;
  int64_t n_rows, hidden, intermediate, n_q_heads, n_kv_heads, head_dim;
  int64_t kv_seq_stride, prefix_len, n_tree_slots;
  float rms_eps, rope_theta;
  const float* rope_inv_freq; /* device float [head_dim / 2]: the inverse frequencies the caller's other code paths
                                 use (HuggingFace: 1 / theta^(2i / head_dim), evaluated by torch), so that rows written
                                 here and rows written by a prefill are rotated by identical angles; NULL: the kernel
                                 evaluates rope_theta^(-2i / head_dim) itself */
  const int64_t* prefix_len_dev; /* device int64 or NULL.  Not NULL: attention reads the prefix length here when the kernels
                                 run, and prefix_len above is the upper bound the launches are laid out for -- a sequence
                                 of layer calls captured into a HIP graph is replayed while the prefix grows (the
                                 reference captures its draft step the same way, with device-side positions:
                                 specdecodes/models/draft_models/subspec_sd_fi.py:65-179); positions / cache_rows are
                                 device arrays already */
  const int32_t* page_indices; /* NULL: k_cache / v_cache are the layer's contiguous [n_kv_heads, kv_seq_stride, head_dim]
                                 caches.  Not NULL: a paged cache -- k_cache is ONE LAYER of a page pool
                                 [max_pages][2 (K, V)][page_len][n_kv_heads][head_dim], v_cache is ignored, cache row p lives
                                 in page page_indices[p / page_len] at token p % page_len (see subspec_tree_attention_paged),
                                 and kv_seq_stride must be n_pages * page_len (rotary rows are written and attention reads
                                 through the table: flashinfer append_paged_kv_cache + the paged wrapper's run,
                                 specdecodes/models/utils/flashinfer/attention_wrapper.py:244-253,288-316) */
  int64_t n_pages, max_pages, page_len;
} subspec_decoder_layer_dims;

typedef struct subspec_decoder_layer_weights {
  const void* input_norm;   /* [hidden] */
  const void* post_norm;    /* [hidden] */
  const uint32_t* qkv_wq;   /* N = (n_q_heads + 2 n_kv_heads) * head_dim, K = hidden */
  const uint32_t* qkv_sz;
  const void* qkv_bias;     /* [N] or NULL */
  const uint32_t* o_wq;     /* N = hidden, K = n_q_heads * head_dim */
  const uint32_t* o_sz;
  const uint32_t* gate_up_wq; /* N = 2 * intermediate, K = hidden */
  const uint32_t* gate_up_sz;
  const uint32_t* down_wq;  /* N = hidden, K = intermediate */
  const uint32_t* down_sz;
} subspec_decoder_layer_weights;

/* 0 when the dimensions are rejected (subspec_last_error says why) */
size_t subspec_int4_decoder_layer_workspace(const subspec_decoder_layer_dims* dims);

int subspec_int4_decoder_layer(const subspec_decoder_layer_dims* dims, const subspec_decoder_layer_weights* weights,
                               void* x, const int32_t* positions, const int32_t* cache_rows, const uint64_t* anc_bits,
                               void* k_cache, void* v_cache, void* workspace, size_t workspace_bytes, void* stream);

/* ------------------------------------------------------------------------------------------
 * Dense 16-bit linear for the rows of a tree:  y[M, N] = x[M, K] * W[N, K]^T (+ bias), 1 <= M <= 384.
 *
 * Replaces  the nn.Linear projections (q/k/v, o, gate/up, down) of the TARGET model's decoder layers in
 *           the tree-decoding forward: ClassicSDGeneratorBase._tree_decoding -> self.target_model(...)
 *           specdecodes/models/generators/classic_sd.py:75-109 (max_verify_tokens = 64 rows by default,
 *           1 + 48 * 6 = 289 rows in configs/exp_offloading/subspec_sd_qwen_7b.yaml:16-19).
 *
 * x  device [M, K], w  device [N, K] row-major, bias [N] or NULL, y [M, N]: all bf16 or all fp16.
 * N % 16 == 0 (N % 32 == 0 above 64 rows), K % 64 == 0; x and w 16-byte aligned.  Products accumulate in fp32 and
 * are rounded once.
 * workspace  subspec_dense_linear_workspace(M, N, K) bytes (fp32 partials when K is split).
 */
size_t subspec_dense_linear_workspace(int64_t M, int64_t N, int64_t K);

int subspec_dense_linear(const void* x, const void* w, const void* bias, void* y, int dtype, int64_t M, int64_t N,
                         int64_t K, void* workspace, size_t workspace_bytes, void* stream);

/* One decoder layer with dense 16-bit projections: same sequence of kernels, arguments, workspace
 * (subspec_int4_decoder_layer_workspace) and limits as subspec_int4_decoder_layer, for the target
 * model's layers (HF Qwen2DecoderLayer inside the forward named above), except that n_rows may reach 384 (a whole
 * 289-node tree in one call; the projection widths must then be multiples of 32); q|k|v and gate|up rows are
 * stored fused.  Weight matrices are row-major [N, K] in the activation dtype. */
typedef struct subspec_dense_layer_weights {
  const void* input_norm;   /* [hidden] */
  const void* post_norm;    /* [hidden] */
  const void* qkv_w;        /* [(n_q_heads + 2 n_kv_heads) * head_dim, hidden] */
  const void* qkv_bias;     /* [N] or NULL */
  const void* o_w;          /* [hidden, n_q_heads * head_dim] */
  const void* gate_up_w;    /* [2 * intermediate, hidden] */
  const void* down_w;       /* [hidden, intermediate] */
} subspec_dense_layer_weights;

int subspec_dense_decoder_layer(const subspec_decoder_layer_dims* dims, const subspec_dense_layer_weights* weights,
                                void* x, const int32_t* positions, const int32_t* cache_rows, const uint64_t* anc_bits,
                                void* k_cache, void* v_cache, void* workspace, size_t workspace_bytes, void* stream);

/* ------------------------------------------------------------------------------------------
 * RMSNorm of [rows, hidden] activations in one launch: y = weight * round(x * rsqrt(mean(x^2) + eps)), the sum
 * in fp32, the normalized value rounded to the activation dtype before the gain is applied (HuggingFace's
 * Qwen2RMSNorm / LlamaRMSNorm rounding points).  The decoder-layer entry points run the same kernel
 * inside a layer; this is the standalone form for the model's final norm and for module-by-module layers.
 *
 * Replaces  FiLlamaRMSNorm.forward -> flashinfer.norm.rmsnorm
 *           specdecodes/models/utils/flashinfer/rms_norm.py:13-41 (the eager module it patches is the
 *           RMSNorm of the HuggingFace decoder layers).
 *
 * x, y   device [rows, hidden] bf16 / fp16 (y may alias x); weight device [hidden], same dtype;
 *        hidden % 8 == 0 and <= 16384; all pointers 16-byte aligned.
 */
int subspec_rms_norm(const void* x, const void* weight, void* y, int dtype, int64_t rows, int64_t hidden, float eps,
                     void* stream);

/* ------------------------------------------------------------------------------------------
 * Layer streaming: asynchronous copy of one weight slab from pinned host memory to its device
 * slab on the caller's copy stream (hipMemcpyAsync).  Ordering against the compute stream
 * (copy-done before use, last-reader-done before overwrite) is the caller's, with events.
 *
 * Replaces  ChunkedPinMemory / PrefetchOffloader's Tensor.copy_(pinned, non_blocking=True) on a side stream
 *           specdecodes/helpers/offloaders/prefetch_offloader_postspec.py:6-48,174-221 and the
 *           keep_first_n_layers_on_gpu placement of recipes/offload/layer_offload.py:9-56.
 */
int subspec_stream_copy_h2d(void* dst_device, const void* src_pinned_host, size_t bytes, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* SUBSPEC_HIP_H */
