/*
 * C ABI of libareno_hip.so: the MI355X (gfx950) kernels behind AReno's native paged
 * KV-cache attention ops.  Plain pointers and sizes only; every pointer named "device"
 * is a HIP device pointer.  No entry point allocates, synchronises the host or throws:
 * each returns ARENO_OK (0) or a negative ARENO_ERR_* code and records a message that
 * areno_hip_last_error() returns (thread-local).  All launches go to `stream`
 * (a hipStream_t passed as void*; NULL is the null stream) and are legal inside HIP
 * stream capture.
 *
 * Layouts (all contiguous, row-major), as the reference engine allocates them
 * (areno/models/qwen3/model.py:309-333, areno/engine/runtime/metadata.py:29-45):
 *   cache pools   k, v            [num_blocks, block_size, kv_heads, head_dim]   cache_dtype
 *   scale pools   k_scale,v_scale [num_blocks, block_size, kv_heads]             scale_dtype (quantized caches only)
 *   block_table                   [batch, max_blocks]  int32, entries must be valid block ids
 *   cache_seqlens                 [batch]              int32, tokens cached before the step
 */
#ifndef ARENO_HIP_H
#define ARENO_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define ARENO_HIP_ABI_VERSION 1

enum areno_dtype {
  ARENO_DT_F32 = 0,
  ARENO_DT_F16 = 1,
  ARENO_DT_BF16 = 2,
  ARENO_DT_I8 = 3,       /* symmetric int8 codes, per (token, kv head) scale */
  ARENO_DT_FP8_E4M3 = 4  /* OCP e4m3fn codes, per (token, kv head) scale */
};

enum areno_status {
  ARENO_OK = 0,
  ARENO_ERR_INVALID_ARGUMENT = -1, /* null pointer, non-positive size, inconsistent shapes */
  ARENO_ERR_UNSUPPORTED = -2,      /* dtype / head_dim / head-ratio combination with no kernel */
  ARENO_ERR_WORKSPACE = -3,        /* workspace pointer null or too small */
  ARENO_ERR_LAUNCH = -4            /* the HIP runtime refused a launch */
};

/* The paged pools of one layer.  k_scale/v_scale are NULL unless cache_dtype is I8 or FP8_E4M3. */
typedef struct areno_paged_cache {
  void* k;
  void* v;
  void* k_scale;
  void* v_scale;
  int64_t num_blocks;
  int32_t block_size;
  int32_t kv_heads;
  int32_t head_dim;
  int32_t cache_dtype; /* enum areno_dtype */
  int32_t scale_dtype; /* ARENO_DT_F16 or ARENO_DT_F32; ignored for unquantized caches */
} areno_paged_cache;

int areno_hip_abi_version(void);
const char* areno_hip_status_string(int status);
const char* areno_hip_last_error(void);

/*
 * Prefill cache store: cache[block_ids[t], block_offsets[t], h, :] = quantize(k[t, h, :]) (same for v), and the
 * row's scale to scale[block_ids[t], block_offsets[t], h] for quantized caches.
 * Replaces _store_prefill_cache's two index_put_ calls
 * (areno/engine/layers/attention_backend/infer.py:245-263).
 *   k, v          device [tokens, kv_heads, head_dim], in_dtype (must equal cache_dtype for unquantized caches)
 *   block_ids     device [tokens] int64,  block_offsets device [tokens] int64
 * Rows whose (id, offset) fall outside the pool are skipped.
 */
int areno_hip_cache_write(const areno_paged_cache* cache, const void* k, const void* v, int32_t in_dtype,
                          int64_t tokens, const int64_t* block_ids, const int64_t* block_offsets, void* stream);

/*
 * Decode cache append: row b goes to cache[block_table[b, L_b / block_size], L_b % block_size] with
 * L_b = cache_seqlens[b].  Replaces paged_decode_update_kernel (areno/accel/csrc/attention.cu:526-553) and
 * _store_decode_cache (attention_backend/infer.py:266-288); quantizes when the cache is I8 / FP8.
 *   k_update, v_update   device [batch, kv_heads, head_dim], in_dtype
 */
int areno_hip_cache_write_decode(const areno_paged_cache* cache, const void* k_update, const void* v_update,
                                 int32_t in_dtype, int32_t batch, const int32_t* block_table, int32_t max_blocks,
                                 const int32_t* cache_seqlens, void* stream);

/*
 * Bytes of device workspace areno_hip_paged_decode needs for these shapes (split-KV partials).
 * num_splits is the caller's hint (the reference passes 8, attention_backend/infer.py:240): the matrix-core kernel
 * cuts the work by itself whatever the hint; on the vector-ALU kernels 1 forces a single partial per row and anything
 * else lets the library pick the chunking.
 * Returns 0 for invalid shapes.
 */
size_t areno_hip_paged_decode_workspace_bytes(int32_t batch, int32_t q_heads, int32_t head_dim, int32_t block_size,
                                              int32_t max_blocks, int32_t num_splits);

/*
 * Single-token paged causal attention, the whole op of areno_paged_causal_attention_decode_forward_cuda
 * (areno/accel/csrc/attention.cu:926-1020; pybind name areno_paged_causal_attention_decode_forward,
 * areno/accel/csrc/extension.cpp:184):
 *   1. if k_update/v_update are non-NULL, append them (areno_hip_cache_write_decode);
 *   2. split-KV pass over keys [first_allowed, L_b], first_allowed = max(0, L_b - window_left) when
 *      window_left >= 0 else 0; query head h reads kv head h / (q_heads / kv_heads);
 *   3. log-sum-exp merge of the partials, normalise, cast to q_dtype.
 * Same results as those three steps in that order; the launches are two on the matrix-core path: the split pass
 * reads the cached keys [first_allowed, L_b), and the merge launch quantizes the update rows, writes them into
 * their page slots and folds key L_b into the result from the update rows' stored values (what a reader of the page
 * would see).  The other kernels, and 16-bit pages of another dtype than the query's, append in a launch in front.
 * k_update / v_update must not alias the pages they are written to.
 *   q, out        device [batch, q_heads, head_dim], q_dtype (F16/BF16; F32 with an F32 cache)
 *   workspace     device, at least areno_hip_paged_decode_workspace_bytes(...) bytes, 256-byte aligned
 */
int areno_hip_paged_decode(const areno_paged_cache* cache, const void* q, const void* k_update, const void* v_update,
                           void* out, int32_t q_dtype, int32_t batch, int32_t q_heads, const int32_t* block_table,
                           int32_t max_blocks, const int32_t* cache_seqlens, int32_t window_left, int32_t num_splits,
                           float softmax_scale, void* workspace, size_t workspace_bytes, void* stream);

/*
 * The same op with a stage mask, for profilers and benchmarks that time one kernel at a time:
 * ARENO_STAGE_APPEND (cache write of the update rows), ARENO_STAGE_SPLIT (split-KV pass into the workspace),
 * ARENO_STAGE_REDUCE (merge of the workspace partials into `out`).  areno_hip_paged_decode is
 * stages = ARENO_STAGE_ALL.  On the matrix-core path the merge launch is the one that appends: REDUCE with APPEND
 * writes the update rows and counts their key, REDUCE without APPEND counts the key from the update rows and leaves
 * the pages alone (for timing loops that replay a step on an unchanged cache), APPEND without REDUCE runs the
 * stand-alone cache write.  No counterpart in the reference, whose launcher always runs its three kernels
 * (areno/accel/csrc/attention.cu:979-1018).
 */
#define ARENO_STAGE_APPEND 1
#define ARENO_STAGE_SPLIT 2
#define ARENO_STAGE_REDUCE 4
#define ARENO_STAGE_ALL 7
int areno_hip_paged_decode_stages(const areno_paged_cache* cache, const void* q, const void* k_update,
                                  const void* v_update, void* out, int32_t q_dtype, int32_t batch, int32_t q_heads,
                                  const int32_t* block_table, int32_t max_blocks, const int32_t* cache_seqlens,
                                  int32_t window_left, int32_t num_splits, float softmax_scale, void* workspace,
                                  size_t workspace_bytes, int32_t stages, void* stream);

/*
 * areno_hip_paged_decode without a workspace argument, for callers that cannot allocate device memory (code under
 * HIP stream capture, serving loops and harnesses that forbid hipMalloc).  No counterpart in the reference, whose
 * launcher allocates its partials with torch (areno/accel/csrc/attention.cu:974-977).  The split-KV partials live in
 * a buffer built into the library: areno_hip_paged_decode_static_capacity() bytes (64 MiB) of device memory that every
 * GPU the library is used on holds until the process ends.  Shapes whose
 * areno_hip_paged_decode_workspace_bytes(...) exceeds the capacity are refused with ARENO_ERR_WORKSPACE.  The call
 * itself allocates and frees nothing; the first call on a device looks the buffer's address up
 * (hipGetSymbolAddress) and should be made outside stream capture.  All calls on one GPU share the buffer: calls that
 * overlap on one GPU (two streams, two threads) race; calls on one stream do not.  Same arguments, results and error
 * behaviour as areno_hip_paged_decode otherwise.
 */
size_t areno_hip_paged_decode_static_capacity(void);
int areno_hip_paged_decode_static(const areno_paged_cache* cache, const void* q, const void* k_update,
                                  const void* v_update, void* out, int32_t q_dtype, int32_t batch, int32_t q_heads,
                                  const int32_t* block_table, int32_t max_blocks, const int32_t* cache_seqlens,
                                  int32_t window_left, int32_t num_splits, float softmax_scale, void* stream);

/*
 * The decode op for batches whose rows come in prefix groups (the samples of one prompt in an RL rollout share the
 * prompt's pages: identical block ids for the prefix).  Rows [i * group_rows, (i + 1) * group_rows) share the pages
 * of their first shared_lens[i] tokens; the kernel reads those pages once for as many rows as fit side by side in
 * the 16 matrix-core columns (16 / (q_heads / kv_heads)) instead of once per row.  Same results as
 * areno_hip_paged_decode up to the order of the fp32 merges.  No counterpart in the reference, which reads every
 * row's history on its own (areno/accel/csrc/attention.cu:555-654).
 *   shared_lens   device [batch / group_rows] int32; each value is clipped to what every row of the group has cached
 *                 and cut to a multiple of 32 tokens; NULL (or a window, or fewer than two rows side by side) makes
 *                 this areno_hip_paged_decode
 *   workspace     at least areno_hip_paged_decode_grouped_workspace_bytes(...) bytes
 *   stages        ARENO_STAGE_* mask as in areno_hip_paged_decode_stages (ARENO_STAGE_ALL for the op)
 */
size_t areno_hip_paged_decode_grouped_workspace_bytes(int32_t batch, int32_t q_heads, int32_t kv_heads,
                                                      int32_t head_dim, int32_t block_size, int32_t max_blocks,
                                                      int32_t num_splits, int32_t group_rows);
int areno_hip_paged_decode_grouped(const areno_paged_cache* cache, const void* q, const void* k_update,
                                   const void* v_update, void* out, int32_t q_dtype, int32_t batch, int32_t q_heads,
                                   const int32_t* block_table, int32_t max_blocks, const int32_t* cache_seqlens,
                                   int32_t window_left, int32_t num_splits, float softmax_scale, int32_t group_rows,
                                   const int32_t* shared_lens, void* workspace, size_t workspace_bytes,
                                   int32_t stages, void* stream);

/*
 * A per-step plan for the decode op.  block_table and cache_seqlens are the same for every layer of a decode step (the
 * reference builds one InferMeta per step and all layers reuse it: areno/engine/inference.py:935,
 * areno/engine/runtime/decode_graph.py:96,140-178), so the work list the split kernel derives from them -- the item
 * table, the prefix sums of the items' 16-token quanta, where every wave's share starts and the block ids of its
 * first tile -- can be built once per step instead of once per layer.  No counterpart in the reference, whose split
 * kernel uses a fixed chunk per thread block (areno/accel/csrc/attention.cu:588-594).
 *   areno_hip_paged_decode_plan_bytes(batch)   bytes of device memory a plan for `batch` rows needs at most
 *   areno_hip_paged_decode_plan(...)           one small launch on `stream` that fills `buffer` (16-byte aligned, the
 *                                              caller's) and describes it in *plan (host memory, the caller's); legal
 *                                              inside stream capture.  `cache` gives the pool geometry and dtypes (its
 *                                              pointers only have to be aligned like the pools the decode calls will
 *                                              pass); with_update = the decode calls will pass k_update / v_update;
 *                                              group_rows / shared_lens as in areno_hip_paged_decode_grouped (0 / NULL:
 *                                              no prefix groups).
 *   areno_hip_paged_decode_planned(...)        areno_hip_paged_decode_grouped with the plan; plan = NULL or a plan with
 *                                              units == 0 (shapes that a kernel without a work list serves) is exactly
 *                                              that call.  Every argument the plan was built from must be the same
 *                                              (shapes and dtypes are checked: ARENO_ERR_INVALID_ARGUMENT; the contents
 *                                              of block_table, cache_seqlens and shared_lens at the time of the plan
 *                                              launch must still be what the decode call sees).  Same results, bit for
 *                                              bit, as the call without a plan.
 * A plan may be reused by any number of decode calls (the layers of a step) and is rebuilt when the tables change.
 */
typedef struct areno_decode_plan {
  void* buffer; /* device memory the plan's tables live in */
  size_t buffer_bytes;
  int32_t batch, q_heads, kv_heads, head_dim, block_size, max_blocks, window_left;
  int32_t cache_dtype, q_dtype, with_update, group_rows;
  int32_t units;       /* waves that share the work; 0: the shapes take a kernel that uses no plan */
  int32_t items;       /* entries of the item list */
  int32_t tile_tokens; /* tokens per tile step of the kernel the plan is for */
} areno_decode_plan;
size_t areno_hip_paged_decode_plan_bytes(int32_t batch);
int areno_hip_paged_decode_plan(areno_decode_plan* plan, void* buffer, size_t buffer_bytes,
                                const areno_paged_cache* cache, int32_t q_dtype, int32_t batch, int32_t q_heads,
                                const int32_t* block_table, int32_t max_blocks, const int32_t* cache_seqlens,
                                int32_t window_left, int32_t with_update, int32_t group_rows,
                                const int32_t* shared_lens, void* stream);
int areno_hip_paged_decode_planned(const areno_paged_cache* cache, const void* q, const void* k_update,
                                   const void* v_update, void* out, int32_t q_dtype, int32_t batch, int32_t q_heads,
                                   const int32_t* block_table, int32_t max_blocks, const int32_t* cache_seqlens,
                                   int32_t window_left, int32_t num_splits, float softmax_scale, int32_t group_rows,
                                   const int32_t* shared_lens, const areno_decode_plan* plan, void* workspace,
                                   size_t workspace_bytes, int32_t stages, void* stream);

/*
 * Packed causal self-attention over new tokens only, GQA without expanding KV:
 * areno_varlen_causal_attention_forward_cuda (areno/accel/csrc/attention.cu:813-861; pybind name
 * areno_varlen_causal_attention_forward, extension.cpp:182).  Token t of the sequence starting at
 * cu_seqlens[s] sees keys [max(cu_seqlens[s], t - window_left), t] (all of [cu_seqlens[s], t] when window_left < 0).
 *   q, out  device [tokens, q_heads, head_dim];  k, v  device [tokens, kv_heads, head_dim];  all `dtype`
 *   cu_seqlens  device [num_seqs + 1] int32
 *   workspace   device, at least areno_hip_prefill_workspace_bytes(kv_heads, head_dim) bytes (may be NULL for F32)
 */
int areno_hip_varlen_attention(const void* q, const void* k, const void* v, void* out, int32_t dtype, int64_t tokens,
                               int32_t q_heads, int32_t kv_heads, int32_t head_dim, const int32_t* cu_seqlens,
                               int32_t num_seqs, int32_t window_left, float softmax_scale, void* workspace,
                               size_t workspace_bytes, void* stream);

/*
 * Causal prefill of new queries over paged (optionally quantized) KV; the new tokens' K/V must already be in
 * the cache (areno_hip_cache_write).  Query i of sequence s sits at absolute position context_lens[s] + i and sees
 * keys [0, that] (clipped on the left by window_left when >= 0).  No counterpart kernel in the reference (its
 * chunked prefill never re-reads earlier chunks, areno/engine/data/rollout_state.py:121-172); semantics are those of
 * _reference_attention with query_start = context_lens[s] (areno/accel/attention.py:25-41).
 *   q, out        device [tokens, q_heads, head_dim], q_dtype (F16/BF16)
 *   cu_seqlens_q  device [num_seqs + 1] int32;  context_lens device [num_seqs] int32
 *   block_table   device [num_seqs, max_blocks] int32
 *   workspace     device, at least areno_hip_prefill_workspace_bytes(cache->kv_heads, cache->head_dim) bytes
 */
int areno_hip_paged_varlen_prefill(const areno_paged_cache* cache, const void* q, void* out, int32_t q_dtype,
                                   int64_t tokens, int32_t q_heads, int32_t num_seqs, const int32_t* block_table,
                                   int32_t max_blocks, const int32_t* cu_seqlens_q, const int32_t* context_lens,
                                   int32_t window_left, float softmax_scale, void* workspace, size_t workspace_bytes,
                                   void* stream);

/*
 * The step in front of the path, fused into one pass over the projection output: per-head QK RMSNorm
 * (areno/engine/layers/attention.py:90-93; y = dtype(x * rsqrt(mean(x^2) + eps) * w) in fp32,
 * areno/accel/csrc/normalization.cu:34-56), rotary embedding with rotate_half pairing and every product and the sum
 * rounded to the activation dtype (areno/engine/layers/rotary.py:17-52), and the scatter of the new K/V rows into the
 * paged cache (areno/engine/layers/attention_backend/infer.py:245-263) through the quantizer of
 * areno_hip_cache_write, so the pages hold exactly quantize(k_out) and quantize(v).
 *   q, q_out      device [tokens, q_heads, head_dim];  k, v, k_out  device [tokens, kv_heads, head_dim];  all `dtype`
 *                 (F16 / BF16); k_out may be NULL when only the pages are wanted
 *   positions     device [tokens] int64, clamped into [0, max_pos)
 *   cos, sin      device [max_pos, head_dim] float32 (the doubled-frequency tables of RotaryEmbedding)
 *   q_weight, k_weight  device [head_dim] float32, NULL = no norm on that tensor
 *   cache         NULL = no cache write (then block_ids / block_offsets are ignored)
 * head_dim 64, 128, 256 or 512; every tensor 16-byte aligned.  The kernel indexes with 32 bits: a call with more
 * tokens than that allows (2^24, or 2^31 elements of q, k and v together) runs as consecutive launches over token
 * ranges; max_pos * head_dim >= 2^30 or num_blocks * block_size >= 2^32 return ARENO_ERR_UNSUPPORTED.
 */
int areno_hip_qk_norm_rope_cache_write(const areno_paged_cache* cache, const void* q, const void* k, const void* v,
                                       void* q_out, void* k_out, int32_t dtype, int64_t tokens, int32_t q_heads,
                                       int32_t kv_heads, int32_t head_dim, const int64_t* positions, const float* cos,
                                       const float* sin, int32_t max_pos, const float* q_weight,
                                       const float* k_weight, float eps, const int64_t* block_ids,
                                       const int64_t* block_offsets, void* stream);

/*
 * The rotary rows of a step's tokens, prepared once for all layers.  position_ids are the same for every layer of a
 * step (the reference passes one tensor down the stack, areno/engine/layers/attention.py:94-96), and what the fused
 * step above does with them -- fetch the token's cosines and sines, cast them to the activation dtype as the eager
 * ops do (areno/engine/layers/rotary.py:46-52) -- it otherwise repeats for every (token, head) row of every layer.
 * No counterpart in the reference, whose RotaryEmbedding indexes and casts the tables per call.
 *   areno_hip_rope_rows_bytes(tokens, head_dim)   bytes of the rows: tokens * 2 * head_dim floats
 *   areno_hip_rope_rows(...)                      one launch: rows[t] = { dtype(cos[pos_t]) , +-dtype(sin[pos_t]) } as
 *                                                 floats, the sign of rotate_half on the sines (minus for the first
 *                                                 half of the head); positions clamped into [0, max_pos); head_dim a
 *                                                 multiple of 8; rows, cos and sin 16-byte aligned
 *   areno_hip_qk_norm_rope_cache_write_rows(...)  areno_hip_qk_norm_rope_cache_write with rope_rows (for the same
 *                                                 tokens in the same order, built for the same dtype) in place of
 *                                                 positions, cos, sin and max_pos; same results, bit for bit
 */
size_t areno_hip_rope_rows_bytes(int64_t tokens, int32_t head_dim);
int areno_hip_rope_rows(float* rows, const int64_t* positions, const float* cos, const float* sin, int64_t tokens,
                        int32_t head_dim, int32_t max_pos, int32_t dtype, void* stream);
int areno_hip_qk_norm_rope_cache_write_rows(const areno_paged_cache* cache, const void* q, const void* k, const void* v,
                                            void* q_out, void* k_out, int32_t dtype, int64_t tokens, int32_t q_heads,
                                            int32_t kv_heads, int32_t head_dim, const float* rope_rows,
                                            const float* q_weight, const float* k_weight, float eps,
                                            const int64_t* block_ids, const int64_t* block_offsets, void* stream);

/*
 * Bytes of device workspace the two prefill entry points above need (the reference allocates nothing here: its
 * varlen kernel keeps one query row per thread block, areno/accel/csrc/attention.cu:145-242).  The matrix-core
 * kernels cut the work into equal shares of key tiles whatever the length distribution, and a query block cut by a
 * share border leaves its un-normalised partial (running max, sum, accumulator) here for the merge kernel.  The
 * size depends only on the head geometry, not on the batch.  16-byte aligned.
 */
size_t areno_hip_prefill_workspace_bytes(int32_t kv_heads, int32_t head_dim);

/*
 * Device-resident page allocator and block tables.  The reference keeps the free list and the page list of every
 * running sequence as Python lists (areno/engine/data/rollout_state.py:55-56), walks them on the host each step
 * and uploads a freshly built rectangular table (areno/engine/inference.py:561-580).  These entry points keep the
 * same state in device memory and make the same transitions there, in the same order, so a row receives the page
 * ids the reference would hand out for the same sequence of requests.
 *   table       device [max_rows, max_blocks] int32: page ids of a row, valid for its first row_blocks[r] columns
 *   row_blocks  device [max_rows] int32: pages a row owns, 0 = the row is not running
 *   free_ring   device [num_blocks] int32: FIFO of free page ids
 *   state       device [4] int32: ring head, free count, status (enum areno_blocks_status, the worst since init),
 *               index of the first request that was refused or cut short in the call that set the status (-1: none)
 * Requests of one call are served in index order.  The host never needs `state` to issue the next call; it reads it
 * when it wants to know that the pool ran dry (the reference raises "paged KV cache exhausted" at that point).
 */
typedef struct areno_block_tables {
  int32_t* table;
  int32_t* row_blocks;
  int32_t* free_ring;
  int32_t* state;
  int32_t max_rows;
  int32_t max_blocks;
  int32_t num_blocks;
  int32_t block_size;
} areno_block_tables;

enum areno_blocks_status {
  ARENO_BLOCKS_OK = 0,
  ARENO_BLOCKS_EXHAUSTED = 1, /* the free list ran out; the request took what was left, later ones nothing */
  ARENO_BLOCKS_ROW_FULL = 2,  /* a row asked for more than max_blocks pages; it was cut to max_blocks */
  ARENO_BLOCKS_BAD_ROW = 3    /* row index out of range, a row named twice in a reserve call, or a row without pages */
};

enum areno_table_padding {
  ARENO_PAD_LAST_BLOCK = 0,   /* eager tables: rollout_state.py:282-285 */
  ARENO_PAD_SCRATCH_BLOCK = 1 /* captured-graph tables: the scratch page id num_blocks, runtime/decode_graph.py:95 */
};

/* All pages free in id order (rollout_state.py:55), no row running, status OK. */
int areno_hip_block_tables_init(const areno_block_tables* tables, void* stream);

/*
 * Prefill admission (rollout_state.py:128-151): row rows[i] must be able to hold token_counts[i] tokens
 * (cursor + chunk length); missing pages are taken from the head of the free list.  rows device [n] int64, distinct.
 */
int areno_hip_block_tables_reserve(const areno_block_tables* tables, const int64_t* rows, const int32_t* token_counts,
                                   int32_t n, void* stream);

/*
 * ensure_decode_blocks (rollout_state.py:212-225): a running row whose next position next_positions[i] (device
 * [n] int32, the decode op's cache_seqlens) starts a page gets that page; other rows, and negative row indices (the
 * padded rows of a bucketed batch), are left alone.
 */
int areno_hip_block_tables_ensure_decode(const areno_block_tables* tables, const int64_t* rows,
                                         const int32_t* next_positions, int32_t n, void* stream);

/* _free_rollout_rows (inference.py:651-658): the pages of the rows go to the tail of the free list, in row order. */
int areno_hip_block_tables_release(const areno_block_tables* tables, const int64_t* rows, int32_t n, void* stream);

/*
 * _block_table_for_active_rows (inference.py:573-580): out_table device [n, max_blocks] int32, row i = pages of
 * rows[i] right-padded as pad_mode says; a negative rows[i] gives a row of scratch ids (the padded rows of a
 * captured decode batch, runtime/decode_graph.py:163-174).  n <= 65535.
 */
int areno_hip_block_tables_gather(const areno_block_tables* tables, const int64_t* rows, int32_t n, int32_t pad_mode,
                                  int32_t* out_table, void* stream);

/*
 * One decode step's bookkeeping in one call: areno_hip_block_tables_ensure_decode followed by
 * areno_hip_block_tables_gather for the same rows (inference.py:561-580 does the two on the host every step).
 * A row that did not get the page its next position needs (the pool ran dry, or the row is at max_blocks; the status
 * word says which) comes out as a row of scratch ids, so that the decode op's append cannot land in a page that holds
 * live tokens; the caller reads `state` before it trusts that step's outputs (the reference raises before it decodes,
 * rollout_state.py:222-224).
 */
int areno_hip_block_tables_decode_step(const areno_block_tables* tables, const int64_t* rows,
                                       const int32_t* next_positions, int32_t n, int32_t pad_mode, int32_t* out_table,
                                       void* stream);

/*
 * Per packed prefill token t of sequence i (cu_seqlens[i] <= t < cu_seqlens[i + 1], device [n + 1] int32): position
 * cursors[i] + t - cu_seqlens[i], its page id and slot (rollout_state.py:141-149).  out_* device [tokens] int64,
 * the dtype of cache_block_ids / cache_block_offsets / position_ids there; out_positions may be NULL.
 */
int areno_hip_block_tables_prefill_slots(const areno_block_tables* tables, const int64_t* rows,
                                         const int32_t* cursors, const int32_t* cu_seqlens, int32_t n, int64_t tokens,
                                         int64_t* out_block_ids, int64_t* out_block_offsets, int64_t* out_positions,
                                         void* stream);

/*
 * Backward of the causal varlen / dense attention ops: areno_varlen_causal_attention_backward_cuda and
 * areno_causal_attention_backward_cuda (areno/accel/csrc/attention.cu:753-811,862-925), which the reference's
 * autograd functions call (areno/accel/attention.py:104-118,170-183).  Gradients are fp32 and every element is
 * written (no zero-fill needed), as there.
 *   grad_out, q, out  device [q_tokens, q_heads, head_dim];  k, v  device [k_tokens, kv_heads, head_dim];  all `dtype`
 *                     (F32 / F16 / BF16), 16-byte aligned
 *   grad_q            device [q_tokens, q_heads, head_dim] float;  grad_k, grad_v  device [k_tokens, kv_heads, head_dim] float
 *   cu_seqlens_q      device [num_seqs + 1] int32;  cu_seqlens_k  the same for the keys, NULL = cu_seqlens_q (varlen op)
 *   context_lens      device [num_seqs] int32 position of each sequence's first query, NULL = 0 (dense op: query_start)
 *   workspace         areno_hip_attention_backward_workspace_bytes(q_tokens, q_heads) bytes: per-row log-sum-exp and dO . O
 * head_dim a multiple of 8 up to 256 (F16 / BF16 at 64 and 128: matrix-core kernels).  Two launches; deterministic
 * (no atomics).
 */
size_t areno_hip_attention_backward_workspace_bytes(int64_t q_tokens, int32_t q_heads);
int areno_hip_attention_backward(const void* grad_out, const void* q, const void* k, const void* v, const void* out,
                                 float* grad_q, float* grad_k, float* grad_v, int32_t dtype, int64_t q_tokens,
                                 int64_t k_tokens, int32_t q_heads, int32_t kv_heads, int32_t head_dim,
                                 const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k, const int32_t* context_lens,
                                 int32_t num_seqs, int32_t window_left, float softmax_scale, void* workspace,
                                 size_t workspace_bytes, void* stream);
/*
 * The same with the gradients in a type of the caller's choice: grad_dtype = ARENO_DT_F32 (the call above), or
 * = dtype for 16-bit inputs: the fp32 sums are rounded once, at the store, to what the reference's autograd
 * functions produce by casting the fp32 gradients afterwards (areno/accel/attention.py:117-118,182-183) -- without the
 * fp32 tensors and the three cast kernels.  grad_q, grad_k, grad_v: 16-byte aligned.  No counterpart in the
 * reference's extension (there the cast is Python's).
 */
int areno_hip_attention_backward_typed(const void* grad_out, const void* q, const void* k, const void* v, const void* out,
                                       void* grad_q, void* grad_k, void* grad_v, int32_t grad_dtype, int32_t dtype,
                                       int64_t q_tokens, int64_t k_tokens, int32_t q_heads, int32_t kv_heads,
                                       int32_t head_dim, const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k,
                                       const int32_t* context_lens, int32_t num_seqs, int32_t window_left,
                                       float softmax_scale, void* workspace, size_t workspace_bytes, void* stream);

/*
 * ---- Diagnostics: not part of any caller's contract -------------------------------------------------------------------
 * The entry points below have no counterpart in the reference and no production caller: the first exists for a
 * test of this library, the others for its benchmark.
 *
 * areno_hip_debug_set_rope_tokens_per_launch: caps the tokens one launch of areno_hip_qk_norm_rope_cache_write takes
 * (0 = only the kernel's own limit) so that its walk over token ranges can be tested at small sizes.  Returns the
 * previous cap.  Process-wide.
 *
 * areno_hip_probe_stream_read: reads `pages` runs of page_bytes bytes from one pool or from two (page i starts at
 * base + page_ids[i] * page_bytes, or at base + i * page_bytes when page_ids is NULL; base_b NULL = one pool) and
 * computes nothing: 512 workgroups of four waves (two per CU), a wave takes one run at a time with eight 16-byte
 * loads per lane in flight.  prefetch_ids != 0: a wave fetches the id of its next run in front of the current run's
 * loads (as the decode kernel fetches block ids a tile ahead) instead of when it gets there.  What this reaches over
 * the K and V pools of a workload is the streaming ceiling the decode kernels' bandwidth is compared with (bench.py):
 * same pages, same bytes per launch; with page_bytes doubled and one pool it reads what a layout with a block's K and
 * V pages side by side would offer.
 *   base_a, base_b  device, 16-byte aligned;  page_bytes a multiple of 1024;  sink  device, >= 4 bytes (written
 *                   practically never)
 *
 * areno_hip_probe_mfma_rate: 1 024 workgroups of four waves issue `iters` rounds of independent matrix products on
 * register operands and nothing else: shape 0 = 16 x 16 x 32 bf16 (8 products a round), 1 = 32 x 32 x 16 bf16 (4 a
 * round), 2 / 3 the same in f16.  Returns the floating-point operations of the launch (-1 on error); timed by the
 * caller, that is the rate the matrix cores sustain for the shape, which the kernels' rates are compared with
 * (bench.py).  sink as above.
 */
int64_t areno_hip_debug_set_rope_tokens_per_launch(int64_t tokens);
int areno_hip_probe_stream_read(const void* base_a, const void* base_b, const int32_t* page_ids, int64_t pages,
                                int32_t page_bytes, int32_t prefetch_ids, void* sink, void* stream);
int64_t areno_hip_probe_mfma_rate(int32_t shape, int32_t iters, void* sink, void* stream);

#ifdef __cplusplus
}
#endif

#endif /* ARENO_HIP_H */
