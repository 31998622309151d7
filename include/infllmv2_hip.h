/*
 * C ABI of libinfllmv2_hip.so — gfx950 (MI355X) kernels for the InfLLM-V2 two-stage sparse
 * attention path.
 *
 * Every function takes plain device pointers, sizes and a HIP stream handle (passed as void*,
 * null = the default stream), launches asynchronously on that stream, allocates nothing and
 * returns 0 on success.  A non-zero return means nothing was launched by the failing step;
 * infllmv2_last_error() then holds a message (thread-local).  "uint64" masks are the int64
 * tensors of the reference (bit 63 set = negative value).
 *
 * Each declaration cites the interface of the reference (paths relative to the reference
 * checkout) that it replaces.  Where the reference's pybind function takes at::Tensor arguments
 * the tensor is flattened here into pointer + sizes + strides, and outputs/scratch that the
 * reference allocates internally are passed in by the caller.
 *
 * Element types: the entry points below take bfloat16 tensors wherever a 16-bit tensor is meant,
 * unless they have a `dtype` argument; their IEEE-half twins are declared at the end of the file.
 */
#ifndef INFLLMV2_HIP_H
#define INFLLMV2_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define INFLLMV2_ABI_VERSION 11

/* ---- library ------------------------------------------------------------------------------ */

const char* infllmv2_last_error(void);
int infllmv2_abi_version(void);
/* 0 iff `device` is a gfx950 GPU.  Replaces the sm80/sm90 gate of
 * csrc/flash_attn/flash_api.cpp:546-550. */
int infllmv2_check_device(int device);

/* ---- block-mask bit operations -------------------------------------------------------------- */

/* csrc/entry.cu:78-96 `topk_to_uint64` (kernel csrc/topk_to_uint64.cuh:10-76).
 * topk_idx (rows, k) int32, result (rows, n_uint64_per_row); entries < 0 are skipped. */
int infllmv2_topk_to_uint64(void* stream, const int32_t* topk_idx, uint64_t* result, int64_t rows,
                            int k, int k_blocks, int n_uint64_per_row);

/* csrc/entry.cu:98-114 `uint64_to_bool` (kernel csrc/uint64_to_bool.cuh:10-66).
 * result (rows, last_dim_size) bytes of 0/1. */
int infllmv2_uint64_to_bool(void* stream, const uint64_t* input, uint8_t* result, int64_t rows,
                            int last_dim_size, int n_uint64_per_row);

/* csrc/entry.cu:61-76 `blockmask_to_uint64` (kernel csrc/blockmask_to_uint64.cuh:10-74). */
int infllmv2_blockmask_to_uint64(void* stream, const uint8_t* blockmask, uint64_t* result,
                                 int64_t rows, int last_dim_size, int n_uint64_per_row);

/* Replaces the uint64_to_bool -> transpose -> synchronize -> blockmask_to_uint64 sequence of
 * infllm_v2/infllmv2_sparse_attention.py:344-350 with one launch.
 * fwd_mask (heads, total_q, n64_fwd) -> bwd_mask (heads, k_blocks, n64_bwd = ceil(total_q/64)):
 * bwd[h, kb, w] bit u = fwd[h, 64 w + u, kb / 64] bit (kb % 64). */
int infllmv2_transpose_blockmask(void* stream, const uint64_t* fwd_mask, uint64_t* bwd_mask, int heads,
                                 int64_t total_q, int n64_fwd, int k_blocks, int n64_bwd);

/* ---- pooling and selection ------------------------------------------------------------------ */

/* csrc/entry.cu:116-154 `max_pooling_1d` (kernel csrc/max_pooling_1d.cuh:107-160, 203-227).
 * dtype: 0 = fp16, 1 = bf16.  input (num_heads, q_len, k_len), output (num_heads, q_len, out_len). */
int infllmv2_max_pooling_1d(void* stream, const void* input, void* output, int dtype, int num_heads,
                            int q_len, int k_len, int out_len, int cache_len, int kernel_size,
                            int stride, int padding, int block_size, int local_blocks, int init_blocks);

/* Same operator for an input whose rows are not densely packed (strides in elements), so the
 * padded score buffer of Stage 1 is pooled in place instead of being copied first
 * (the reference forces `.contiguous()`, infllm_v2/max_pooling_1d.py:13). */
int infllmv2_max_pooling_1d_strided(void* stream, const void* input, void* output, int dtype,
                                    int num_heads, int q_len, int k_len, int64_t in_head_stride,
                                    int64_t in_row_stride, int out_len, int cache_len, int kernel_size,
                                    int stride, int padding, int block_size, int local_blocks,
                                    int init_blocks);

/* csrc/entry.cu:156-195 `max_pooling_1d_varlen` (kernel csrc/max_pooling_1d.cuh:12-103, 165-199).
 * Like the reference this variant reads cu_seqlens_q[batch_size] back to the host (one stream
 * synchronisation) to learn the number of packed rows. */
int infllmv2_max_pooling_1d_varlen(void* stream, const void* input, void* output,
                                   const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k,
                                   const int32_t* cache_lens, int dtype, int batch_size, int num_heads,
                                   int max_seqlen_q, int max_seqlen_k, int out_len, int kernel_size,
                                   int stride, int padding, int block_size, int local_blocks,
                                   int init_blocks);

/* The same with the packed row count and input strides given by the caller: no host sync. */
int infllmv2_max_pooling_1d_varlen_strided(void* stream, const void* input, void* output,
                                           const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k,
                                           const int32_t* cache_lens, int dtype, int batch_size,
                                           int num_heads, int total_q, int max_seqlen_q,
                                           int max_seqlen_k, int64_t in_head_stride,
                                           int64_t in_row_stride, int out_len, int kernel_size,
                                           int stride, int padding, int block_size, int local_blocks,
                                           int init_blocks);

/* csrc/entry.cu:31-45 `topk` (kernel csrc/topk.cuh:99-181): per row of `dim` values the `top`
 * largest (value descending, equal values by ascending position); output rows have stride
 * top_size = next power of two >= top (csrc/topk.cuh:108,119-141).  Unlike the reference
 * (dim <= 1024, top <= 32) rows up to 8192 and top up to 2048 are accepted. */
int infllmv2_topk(void* stream, int num_tokens, int dim, int top, int dtype, const void* x,
                  void* topk_val, int32_t* topk_pos);

/* Block selection between pooling and packing.  The reference leaves this step to the caller
 * (README.md:42,125-126: torch.topk); its stated order is csrc/topk.cuh:17,26,37.
 * pooled: rows of n 16-bit scores (fp16 or bf16 bits; row stride in elements);
 * topk_idx (rows, k) int32 = first k columns of a stable descending sort, -1 padded. */
int infllmv2_topk_blocks(void* stream, const void* pooled, int64_t row_stride, int32_t* topk_idx,
                         int64_t rows, int n, int k);

/* The same selection with the packing of csrc/topk_to_uint64.cuh:10-52 done by the same wavefronts: mask_words
 * (rows, n_uint64_per_row; null = not wanted) receives bit (c % 64) of word c / 64 for every selected column c,
 * i.e. what infllmv2_topk_to_uint64 computes from topk_idx, so that Stage 2 needs no separate packing launch.
 * dtype 0 = fp16, 1 = bf16.  by_index != 0 writes the selected columns in ascending order instead of value order
 * (the order the reference's callers sort them into, tests/utils.py:124-126; no ordering work).  drop_neg_inf != 0
 * never selects a column whose score is -inf (a block with no visible key: the future of a causal query), so rows
 * with fewer than k reachable blocks are padded with -1 instead. */
int infllmv2_topk_select(void* stream, const void* pooled, int64_t row_stride, int dtype, int32_t* topk_idx,
                         uint64_t* mask_words, int64_t rows, int n, int k, int n_uint64_per_row, int by_index,
                         int drop_neg_inf);

/* ---- Compressed keys (caller-side in the reference) ----------------------------------------- */

/* The Stage-1 inputs are means of K over sliding windows; the reference leaves their construction to its callers,
 * and its tests build them with compress_tensor / calc_chunks_with_stride
 * (tests/test_stage1_compressed_lse.py:16-99): row j of a sequence = mean of K rows [stride*j, stride*j+kernel_size),
 * full windows only.  k (total_k, Hk, d) bf16 with strides {row, head}; out (sum_b L_b, Hk, d) bf16, dense, where
 * L_b = (len_b - kernel_size) / stride + 1 (0 if len_b < kernel_size); cu_seqlens_out (batch + 1) is written by
 * the call.  Rows j < first_row of every sequence are left untouched (first_row > 0 appends to compressed keys
 * built earlier, as a decode loop does every `stride` tokens).  fp32 sum in window order, one rounding. */
int infllmv2_compress_keys(void* stream, const void* k, void* out, const int32_t* cu_seqlens_k,
                           int32_t* cu_seqlens_out, int batch, int max_seqlen_k, int num_heads_k, int head_dim,
                           int64_t k_row_stride, int64_t k_head_stride, int kernel_size, int stride, int first_row);

/* The same means for per-sequence key caches, as a batched decode loop keeps them: kcache (batch, capacity, Hk, d)
 * holds new_lens[b] keys of sequence b, out_cache (batch, rows capacity, Hk, d) its compressed keys; strides
 * {batch, row, head}.  Rows whose windows were completed between old_lens[b] (null: 0) and new_lens[b] tokens are
 * written, at most max_new_rows per sequence (the caller's bound: 1 for a one-token step with kernel_size a multiple
 * of stride); out_lens (batch, or null) receives the number of rows the compressed cache then holds.  kcache_rows and
 * out_rows are the row capacities of one sequence's key cache and compressed cache: a length beyond the key cache is
 * read as its capacity, no row >= out_rows is written, and out_lens never counts a row this call did not cover.  The caller
 * side of the reference does this in Python for one sequence at a time (tests/test_stage1_compressed_lse.py:56-99). */
int infllmv2_compress_keys_cache(void* stream, const void* kcache, void* out_cache, const int32_t* old_lens,
                                 const int32_t* new_lens, int32_t* out_lens, int batch, int max_new_rows,
                                 int num_heads_k, int head_dim, const int64_t* kcache_strides,
                                 const int64_t* out_strides, int kernel_size, int stride, int kcache_rows,
                                 int out_rows);
/* Two compressed caches of the same key cache in one call - the fine (kernel_size_a / stride_a) and the coarse
 * (kernel_size_b / stride_b) keys that Stage 1 reads, which a decode step extends together: the same results as two
 * calls of infllmv2_compress_keys_cache with the same lengths, in one launch when both are appends of a few rows. */
int infllmv2_compress_keys_cache_pair(void* stream, const void* kcache, void* out_cache_a, void* out_cache_b,
                                      const int32_t* old_lens, const int32_t* new_lens, int32_t* out_lens_a,
                                      int32_t* out_lens_b, int batch, int max_new_rows_a, int max_new_rows_b,
                                      int num_heads_k, int head_dim, const int64_t* kcache_strides,
                                      const int64_t* out_strides_a, const int64_t* out_strides_b, int kernel_size_a,
                                      int stride_a, int kernel_size_b, int stride_b, int kcache_rows, int out_rows_a,
                                      int out_rows_b);

/* ---- Stage 1: scoring over compressed keys --------------------------------------------------- */

/* csrc/entry.cu:15,211 `varlen_fwd_stage1` = mha_varlen_fwd_stage1
 * (csrc/flash_attn/flash_api.cpp:784-1049; kernel flash_fwd_kernel.h:1203-1744).
 * q (total_q, Hq, 128) with strides {token, head-in-group, kv-head}; k = fine compressed keys
 * (sum Lk, Hk, 128), v = the key set of the log-sum-exp (sum Lc, Hk, 128), strides {row, head};
 * cu_seqlens_{q,k,v} are cumulative token / Lk / Lc counts.  score (Hk, total_q, row) bf16 with the
 * given head/row strides (row stride >= max_seqlen_k): every column < max_seqlen_k of every row is
 * written (0 where the reference leaves its zero fill or produces NaN that its wrapper zeroes). */
int infllmv2_varlen_fwd_stage1(void* stream, const void* q, const void* k, const void* v, void* score,
                               const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k,
                               const int32_t* cu_seqlens_v, int batch, int64_t total_q, int num_heads,
                               int num_heads_k, int head_dim, int max_seqlen_q, int max_seqlen_k,
                               const int64_t* q_strides, const int64_t* k_strides,
                               const int64_t* v_strides, int64_t score_head_stride,
                               int64_t score_row_stride, float softmax_scale, int is_causal);

/* Stage 1 and the max-pooling onto key blocks in one launch: what infllmv2_max_pooling_1d(_varlen) returns for the
 * score tensor of infllmv2_varlen_fwd_stage1, bit for bit, without that tensor ever reaching memory.  Replaces the
 * caller's pair of calls `infllmv2_attn_stage1` (infllm_v2/infllmv2_sparse_attention.py:483-606) followed by
 * `max_pooling_1d` / `max_pooling_1d_varlen` (infllm_v2/max_pooling_1d.py:4-46, 49-137; csrc/max_pooling_1d.cuh:12-160)
 * for the pooling window those callers use (kernel 5, stride 4, padding 1 on 64-token blocks; anything else is
 * rejected).  q/k/v, cu_seqlens and strides as in infllmv2_varlen_fwd_stage1; cache_lens (batch) or null with one
 * cache_len for all sequences; pooled (Hk, total_q, out_len) bf16, dense. */
int infllmv2_varlen_fwd_stage1_pooled(void* stream, const void* q, const void* k, const void* v, void* pooled,
                                      const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k,
                                      const int32_t* cu_seqlens_v, const int32_t* cache_lens, int cache_len,
                                      int batch, int64_t total_q, int num_heads, int num_heads_k, int head_dim,
                                      int max_seqlen_q, int max_seqlen_k, const int64_t* q_strides,
                                      const int64_t* k_strides, const int64_t* v_strides, int out_len,
                                      float softmax_scale, int is_causal, int kernel_size, int stride, int padding,
                                      int block_size, int local_blocks, int init_blocks);

/* Stage 1 for decode: one query token per sequence, a batch of sequences, each against its own compressed keys.  The
 * reference serves this case with the same `varlen_fwd_stage1` launch (infllm_v2/infllmv2_sparse_attention.py:483-606
 * with cu_seqlens_q = 0, 1, 2, ...; flash_api.cpp:784-1049), one 32-thread block per sequence and KV head; here the
 * compressed keys of every (sequence, KV head) are cut into runs that are scored in parallel (memory-bound), which
 * needs a small workspace for the partial log-sum-exps.
 * q: row b (or row cu_seqlens_q[b] when cu_seqlens_q is given; sequences with no query are skipped), strides
 *   {token, head-in-group, kv-head}.
 * k (fine keys), v (the key set of the log-sum-exp): strides {batch, row, head}; either packed rows with cumulative
 *   lengths (cu_seqlens_k / cu_seqlens_v, batch stride unused) or per-sequence caches (sequence b at b * batch stride)
 *   with k_lens / v_lens (batch) rows each: exactly one of the two pointers per key set.
 * is_causal: 0 = every key is visible (a decode step: all compressed keys lie in the query's past); 1 = the rule of
 *   mask.h:273-281 for a 1-token query (the last key of each set is hidden).
 * pooled == 0: out is the score tensor (Hk, rows, >= max_seqlen_k) with the given head / row strides, every column
 *   < max_seqlen_k of the sequences' rows written.  pooled != 0: out is max_pooling_1d_varlen of those rows
 *   (csrc/max_pooling_1d.cuh:12-103; window 5/4/1 on 64-token blocks only), out_len entries per row, with the query
 *   at position cache_lens[b] (or cache_len for all), bit-identical to pooling the score rows of the same call. */
size_t infllmv2_stage1_decode_workspace_bytes(int batch, int num_heads_k, int max_seqlen_k, int max_seqlen_v);
int infllmv2_stage1_decode(void* stream, const void* q, const void* k, const void* v, void* out,
                           const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k, const int32_t* k_lens,
                           const int32_t* cu_seqlens_v, const int32_t* v_lens, void* workspace,
                           size_t workspace_bytes, int batch, int num_heads, int num_heads_k, int head_dim,
                           int max_seqlen_k, int max_seqlen_v, const int64_t* q_strides, const int64_t* k_strides,
                           const int64_t* v_strides, int64_t out_head_stride, int64_t out_row_stride,
                           float softmax_scale, int is_causal, int pooled, const int32_t* cache_lens, int cache_len,
                           int out_len, int kernel_size, int stride, int padding, int block_size, int local_blocks,
                           int init_blocks);

/* ---- Stage 2: block-sparse attention -------------------------------------------------------- */

/* Scratch needed by infllmv2_varlen_fwd / _bwd for the fragment-major K/V block images. */
size_t infllmv2_kv_image_bytes(int64_t total_k, int batch, int num_heads_k);

/* csrc/entry.cu:14,210 `varlen_fwd` = mha_varlen_fwd (csrc/flash_attn/flash_api.cpp:519-782) on
 * the sparse path (blockmask given) and on the dense path (blockmask null).
 * bf16, head_dim 128, num_heads == g * num_heads_k with g = 16 (the reference build) or 1, 2, 4, 8; the same holds
 * for every entry point that takes num_heads and num_heads_k.
 * q/out: element strides {token, head-in-group, kv-head}; the caller's (T, Hq, d) tensor is
 *   {Hq*d, d, g*d}; the reference's re-laid-out (T*16, Hk, d) tensor is {16*Hk*d, Hk*d, d}.
 * k/v: (total_k, Hk, d), strides {row, head}.  softmax_lse strides {token, head-in-group, kv-head};
 *   the reference's (Hk, T*16) layout (flash_api.cpp:665) is {16, 1, T*16}.
 * blockmask (Hk, total_q, n_uint64_per_row): block indices local to each sequence, rows by packed
 *   token index (flash_blockmask.h:20-31).
 * workspace: infllmv2_kv_image_bytes() bytes, 16-byte aligned; filled here unless kv_prepacked. */
int infllmv2_varlen_fwd(void* stream, const void* q, const void* k, const void* v, void* out,
                        float* softmax_lse, const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k,
                        const uint64_t* blockmask, void* workspace, size_t workspace_bytes,
                        int kv_prepacked, int batch, int64_t total_q, int64_t total_k, int num_heads,
                        int num_heads_k, int head_dim, int max_seqlen_q, int max_seqlen_k,
                        const int64_t* q_strides, const int64_t* k_strides, const int64_t* v_strides,
                        const int64_t* o_strides, const int64_t* lse_strides, int n_uint64_per_row,
                        float softmax_scale, int is_causal);

/* First half of infllmv2_varlen_fwd on its own: rewrites k, v (total_k, Hk, 128; strides {row, head})
 * into the block images in `workspace`.  A later infllmv2_varlen_fwd / _bwd call on the same k, v
 * may then pass kv_prepacked = 1 (k and v are not read).  No counterpart in the reference, whose
 * kernels read K/V in the caller's layout. */
int infllmv2_pack_kv(void* stream, const void* k, const void* v, const int32_t* cu_seqlens_k,
                     void* workspace, size_t workspace_bytes, int batch, int64_t total_k,
                     int num_heads_k, int head_dim, int max_seqlen_k, const int64_t* k_strides,
                     const int64_t* v_strides);

/* Scratch for infllmv2_varlen_bwd: the K/V block images, the transposed mask, D = rowsum(dO*O),
 * transposed per-token images of q and dout, fp32 dK/dV accumulators. */
size_t infllmv2_varlen_bwd_workspace_bytes(int batch, int64_t total_q, int64_t total_k, int num_heads_k,
                                           int max_seqlen_k);
/* The same plus the slots of the deterministic mode of infllmv2_varlen_bwd (one 64 KiB slot per KV head, key block
 * and 512-token slice of the packed query axis: 4.4 GB at 32768 tokens, growing with the square of the length). */
size_t infllmv2_varlen_bwd_deterministic_workspace_bytes(int batch, int64_t total_q, int64_t total_k, int num_heads_k,
                                                         int max_seqlen_k);
/* csrc/entry.cu:17,213 `varlen_bwd` = mha_varlen_bwd (csrc/flash_attn/flash_api.cpp:1278-1547; kernels
 * flash_bwd_kernel.h:80-856, flash_bwd_preprocess_kernel.h:56-137,181-263) together with the mask
 * transposition the reference does in Python (infllmv2_sparse_attention.py:344-350): it takes the
 * FORWARD mask (Hk, total_q, n_uint64_per_row), or null for dense attention.
 * dout, q, out, dq: strides {token, head-in-group, kv-head} as in infllmv2_varlen_fwd; k, v, dk, dv:
 * {row, head}; softmax_lse: the forward's output with its strides.  dq, dk, dv are fully written
 * (bf16).  workspace: infllmv2_varlen_bwd_workspace_bytes() bytes, 256-byte aligned.  dQ is always
 * bit-reproducible.  dK/dV are accumulated with fp32 atomics (one flush per 64-key block and slice of 512 query tokens, 128 when total_q <= 8192),
 * so their last bits can differ between runs, unless `deterministic` is set (the flag of flash_api.cpp:1448-1453,
 * which there concerns dQ): then every work item stores its tiles in a slot of its own and a second kernel adds them
 * in a fixed order; the workspace must then hold infllmv2_varlen_bwd_deterministic_workspace_bytes() bytes. */
int infllmv2_varlen_bwd(void* stream, const void* dout, const void* q, const void* k, const void* v,
                        const void* out, const float* softmax_lse, void* dq, void* dk, void* dv,
                        const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k,
                        const uint64_t* fwd_blockmask, void* workspace, size_t workspace_bytes, int batch,
                        int64_t total_q, int64_t total_k, int num_heads, int num_heads_k, int head_dim,
                        int max_seqlen_q, int max_seqlen_k, const int64_t* q_strides,
                        const int64_t* k_strides, const int64_t* v_strides, const int64_t* o_strides,
                        const int64_t* do_strides, const int64_t* dq_strides, const int64_t* dk_strides,
                        const int64_t* dv_strides, const int64_t* lse_strides, int n_uint64_per_row,
                        float softmax_scale, int is_causal, int deterministic);

/* ---- Stage 2: decode against a KV cache -------------------------------------------------------- */

/* The split count infllmv2_fwd_kvcache will use: `requested` if > 0 (capped at 64), else a heuristic
 * (replaces num_splits_heuristic, csrc/flash_attn/flash_api.cpp:261-295). */
int infllmv2_fwd_kvcache_num_splits(int batch, int num_heads_k, int requested);
/* fp32 partial outputs and LSEs of the splits, plus room for the query turned by the rotary embedding. */
size_t infllmv2_fwd_kvcache_workspace_bytes(int batch, int num_heads_k, int num_splits);

/* csrc/entry.cu:18,214 `fwd_kvcache` = mha_fwd_kvcache (csrc/flash_attn/flash_api.cpp:1549-1843; kernels
 * flash_fwd_kernel.h:606-1199 and 1794-1975) for seqlen_q == 1.
 * q, out (batch, 1, Hq, 128): strides {batch, head}.  kcache, vcache (cache_batch, capacity, Hk, 128),
 * k_new, v_new (batch, seqlen_new, Hk, 128) or null: strides {batch, row, head}.  cache_seqlens (batch) int32
 * or null (= capacity).  New rows are written at cache rows cache_seqlens[b] + t first, then attention runs
 * over the sequence's keys restricted to the blocks set in blockmask (batch, Hk, n_uint64_per_row), or all
 * blocks when it is null.  softmax_lse (batch, Hq) fp32.  num_splits >= 1 as returned by
 * infllmv2_fwd_kvcache_num_splits.  Options, each null / 0 when unused:
 *  - cache_batch_idx (batch) int32: sequence b lives in cache row cache_batch_idx[b] (flash_api.cpp:1800-1808);
 *  - cache_leftpad (batch) int32: the sequence's keys are cache rows [leftpad[b], cache_seqlens[b] + seqlen_new)
 *    and mask block j covers the 64 keys from row leftpad[b] + 64 j (flash_api.cpp:1762-1771, block_info.h:23-43);
 *  - block_table (batch, pages per sequence) int32 with its batch stride, page_block_size: kcache/vcache are
 *    (pages, page_block_size, Hk, 128), cache_capacity = pages per sequence x page_block_size, row r of sequence b
 *    is row r % page_block_size of page block_table[b][r / page_block_size] (flash_api.cpp:1593-1611;
 *    flash_fwd_kernel.h:696-712); the page size must be a multiple of 64 (the reference asks for 256); not
 *    together with cache_batch_idx or cache_leftpad, as in the reference;
 *  - rotary_cos, rotary_sin (seqlen_ro >= capacity, rotary_dim / 2) bf16, dense: the appended keys are turned at
 *    their cache rows and the query at cache_seqlens[b] before use, interleaved pairs (2i, 2i+1) or contiguous
 *    pairs (i, i + rotary_dim / 2) (flash_api.cpp:1773-1798; flash_fwd_kernel.h:787-929; rotary.h); needs k_new. */
int infllmv2_fwd_kvcache(void* stream, const void* q, void* kcache, void* vcache, const void* k_new,
                         const void* v_new, const int32_t* cache_seqlens, void* out, float* softmax_lse,
                         const uint64_t* blockmask, void* workspace, size_t workspace_bytes, int batch,
                         int seqlen_q, int num_heads, int num_heads_k, int head_dim, int cache_capacity,
                         int seqlen_new, const int64_t* q_strides, const int64_t* kcache_strides,
                         const int64_t* vcache_strides, const int64_t* knew_strides,
                         const int64_t* vnew_strides, const int64_t* o_strides, int n_uint64_per_row,
                         int num_splits, float softmax_scale, const int32_t* cache_batch_idx,
                         const int32_t* cache_leftpad, const int32_t* block_table,
                         int64_t block_table_batch_stride, int page_block_size, const void* rotary_cos,
                         const void* rotary_sin, int rotary_dim, int rotary_interleaved);

/* No counterpart in the reference.  infllmv2_fwd_kvcache for callers that cannot allocate device memory (code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc): the same kernels and arguments, without
 * the workspace pair.  The split partials and the turned query go to a buffer of INFLLMV2_STATIC_SCRATCH_BYTES that is
 * part of the library's device code (one copy per GPU, held until the process ends); the call allocates and frees
 * nothing.  Sizes with infllmv2_fwd_kvcache_workspace_bytes(batch, num_heads_k, num_splits) above that limit are
 * rejected.  All calls on one GPU share the buffer: calls that overlap on one GPU (different streams or threads) race;
 * the buffer needs no clearing between calls (every element read has been written by the same call). */
#define INFLLMV2_STATIC_SCRATCH_BYTES (32u << 20)
int infllmv2_fwd_kvcache_static(void* stream, const void* q, void* kcache, void* vcache, const void* k_new,
                                const void* v_new, const int32_t* cache_seqlens, void* out, float* softmax_lse,
                                const uint64_t* blockmask, int batch, int seqlen_q, int num_heads, int num_heads_k,
                                int head_dim, int cache_capacity, int seqlen_new, const int64_t* q_strides,
                                const int64_t* kcache_strides, const int64_t* vcache_strides,
                                const int64_t* knew_strides, const int64_t* vnew_strides, const int64_t* o_strides,
                                int n_uint64_per_row, int num_splits, float softmax_scale,
                                const int32_t* cache_batch_idx, const int32_t* cache_leftpad,
                                const int32_t* block_table, int64_t block_table_batch_stride, int page_block_size,
                                const void* rotary_cos, const void* rotary_sin, int rotary_dim,
                                int rotary_interleaved);

/* ---- IEEE half (fp16) twins ---------------------------------------------------------------------
 *
 * The reference switches between half and bfloat16 on the tensors' dtype (csrc/entry.cu:20-29; its build
 * instantiates bfloat16 only).  Here every entry point that reads or writes attention tensors exists once per element
 * type: the plain name takes bfloat16, the name with the suffix _f16 takes IEEE half, with the same arguments, the
 * same semantics and the same workspace sizes (both types are two bytes wide; infllmv2_pack_kv, infllmv2_kv_image_bytes
 * and the other size queries serve both).  All 16-bit tensors of one call have the one element type: q, k, v, out,
 * dout, dq, dk, dv, caches, compressed keys, scores, rotary tables.  fp32 accumulation, one rounding of P, dS and of
 * each output to the element type, as for bfloat16.  Pooling, top-k and the mask operations take their element type
 * as an argument or have none.  infllmv2_fwd_kvcache_static has no fp16 twin. */
int infllmv2_compress_keys_f16(void* stream, const void* k, void* out, const int32_t* cu_seqlens_k,
                               int32_t* cu_seqlens_out, int batch, int max_seqlen_k, int num_heads_k, int head_dim,
                               int64_t k_row_stride, int64_t k_head_stride, int kernel_size, int stride, int first_row);
int infllmv2_compress_keys_cache_f16(void* stream, const void* kcache, void* out_cache, const int32_t* old_lens,
                                     const int32_t* new_lens, int32_t* out_lens, int batch, int max_new_rows,
                                     int num_heads_k, int head_dim, const int64_t* kcache_strides,
                                     const int64_t* out_strides, int kernel_size, int stride, int kcache_rows,
                                     int out_rows);
int infllmv2_compress_keys_cache_pair_f16(void* stream, const void* kcache, void* out_cache_a, void* out_cache_b,
                                          const int32_t* old_lens, const int32_t* new_lens, int32_t* out_lens_a,
                                          int32_t* out_lens_b, int batch, int max_new_rows_a, int max_new_rows_b,
                                          int num_heads_k, int head_dim, const int64_t* kcache_strides,
                                          const int64_t* out_strides_a, const int64_t* out_strides_b,
                                          int kernel_size_a, int stride_a, int kernel_size_b, int stride_b,
                                          int kcache_rows, int out_rows_a, int out_rows_b);
int infllmv2_varlen_fwd_stage1_f16(void* stream, const void* q, const void* k, const void* v, void* score,
                                   const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k,
                                   const int32_t* cu_seqlens_v, int batch, int64_t total_q, int num_heads,
                                   int num_heads_k, int head_dim, int max_seqlen_q, int max_seqlen_k,
                                   const int64_t* q_strides, const int64_t* k_strides,
                                   const int64_t* v_strides, int64_t score_head_stride,
                                   int64_t score_row_stride, float softmax_scale, int is_causal);
int infllmv2_varlen_fwd_stage1_pooled_f16(void* stream, const void* q, const void* k, const void* v, void* pooled,
                                          const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k,
                                          const int32_t* cu_seqlens_v, const int32_t* cache_lens, int cache_len,
                                          int batch, int64_t total_q, int num_heads, int num_heads_k, int head_dim,
                                          int max_seqlen_q, int max_seqlen_k, const int64_t* q_strides,
                                          const int64_t* k_strides, const int64_t* v_strides, int out_len,
                                          float softmax_scale, int is_causal, int kernel_size, int stride, int padding,
                                          int block_size, int local_blocks, int init_blocks);
int infllmv2_stage1_decode_f16(void* stream, const void* q, const void* k, const void* v, void* out,
                               const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k, const int32_t* k_lens,
                               const int32_t* cu_seqlens_v, const int32_t* v_lens, void* workspace,
                               size_t workspace_bytes, int batch, int num_heads, int num_heads_k, int head_dim,
                               int max_seqlen_k, int max_seqlen_v, const int64_t* q_strides, const int64_t* k_strides,
                               const int64_t* v_strides, int64_t out_head_stride, int64_t out_row_stride,
                               float softmax_scale, int is_causal, int pooled, const int32_t* cache_lens, int cache_len,
                               int out_len, int kernel_size, int stride, int padding, int block_size, int local_blocks,
                               int init_blocks);
int infllmv2_varlen_fwd_f16(void* stream, const void* q, const void* k, const void* v, void* out,
                            float* softmax_lse, const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k,
                            const uint64_t* blockmask, void* workspace, size_t workspace_bytes,
                            int kv_prepacked, int batch, int64_t total_q, int64_t total_k, int num_heads,
                            int num_heads_k, int head_dim, int max_seqlen_q, int max_seqlen_k,
                            const int64_t* q_strides, const int64_t* k_strides, const int64_t* v_strides,
                            const int64_t* o_strides, const int64_t* lse_strides, int n_uint64_per_row,
                            float softmax_scale, int is_causal);
int infllmv2_varlen_bwd_f16(void* stream, const void* dout, const void* q, const void* k, const void* v,
                            const void* out, const float* softmax_lse, void* dq, void* dk, void* dv,
                            const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k,
                            const uint64_t* fwd_blockmask, void* workspace, size_t workspace_bytes, int batch,
                            int64_t total_q, int64_t total_k, int num_heads, int num_heads_k, int head_dim,
                            int max_seqlen_q, int max_seqlen_k, const int64_t* q_strides,
                            const int64_t* k_strides, const int64_t* v_strides, const int64_t* o_strides,
                            const int64_t* do_strides, const int64_t* dq_strides, const int64_t* dk_strides,
                            const int64_t* dv_strides, const int64_t* lse_strides, int n_uint64_per_row,
                            float softmax_scale, int is_causal, int deterministic);
int infllmv2_fwd_kvcache_f16(void* stream, const void* q, void* kcache, void* vcache, const void* k_new,
                             const void* v_new, const int32_t* cache_seqlens, void* out, float* softmax_lse,
                             const uint64_t* blockmask, void* workspace, size_t workspace_bytes, int batch,
                             int seqlen_q, int num_heads, int num_heads_k, int head_dim, int cache_capacity,
                             int seqlen_new, const int64_t* q_strides, const int64_t* kcache_strides,
                             const int64_t* vcache_strides, const int64_t* knew_strides,
                             const int64_t* vnew_strides, const int64_t* o_strides, int n_uint64_per_row,
                             int num_splits, float softmax_scale, const int32_t* cache_batch_idx,
                             const int32_t* cache_leftpad, const int32_t* block_table,
                             int64_t block_table_batch_stride, int page_block_size, const void* rotary_cos,
                             const void* rotary_sin, int rotary_dim, int rotary_interleaved);

#ifdef __cplusplus
}
#endif
#endif /* INFLLMV2_HIP_H */
