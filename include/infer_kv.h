/* infer_kv.h - C ABI of libinfer_kv.so: the paged KV-cache hot path on MI355X (gfx950).
 *
 * Three pieces, one library:
 *   1. KV append         - slot_mapping-driven scatter of new K/V rows into the paged caches.
 *   2. Paged decode attn - block_table-gathered GQA attention of one query token per sequence.
 *   3. Block pool        - host-side allocator of cache blocks with a prefix cache.
 *
 * Conventions for every device entry point:
 *   - all pointers are device pointers unless the name says "host"; they are borrowed for the
 *     duration of the call on `stream` (a hipStream_t passed as void*; NULL = default stream);
 *   - the call only enqueues work: it never synchronises, never allocates, never frees, and
 *     never throws; it is safe to record into a HIP graph;
 *   - return value: 0 on success, a negative INFER_KV_E* code for a rejected argument, or a
 *     positive hipError_t reported by the launch;
 *   - element type is bfloat16 (the only type the reference instantiates: src/kvcache.cc:305),
 *     strides are in ELEMENTS, metadata is int32.
 *
 * The reference has no FFI of its own for this path: the append is a Triton kernel and the
 * attention is the pip package flash_attn, both called from Python.  Each declaration below
 * cites the reference call it replaces (paths into the reference tree).
 */
#ifndef INFER_KV_H
#define INFER_KV_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define INFER_KV_OK            0
#define INFER_KV_EINVAL       -1   /* null pointer, non-positive size, unsupported shape        */
#define INFER_KV_EALIGN       -2   /* pointer or stride not aligned for the vector path         */
#define INFER_KV_EWORKSPACE   -3   /* workspace too small                                       */
#define INFER_KV_EUNSUPPORTED -4   /* head_dim / group size / block size outside what is built  */
#define INFER_KV_ESTATE       -5   /* block pool: the call violates an invariant the reference
                                      asserts (double allocate, out of blocks, ...); see
                                      infer_pool_last_error()                                   */
#define INFER_KV_EBUSY        -7   /* the library's own scratch array is still in use by work
                                      pending on another stream (infer_paged_decode_noalloc_bf16) */
#define INFER_KV_ENOTINIT     -6   /* first decode call on this device made while its stream is
                                      being captured: call infer_kv_init() before the capture    */

/* Library version, "major.minor". */
const char* infer_kv_version(void);

/* Human-readable text for a code returned by any entry point (negative codes: this library;
 * positive: hipGetErrorString). */
const char* infer_kv_strerror(int code);

/* One-time set-up for the CURRENT device (host only, no stream work): the decode kernels' LDS limit
 * (hipFuncSetAttribute), the compute-unit count and the address of the library's own scratch array
 * (hipGetSymbolAddress).  Every decode entry point does the same on its first call on a device, but
 * not while its stream is being captured (INFER_KV_ENOTINIT then): a caller that captures HIP graphs
 * calls this once per device beforehand.  Thread safe; later calls return at once. */
int infer_kv_init(void);

/* ------------------------------------------------------------------ 1. KV append
 * Replaces store_kvcache / store_kvcache_kernel (infer/ops/attention.py:16-45), called from
 * Attention.forward_offical_fa_impl (infer/ops/attention.py:108-109).
 *
 * For every row i in [0, n_rows): slot = slot_mapping[i]; if 0 <= slot < num_slots then
 *   k_cache[slot * dkv .. +dkv) = key[i * key_stride0 .. +dkv)   (same for value -> v_cache).
 * Rows whose slot is negative (padding) or >= num_slots are skipped; the reference has no such
 * guard (a -1 slot writes out of bounds there).  dkv = num_kv_heads * head_dim; the caches are
 * [num_slots, dkv] row-major (the reference asserts k_cache.stride(1) == dkv).  key/value rows
 * may be strided views of a fused qkv projection (row stride != dkv) but each row is contiguous.
 * Duplicate slots in one call race (last writer unspecified), as in the reference.
 * Requires dkv % 8 == 0 and 16-byte aligned rows (pointers and strides), else INFER_KV_EALIGN.
 */
int infer_kv_append_bf16(const void* key, int64_t key_stride0,
                         const void* value, int64_t value_stride0,
                         void* k_cache, void* v_cache,
                         const int32_t* slot_mapping,
                         int64_t n_rows, int64_t dkv, int64_t num_slots,
                         void* stream);

/* The dense per-sequence view that the getters of the reference's cache pool promise (Tensor<T>
 * get_key_cache / get_value_cache, include/kvcache.hpp:47-48: [len, heads, head_size] contiguous): tokens
 * 0 .. num_tokens-1 of ONE sequence gathered from the paged cache [num_blocks, block_size, dkv] through its
 * block-table row (device memory, ceil(num_tokens / block_size) entries, clamped into [0, num_blocks)) into
 * out [num_tokens, dkv].  The attention kernels never need it (they gather on the fly); it serves callers
 * that want a sequence's K or V as one tensor, and is the inverse of the append (bit-exact copy).
 * Requires dkv % 8 == 0 and 16-byte aligned pointers. */
int infer_kv_gather_bf16(const void* cache, const int32_t* block_table_row,
                         int64_t num_tokens, int64_t dkv, int64_t block_size, int64_t num_blocks,
                         void* out, void* stream);

/* ------------------------------------------------------------------ 1b. fused QK-norm + RoPE + KV append
 * Replaces, in one launch, the four steps in front of attention in QwenAttention.forward
 * (infer/models/Qwen3.py:113-131): q_norm and k_norm (RMSNorm.rms_forward, infer/ops/norm.py:63-73,
 * per head over head_dim with a [head_dim] bf16 weight), the in-place neox rotary embedding
 * (rotary_embedding_kernel, src/operators/rope/rope.cu:43-133; rot_dim == head_dim) and
 * store_kvcache (infer/ops/attention.py:16-45).
 *
 * q [n_rows, Hq, D] and k [n_rows, Hkv, D] (row strides in elements, heads contiguous) are
 * normalised and rotated; q is updated in place; the new k row goes to k_cache[slot] and, when
 * write_k_inplace != 0, also back into k; the v row is copied to v_cache[slot].  Rows whose slot is
 * negative or >= num_slots update q (and k in place) only.  positions are int64 and are clamped
 * into [0, max_position); cos_sin_cache is [max_position, D] bf16 = cos(D/2) | sin(D/2) per row.
 * Arithmetic rounds where the reference rounds (see the kernel source).  head_dim must be 128.
 */
int infer_kv_qk_norm_rope_append_bf16(void* q, int64_t q_stride0, void* k, int64_t k_stride0,
                                      const void* v, int64_t v_stride0,
                                      const int64_t* positions,
                                      const void* q_norm_weight, const void* k_norm_weight, float eps,
                                      const void* cos_sin_cache, int64_t max_position,
                                      void* k_cache, void* v_cache, const int32_t* slot_mapping,
                                      int64_t n_rows, int64_t num_q_heads, int64_t num_kv_heads,
                                      int64_t head_dim, int64_t num_slots,
                                      int write_k_inplace, void* stream);

/* ------------------------------------------------------------------ 2. paged decode attention
 * Replaces flash_attn_with_kvcache(q[B,1,Hq,D], k_cache, v_cache, cache_seqlens=context_lens,
 * block_table=block_tables, softmax_scale=scale, causal=True) at infer/ops/attention.py:118-120,
 * and is the body the stub src/operators/flashattn/flashattn_decode.cu:11-13 never got.
 *
 *   out[b, h, :] = softmax_t( scale * q[b, h, :] . K_b[t, h / G, :] ) V_b[t, h / G, :],
 *   t in [0, context_lens[b]),  G = num_q_heads / num_kv_heads,
 *   K_b[t] = k_cache[block_table[b, t / block_size], t % block_size]   (same for V).
 *
 * Rows with context_lens[b] <= 0 (graph padding) write zeros.  Table entries past
 * ceil(len / block_size) are never read; entries that are read are clamped into
 * [0, num_blocks) so a corrupt table cannot fault the GPU, and a length beyond what a table row can
 * address (table_cols * block_size) is cut to that, so a corrupt length cannot make the gather run
 * past its row.
 *
 * Layouts (strides in elements): q [B, Hq, D] with row stride q_stride0, heads contiguous;
 * out likewise with out_stride0; caches [num_blocks, block_size, Hkv, D] with block stride
 * cache_block_stride and token stride cache_token_stride (heads contiguous, D innermost);
 * block_table [B, table_cols] with row stride bt_stride0 >= table_cols; context_lens [B].
 *
 * The work is cut into equal shares of KV tokens regardless of sequence boundaries, one share per
 * wavefront.  Partial (max, sum, accumulator) results of one sequence that meet inside a workgroup are
 * folded there and go to `workspace` as one record; a second small kernel folds the records of a
 * sequence that reaches into neighbouring workgroups and writes the result.  Size the workspace with
 * infer_paged_decode_workspace_bytes() for the largest batch that will be passed; its contents need
 * no initialisation.  Calls that share a workspace must be ordered on one stream (the records of one
 * call are live until its merge kernel has run); calls on different streams need a workspace each.
 *
 * split_workgroups: span positions (workgroups per group of KV heads along the token axis) of this
 * call, 0 = choose from the device's compute-unit count (the tuned default), at most 1024.  The
 * library keeps no state between calls: two calls may use different counts, also concurrently.
 *
 * Built for head_dim == 128, 1 <= G <= 16, block_size % 32 == 0 (the reference requires a
 * multiple of 256: infer/config.py:21).
 */
size_t infer_paged_decode_workspace_bytes(int64_t max_batch, int64_t num_q_heads,
                                          int64_t num_kv_heads, int64_t head_dim);

int infer_paged_decode_bf16(const void* q, int64_t q_stride0,
                            const void* k_cache, const void* v_cache,
                            int64_t cache_block_stride, int64_t cache_token_stride,
                            void* out, int64_t out_stride0,
                            const int32_t* block_table, int64_t bt_stride0, int64_t table_cols,
                            const int32_t* context_lens,
                            int64_t batch, int64_t num_q_heads, int64_t num_kv_heads,
                            int64_t head_dim, int64_t block_size, int64_t num_blocks,
                            float scale, int64_t split_workgroups,
                            void* workspace, size_t workspace_bytes,
                            void* stream);

/* The two phases of infer_paged_decode_bf16 on their own: `split` streams the KV cache and leaves
 * partial results in the workspace, `merge` combines them into `out`.  Calling split then merge
 * on one stream is exactly infer_paged_decode_bf16.  They serve callers that want the partial results
 * themselves (a context-parallel split across devices would exchange exactly these records) and
 * profilers that time the bandwidth-bound phase alone.  The merge finds the records from the
 * workspace alone, so it does not need to know the split count. */
int infer_paged_decode_split_bf16(const void* q, int64_t q_stride0,
                                  const void* k_cache, const void* v_cache,
                                  int64_t cache_block_stride, int64_t cache_token_stride,
                                  const int32_t* block_table, int64_t bt_stride0, int64_t table_cols,
                                  const int32_t* context_lens,
                                  int64_t batch, int64_t num_q_heads, int64_t num_kv_heads,
                                  int64_t head_dim, int64_t block_size, int64_t num_blocks,
                                  float scale, int64_t split_workgroups,
                                  void* workspace, size_t workspace_bytes,
                                  void* stream);

int infer_paged_decode_merge_bf16(void* out, int64_t out_stride0,
                                  const int32_t* context_lens,
                                  int64_t batch, int64_t num_q_heads, int64_t num_kv_heads,
                                  int64_t head_dim,
                                  const void* workspace, size_t workspace_bytes,
                                  void* stream);

/* The decode call with the context length given as ONE host integer for the whole batch, the
 * `cache_seqlens: int` form of flash_attn_with_kvcache (the function called at
 * infer/ops/attention.py:118-120; the reference itself passes the per-sequence tensor, so this form is
 * NOT on the reference's call path).  Same result as infer_paged_decode_bf16 with
 * context_lens[b] == context_len for every b; context_len == 0 gives zeros.  Knowing the length, the
 * host can tell whether every sequence lies inside the spans of one workgroup (batch 64 x 512 ... 4096
 * tokens on 256 compute units do): the workgroups then write the result themselves and there is no
 * merge launch; other shapes run the two kernels of infer_paged_decode_bf16 without reading a lengths
 * array.  The workspace is the one of infer_paged_decode_bf16 (used by the second case). */
int infer_paged_decode_uniform_bf16(const void* q, int64_t q_stride0,
                                    const void* k_cache, const void* v_cache,
                                    int64_t cache_block_stride, int64_t cache_token_stride,
                                    void* out, int64_t out_stride0,
                                    const int32_t* block_table, int64_t bt_stride0, int64_t table_cols,
                                    int64_t context_len,
                                    int64_t batch, int64_t num_q_heads, int64_t num_kv_heads,
                                    int64_t head_dim, int64_t block_size, int64_t num_blocks,
                                    float scale,
                                    void* workspace, size_t workspace_bytes,
                                    void* stream);

/* infer_paged_decode_bf16 for callers that cannot allocate and have no workspace to bring: code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart in
 * the reference.  Same arguments, result and kernels as infer_paged_decode_bf16 with
 * split_workgroups = 0, but the split-KV records go to a fixed array in the library's device image
 * (16 MiB per GPU the library runs on, held by every process that loads the library until it ends,
 * whether or not this entry is called) instead of a workspace.  The call allocates nothing and frees
 * nothing.  Shapes whose records do not fit return INFER_KV_EWORKSPACE: the need is about
 * Hkv * (CUs * 4 / Hkv + batch) * 520 * G bytes, i.e. 3.2 MB at batch 64, Hq/Hkv = 32/8 and 4.5 MB at
 * batch 8, 64/8 on 256 compute units, against the INFER_KV_DECODE_NOALLOC_SCRATCH_BYTES of the array.
 * The array keeps the last call's contents and needs no clearing (every record that is read was
 * written by the same call).  All calls on one GPU share it: calls ordered on one stream are safe; a
 * call on another stream than the previous one is refused with INFER_KV_EBUSY while that stream still
 * has work pending (a cheap host-side check; calls racing on two host threads, and a capture that will
 * be replayed beside other users of the array, remain the caller's to order).  The address of the array is
 * resolved by infer_kv_init() or by the first decode call on the device outside stream capture. */
#define INFER_KV_DECODE_NOALLOC_SCRATCH_BYTES ((size_t)16 << 20)
int infer_paged_decode_noalloc_bf16(const void* q, int64_t q_stride0,
                                    const void* k_cache, const void* v_cache,
                                    int64_t cache_block_stride, int64_t cache_token_stride,
                                    void* out, int64_t out_stride0,
                                    const int32_t* block_table, int64_t bt_stride0, int64_t table_cols,
                                    const int32_t* context_lens,
                                    int64_t batch, int64_t num_q_heads, int64_t num_kv_heads,
                                    int64_t head_dim, int64_t block_size, int64_t num_blocks,
                                    float scale, void* stream);

/* ------------------------------------------------------------------ 2b. paged varlen prefill attention
 * Replaces flash_attn_varlen_func(Q, K, V, max_seqlen_q, cu_seqlens_q, max_seqlen_k, cu_seqlens_k,
 * softmax_scale, causal=True, block_table) at infer/ops/attention.py:110-116.
 *
 * Queries are packed: q [total_q, Hq, D] (row stride q_stride0), sequence s owns rows
 * [cu_seqlens_q[s], cu_seqlens_q[s+1]); out has the same layout.  Keys/values:
 *   block_table != NULL : k, v are the paged caches [num_blocks, block_size, Hkv, D] and sequence s
 *                         uses tokens [0, sk_s) of row s of the table, sk_s from cu_seqlens_k
 *                         (the reference's prefix-cache case, attention.py:111-112);
 *   block_table == NULL : k, v are packed rows [kv_rows, Hkv, D] indexed by cu_seqlens_k
 *                         (kv_token_stride is the row stride, kv_block_stride is ignored).
 * kv_rows = number of token rows addressable through k/v (packed: rows of the tensor; paged:
 * num_blocks * block_size); it only bounds reads.  causal != 0 applies the bottom-right aligned
 * mask (key j visible to query i of the sequence iff j <= i + (sk - sq)).  Queries of a sequence
 * with sk == 0 produce zeros, and so do the first sq - sk queries of a sequence with sq > sk (no key is
 * visible to them).  With a block table, table_cols is the number of entries per row
 * (bt_stride0 >= table_cols) and a key length beyond table_cols * block_size is cut to that.  scale
 * must be positive (INFER_KV_EINVAL otherwise).  Same shape limits as the decode entry points.  No
 * workspace.
 */
int infer_paged_prefill_bf16(const void* q, int64_t q_stride0,
                             const void* k, const void* v,
                             int64_t kv_block_stride, int64_t kv_token_stride, int64_t kv_rows,
                             void* out, int64_t out_stride0,
                             const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k,
                             const int32_t* block_table, int64_t bt_stride0, int64_t table_cols,
                             int64_t num_seqs, int64_t max_seqlen_q,
                             int64_t num_q_heads, int64_t num_kv_heads, int64_t head_dim,
                             int64_t block_size, int64_t num_blocks,
                             float scale, int causal, void* stream);

/* ------------------------------------------------------------------ 2c. the operators of a decode step around the path
 * What the engine runs between two attention calls of a captured decode step, so that the step is
 * HIP kernels of this library plus library GEMMs.
 *
 * infer_rms_norm_bf16 replaces RMSNorm.forward (infer/ops/norm.py:63-98; the torch path the engine
 * runs, rms_forward / add_rms_forward).  Without residual: out = bf16(x * rsqrt(mean(x^2) + eps)) *
 * weight.  With residual: s = float(x) + float(residual); residual <- bf16(s); out from the
 * unrounded s.  out may alias x.  Rows are [n_rows, hidden] bf16 with the given row strides
 * (elements); hidden % 8 == 0 and hidden <= 8192.
 */
int infer_rms_norm_bf16(const void* x, int64_t x_stride0, void* residual, int64_t residual_stride0,
                        const void* weight, void* out, int64_t out_stride0,
                        int64_t n_rows, int64_t hidden, float eps, void* stream);

/* Replaces silu_and_mul(result, input) (src/operators/silu/silu.cu:13-54; schema src/bindings.cpp:22):
 * out[r, j] = bf16(silu(x[r, j])) * x[r, d + j] for x [n_rows, 2 d] bf16, d % 8 == 0. */
int infer_silu_and_mul_bf16(void* out, int64_t out_stride0, const void* x, int64_t x_stride0,
                            int64_t n_rows, int64_t d, void* stream);

/* Replaces the host loop of ModelRunner.prepare_decode (infer/engine/model_runner.py:110-126) by
 * one launch on device-resident state.  seq_lens[b] = len(seq) including the token fed this step:
 *   context_lens[b] = len, positions[b] = len - 1 + position_offset,
 *   slot_mapping[b] = block_table[b, (len-1) / block_size] * block_size + (len-1) % block_size.
 * position_offset = 1 reproduces the reference (model_runner.py:117 feeds len(seq)); 0 gives the
 * zero-based position of its prefill branch (:84).  Rows with seq_lens[b] <= 0 (graph padding) get
 * slot -1, context length 0 and position 0, so they neither touch the cache nor attend. */
int infer_decode_metadata(const int32_t* seq_lens, const int32_t* block_table, int64_t bt_stride0,
                          int64_t batch, int64_t block_size, int64_t table_cols,
                          int64_t position_offset, int64_t* positions, int32_t* slot_mapping,
                          int32_t* context_lens, void* stream);

/* Replaces Linear.forward (infer/ops/MLP.py:103-149, F.linear; the op matmul(input, weight, output) of
 * src/bindings.cpp:7) at the batch sizes of a decode step, for weight matrices with few rows (o_proj,
 * down_proj): y[M, N] = x[M, K] . w[N, K]^T, bf16 in, float32 accumulate, bf16 out, M <= 128.  The
 * weights (row-major [N, K], contiguous) are streamed from HBM once; K is cut over workgroups and
 * float32 partial sums pass through `workspace` (infer_skinny_gemm_workspace_bytes says how much,
 * 0 if the shape needs no split).  K must be a multiple of 128 and N a multiple of 8; other shapes
 * return INFER_KV_EUNSUPPORTED and belong to the vendor GEMM. */
size_t infer_skinny_gemm_workspace_bytes(int64_t m, int64_t n, int64_t k);
int infer_skinny_gemm_bf16(const void* x, int64_t x_stride0, const void* w, void* y, int64_t y_stride0,
                           int64_t m, int64_t n, int64_t k, void* workspace, size_t workspace_bytes,
                           void* stream);
/* The same product without the final reduction, for a consumer that adds the partial sums itself
 * (infer_rms_norm_splitk_bf16): *splits_out > 1 means `workspace` now holds float32 partial sums
 * [splits][m][n] and y was not written; *splits_out == 1 means the shape needed no split and y holds
 * the bf16 result. */
int infer_skinny_gemm_partial_bf16(const void* x, int64_t x_stride0, const void* w, void* y, int64_t y_stride0,
                                   int64_t m, int64_t n, int64_t k, void* workspace, size_t workspace_bytes,
                                   int* splits_out, void* stream);
/* infer_rms_norm_bf16 whose input is still in pieces: x[r] = bf16(sum over s of partial[s][r]) with
 * partial[s][r] at partial + s * split_stride + r * partial_stride0 (float32 elements), added in
 * split order and rounded once - bit-identical to reducing first - then the same normalisation.
 * Fuses the reduction of a split-K o_proj / down_proj into the RMSNorm that follows it
 * (infer/models/Qwen3.py:226-236). */
int infer_rms_norm_splitk_bf16(const float* partial, int64_t splits, int64_t split_stride,
                               int64_t partial_stride0, void* residual, int64_t residual_stride0,
                               const void* weight, void* out, int64_t out_stride0,
                               int64_t n_rows, int64_t hidden, float eps, void* stream);

/* ------------------------------------------------------------------ 3. block pool (host only)
 * C view of infer::BlockPool (include/infer_kv/block_pool.hpp), the native counterpart of the
 * reference's Python BlockManager (infer/engine/block_mannager.py:44-133), which is the block
 * pool the reference engine runs (its C++ include/kvcache.hpp / src/kvcache.cc is never
 * compiled).  Token ids are int64, block ids int32.  Functions that the reference guards with
 * `assert` return INFER_KV_ESTATE and leave a message in infer_pool_last_error() (thread local).
 */
typedef struct infer_pool infer_pool;

infer_pool* infer_pool_create(int32_t num_blocks, int32_t block_size);   /* BlockManager.__init__ :46-52 */
void infer_pool_destroy(infer_pool* pool);
const char* infer_pool_last_error(void);
int32_t infer_pool_num_free(const infer_pool* pool);
int32_t infer_pool_num_used(const infer_pool* pool);

/* can_allocate :76-77 -> 1 / 0. */
int infer_pool_can_allocate(const infer_pool* pool, int64_t num_tokens);

/* allocate :79-103.  Writes ceil(num_tokens / block_size) block ids to table_out and returns the
 * number of tokens already present in the cache (a multiple of block_size), or a negative code. */
int64_t infer_pool_allocate(infer_pool* pool, const int64_t* token_ids, int64_t num_tokens,
                            int32_t* table_out, int64_t table_capacity);

/* deallocate :105-112 (references dropped in reverse table order). */
int infer_pool_deallocate(infer_pool* pool, const int32_t* table, int64_t num_blocks);

/* can_append :114-115 -> 1 / 0. */
int infer_pool_can_append(const infer_pool* pool, int64_t seq_len);

/* may_append :117-133, called after the sequence grew to seq_len tokens.  May append one block id
 * to `table` (capacity must allow num_blocks + 1 then).  Returns the new number of blocks. */
int64_t infer_pool_may_append(infer_pool* pool, const int64_t* token_ids, int64_t seq_len,
                              int32_t* table, int64_t num_blocks, int64_t table_capacity);
/* The same step given only the block_size tokens of the block that seq_len just filled (read only
 * when seq_len % block_size == 0, may be NULL otherwise), so a per-token caller does not have to
 * hand over the whole sequence. */
int64_t infer_pool_may_append_block(infer_pool* pool, const int64_t* last_block_tokens, int64_t seq_len,
                                    int32_t* table, int64_t num_blocks, int64_t table_capacity);

/* compute_hash :54-60: xxh64(seed 0) over [prefix hash as 8 LE bytes, if has_prefix] ++ int64 LE ids. */
uint64_t infer_pool_hash(const int64_t* token_ids, int64_t n, int has_prefix, uint64_t prefix_hash);

/* XXH64 itself (the reference gets it from the un-vendored pip package `xxhash`). */
uint64_t infer_xxh64(const void* data, size_t len, uint64_t seed);

/* Introspection. */
int32_t infer_pool_ref_count(const infer_pool* pool, int32_t block_id);
int infer_pool_block_hash(const infer_pool* pool, int32_t block_id, uint64_t* hash_out);  /* 1 if sealed */
int64_t infer_pool_free_ids(const infer_pool* pool, int32_t* out, int64_t capacity);      /* FIFO order */

#ifdef __cplusplus
}
#endif
#endif /* INFER_KV_H */
