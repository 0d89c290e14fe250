/*
 * msgl_paged_attention.h -- C ABI of the MI355X (gfx950) paged-attention hot path.
 *
 * Three operators, the ones the reference's `mini_sglang_mlx_kernel._ext` module
 * binds for this path (mini-sglang-mlx-kernel/csrc/bindings.cpp:27-55):
 *
 *   store_kv_cache            in-place scatter of new K/V rows into the slot-indexed pools
 *   paged_decode_attention    GQA split-K decode over slots gathered through kv_indices
 *   paged_prefill_attention   extend attention (causal / full / window / bidirectional+window)
 *
 * and the step's metadata build that feeds them (slot table -> CSR arrays), which the
 * reference does in Python (mini_sglang_mlx/attention/backend.py:205-307).
 *
 * Conventions shared by every entry point
 *   - every pointer is a DEVICE pointer in the address space of the current HIP
 *     device; `stream` is a hipStream_t passed as void* (NULL = the null stream);
 *   - the library never allocates, frees, retains or synchronises: launches are
 *     stream-ordered and the call returns as soon as they are enqueued;
 *   - pools are (num_slots, num_kv_heads, head_dim) with the two inner dimensions
 *     contiguous; `*_stride0` is the distance between consecutive slots in ELEMENTS;
 *   - q / out are contiguous (rows, num_q_heads, head_dim);
 *   - index arrays are int32; kv_indices holds one pool slot per token (the
 *     reference's token-granular contract);
 *   - return value: MSGL_OK (0) or a negative MSGL_ERR_* code; no exception and
 *     no abort crosses this boundary.  msgl_strerror() gives the text.
 */
#ifndef MSGL_PAGED_ATTENTION_H
#define MSGL_PAGED_ATTENTION_H

#include <stddef.h>
#include <stdint.h>

#if defined(__GNUC__)
#define MSGL_API __attribute__((visibility("default")))
#else
#define MSGL_API
#endif

#ifdef __cplusplus
extern "C" {
#endif

/* element types of q / k / v / pools / out (F16: store and decode; prefill is bf16 only,
 * as paged_prefill_attention.metal:646-647) */
#define MSGL_DTYPE_BF16 0
#define MSGL_DTYPE_F16 1

#define MSGL_OK 0
#define MSGL_ERR_NULL_POINTER (-1)      /* a required pointer is NULL */
#define MSGL_ERR_HEAD_DIM (-2)          /* head_dim is not 128 or 256 */
#define MSGL_ERR_HEAD_RATIO (-3)        /* num_q_heads is not a multiple of num_kv_heads */
#define MSGL_ERR_GROUP_TOO_LARGE (-4)   /* decode: num_q_heads / num_kv_heads > 16 */
#define MSGL_ERR_DTYPE (-5)             /* unsupported element type for this operator */
#define MSGL_ERR_BATCH (-6)             /* prefill: batch <= 0 */
#define MSGL_ERR_WINDOW (-7)            /* prefill: sliding_window_size < 0 */
#define MSGL_ERR_WORKSPACE (-8)         /* workspace missing or smaller than *_workspace_bytes() */
#define MSGL_ERR_SHAPE (-9)             /* negative size, stride smaller than a row, ... */
#define MSGL_ERR_ALIGNMENT (-10)        /* pointer or stride not aligned for the vector width used */
#define MSGL_ERR_LAUNCH (-11)           /* the HIP runtime refused a launch (hipGetLastError) */
#define MSGL_ERR_HEAD_DIM_MULT4 (-12)   /* store: head_dim is not a multiple of 4 */
#define MSGL_ERR_GDN_DIMS (-13)         /* gdn_state_inplace: dk and dv must both be 128 */
#define MSGL_ERR_SCRATCH_LIMIT (-14)    /* *_noalloc: sizes exceed the built-in scratch */

/* Library version: major*10000 + minor*100 + patch. */
MSGL_API int msgl_version(void);

/* Static, never-NULL description of a return code. */
MSGL_API const char* msgl_strerror(int code);

/*
 * store_kv_cache -- replaces mini_sglang_mlx::store_kv_cache
 * (mini-sglang-mlx-kernel/csrc/store_kv_cache.cpp:14-107, kernel store_kv_cache.metal:7-31):
 *     k_cache[indices[r], :, :] = k[r, :, :];  v_cache[indices[r], :, :] = v[r, :, :]
 * Bit copy of `elem_bytes`-wide elements (2 for bf16/f16).  The caller guarantees
 * indices are unique and inside [0, num_slots); duplicate indices race, as in the
 * reference.  Unlike the reference, which applies k's strides to v and k_cache's to
 * v_cache (store_kv_cache.cpp:65-66), all four leading strides are taken explicitly.
 * `length == 0` is a no-op.
 */
MSGL_API int msgl_store_kv_cache(void* k_cache, void* v_cache, const int32_t* indices,
                        const void* k, const void* v,
                        int64_t length, int64_t num_kv_heads, int64_t head_dim,
                        int64_t num_slots,
                        int64_t k_cache_stride0, int64_t v_cache_stride0,
                        int64_t k_stride0, int64_t v_stride0,
                        int32_t elem_bytes, void* stream);

/*
 * Workspace (bytes) that msgl_paged_decode_attention needs for these sizes.
 * `total_kv` is the length of kv_indices.  Replaces the per-call att_out/att_lse
 * allocation of PagedDecodeAttention::eval_gpu (paged_decode_attention.cpp:118-129).
 */
MSGL_API size_t msgl_paged_decode_workspace_bytes(int64_t batch, int64_t total_kv,
                                         int64_t num_q_heads, int64_t num_kv_heads,
                                         int64_t head_dim);

/*
 * paged_decode_attention -- replaces mini_sglang_mlx::paged_decode_attention
 * (paged_decode_attention.cpp:15-73; kernels paged_decode_attention.metal:313-586).
 *   q   (batch, num_q_heads, head_dim)      out (batch, num_q_heads, head_dim)
 *   kv_indptr (batch+1)   kv_indices (total_kv)   num_kv_splits (batch)
 * Request b attends to all kv_indptr[b+1]-kv_indptr[b] tokens listed for it.
 * The concatenated KV stream of the batch is cut into equal segments, one resident round of
 * workgroups on MI355X; partial results are merged by log-sum-exp.  The result does not
 * depend on the split, so `num_kv_splits` / `max_kv_splits` (the reference's
 * split hints, backend.py:304-307) are accepted and validated but do not steer
 * the cut.  A request with no tokens gets zeros (the reference leaves its rows
 * unwritten, paged_decode_attention.metal:354).
 * `dtype`: MSGL_DTYPE_BF16 or MSGL_DTYPE_F16, the two the reference instantiates for decode
 * (paged_decode_attention.metal:596-604); q, both pools and out share it.
 */
MSGL_API int msgl_paged_decode_attention(const void* q, const void* k_cache, const void* v_cache,
                                const int32_t* kv_indptr, const int32_t* kv_indices,
                                const int32_t* num_kv_splits, void* out,
                                void* workspace, size_t workspace_bytes,
                                int64_t batch, int64_t total_kv,
                                int64_t num_q_heads, int64_t num_kv_heads, int64_t head_dim,
                                int64_t num_slots,
                                int64_t k_cache_stride0, int64_t v_cache_stride0,
                                float sm_scale, int32_t max_kv_splits,
                                int32_t dtype, void* stream);

/*
 * paged_decode_attention for callers that cannot allocate -- no counterpart in the reference
 * (its decode op allocates att_out / att_lse on every call, paged_decode_attention.cpp:118-129).
 * For code under HIP graph capture, tight serving loops and harnesses that forbid hipMalloc:
 * same arguments and same result (bit for bit) as msgl_paged_decode_attention, minus the
 * workspace, which is a file-scope device array of MSGL_DECODE_SCRATCH_BYTES that is part of
 * the library's code object (every GPU the library runs on holds it until the process ends).
 * The call makes no hipMalloc / hipFree and no allocating library call; the first call on a
 * device looks the array's address up (hipGetSymbolAddress) and keeps it, so make that first
 * call outside a capture.  Sizes whose split-K partials need more than the array
 * ((segments + batch) * num_q_heads * (head_dim + 1) floats; 3.2 MB at batch 64, 32 / 8 heads
 * of 128) return MSGL_ERR_SCRATCH_LIMIT and launch nothing.  Every call on one GPU uses the
 * same array, whatever the stream: calls that overlap in time on one GPU race.  Nothing in the
 * array has to start at zero (the attention kernel writes every entry the merge reads).
 */
#define MSGL_DECODE_SCRATCH_BYTES (8 * 1024 * 1024)
MSGL_API int msgl_paged_decode_attention_noalloc(const void* q, const void* k_cache,
                                const void* v_cache,
                                const int32_t* kv_indptr, const int32_t* kv_indices,
                                const int32_t* num_kv_splits, void* out,
                                int64_t batch, int64_t total_kv,
                                int64_t num_q_heads, int64_t num_kv_heads, int64_t head_dim,
                                int64_t num_slots,
                                int64_t k_cache_stride0, int64_t v_cache_stride0,
                                float sm_scale, int32_t max_kv_splits,
                                int32_t dtype, void* stream);

/*
 * Workspace (bytes) that msgl_paged_prefill_attention needs for these sizes: the partials of the
 * split-K route, or those of the tile kernels when the launch is too small to fill the chip and
 * the keys of each query block are shared out over several workgroups, or (head_dim 128, 2, 4, 8
 * or 16 query blocks of 256 rows per request and kv head, enough work to fill the chip) the
 * slots and count words of gang ranges, with which one workgroup per compute unit stays for the
 * launch and the (request, kv head) units are shared out by length; 0 otherwise.  The split-K
 * route needs its workspace (MSGL_ERR_WORKSPACE without it); the tile kernels fall back to one
 * pass over the keys per query block when the workspace is missing or too small.  total_kv must
 * be at least kv_indptr[batch], here and in msgl_paged_prefill_attention: key shares, grids and
 * this size are derived from it (a smaller value leaves requests' rows unwritten).  Nothing in
 * the workspace has to be initialised.
 */
MSGL_API size_t msgl_paged_prefill_workspace_bytes(int64_t batch, int64_t total_q, int64_t total_kv,
                                          int64_t num_q_heads, int64_t num_kv_heads,
                                          int64_t head_dim, int64_t max_len_extend);

/*
 * paged_prefill_attention -- replaces mini_sglang_mlx::paged_prefill_attention
 * (paged_prefill_attention.cpp:18-87; kernel paged_prefill_attention.metal:382-640).
 *   q   (total_q, num_q_heads, head_dim)    out (total_q, num_q_heads, head_dim)
 *   qo_indptr (batch+1)  kv_indptr (batch+1)  kv_indices (total_kv)  prefix_lens (batch)
 * Query i of request b sits at position prefix_lens[b] + i; key j (index in the
 * request's kv stream) is visible iff
 *     (is_cross_attention || j <= qpos) && (window == 0 || j >= qpos - window + 1)
 * (paged_prefill_attention.metal:339-347).  A query with no visible key gets zeros
 * (:627-630).  Requests whose query length exceeds `max_len_extend` are computed only
 * for their first max_len_extend queries, as in the reference's grid
 * (paged_prefill_attention.cpp:152-159).  Short query blocks (speculative verify,
 * draft proposal) are routed to the bandwidth-bound split-K kernel, long ones to
 * the MFMA tile kernel of their head_dim; same arguments, same result.  A launch of the tile
 * kernels with fewer query blocks than compute units (one long request, a short extend) shares
 * the keys of every block out over up to 32 workgroups and merges their fp32 partials by
 * log-sum-exp in a second kernel.
 */
MSGL_API int msgl_paged_prefill_attention(const void* q, const void* k_cache, const void* v_cache,
                                 const int32_t* qo_indptr, const int32_t* kv_indptr,
                                 const int32_t* kv_indices, const int32_t* prefix_lens,
                                 void* out, void* workspace, size_t workspace_bytes,
                                 int64_t batch, int64_t total_q, int64_t total_kv,
                                 int64_t num_q_heads, int64_t num_kv_heads, int64_t head_dim,
                                 int64_t num_slots,
                                 int64_t k_cache_stride0, int64_t v_cache_stride0,
                                 float sm_scale, int32_t max_len_extend,
                                 int32_t is_cross_attention, int32_t sliding_window_size,
                                 int32_t dtype, void* stream);

/*
 * build_attention_metadata -- replaces AttnBackend.build_prefill_metadata /
 * build_decode_metadata, _build_indptr and _compute_num_kv_splits
 * (mini_sglang_mlx/attention/backend.py:205-307) with one launch and no host round trip:
 *     kv_indptr  = cumsum([0] + kv_lens)          qo_indptr = cumsum([0] + extend_lens)
 *     kv_indices = concat(page_table[table_rows[b], :kv_lens[b]])
 *     prefix_lens[b] = kv_lens[b] - extend_lens[b]
 *     positions  = concat(arange(prefix_lens[b], kv_lens[b]))
 *     num_kv_splits[b] = min(max_kv_splits, max(1, ceil(kv_lens[b] / 128)))
 * page_table is the (n_table_rows, max_seq_len) int32 slot table (one slot id per token,
 * engine.py:84-87) with leading stride `table_stride0` elements; table_rows, kv_lens and
 * extend_lens are int32 [batch].  extend_lens == NULL means one query per request (decode:
 * positions[b] = kv_lens[b] - 1, qo_indptr = 0..batch).  qo_indptr, prefix_lens, positions and
 * num_kv_splits may be NULL (not produced).  Lengths are clamped to [0, max_seq_len]
 * (extend_lens to [0, kv_len]) and table rows to the table, so no access leaves the
 * arguments; writes to kv_indices / positions stop at kv_capacity / q_capacity elements while
 * kv_indptr[batch] / qo_indptr[batch] always hold the full totals, so the caller can detect
 * a capacity that was too small.  batch <= 8000.
 */
MSGL_API int msgl_build_attention_metadata(const int32_t* page_table, int64_t table_stride0,
                                  int64_t n_table_rows, int64_t max_seq_len,
                                  const int32_t* table_rows, const int32_t* kv_lens,
                                  const int32_t* extend_lens, int64_t batch,
                                  int32_t* kv_indptr, int32_t* kv_indices, int64_t kv_capacity,
                                  int32_t* qo_indptr, int32_t* prefix_lens, int32_t* positions,
                                  int64_t q_capacity, int32_t* num_kv_splits,
                                  int32_t max_kv_splits, void* stream);

/*
 * qk_norm_rope_store -- replaces the chain in front of the attention call in the reference's
 * Qwen3 attention layer (mini_sglang_mlx/models/qwen3.py:60-68) together with the store that
 * AttnBackend.forward does first (mini_sglang_mlx/attention/backend.py:139):
 *     q = q_norm(q); k = k_norm(k)               per-head RMSNorm, weights (head_dim,)
 *     q = rope(q, positions); k = rope(k, positions)   rotate-half form, rotary_dim = head_dim
 *     k_cache[out_loc[t]] = k[t]; v_cache[out_loc[t]] = v[t]
 * in one pass over q, k, v.  q / k / v are (n_tokens, heads, head_dim) bf16 with the two inner
 * dimensions contiguous and leading strides `*_stride0` in elements (views into a fused QKV
 * projection are fine); q_out is contiguous (n_tokens, num_q_heads, head_dim).  positions and
 * out_loc are int32 [n_tokens]; out_loc values must be unique and inside [0, num_slots).
 * v is copied bit for bit.  head_dim 128 or 256, all pointers 16-byte aligned, strides
 * multiples of 8 elements.  Attention is then called on q_out WITHOUT another store.
 */
MSGL_API int msgl_qk_norm_rope_store(const void* q, const void* k, const void* v,
                            int64_t q_stride0, int64_t k_stride0, int64_t v_stride0,
                            const void* q_weight, const void* k_weight,
                            const int32_t* positions, const int32_t* out_loc,
                            void* q_out, void* k_cache, void* v_cache,
                            int64_t k_cache_stride0, int64_t v_cache_stride0, int64_t num_slots,
                            int64_t n_tokens, int64_t num_q_heads, int64_t num_kv_heads,
                            int64_t head_dim, float rms_norm_eps, float rope_base,
                            int32_t dtype, void* stream);

/*
 * gdn_state_inplace -- replaces mini_sglang_mlx::gdn_state_inplace
 * (mini-sglang-mlx-kernel/csrc/gdn_state.cpp:87-183, kernel gdn_state.metal:14-99), the gated
 * delta-rule recurrence of the hybrid (Qwen3.5) layers with a slot-indexed state:
 * for request b, state S = state[slot_ids[b]] of shape (hv, dv, dk), and each of its tokens t
 * in order
 *     S *= g[t, h];  delta = (v[t, h, :] - S[h] k[t, h / (hv / hk)]) * beta[t, h]
 *     S[h] += outer(delta, k[t, h / (hv / hk)]);  y[t, h, :] = S[h] q[t, h / (hv / hk)]
 * q, k: (tokens, hk, 128) bf16; v, y: (tokens, hv, 128) bf16; g, beta: (tokens, hv) bf16
 * contiguous; state: (num_slots, hv, 128, 128) fp32, updated in place; slot_ids int32 [batch]
 * (distinct, inside [0, num_slots)); qo_indptr int32 [batch + 1], the token range of each
 * request, ignored in single_token_mode (one token per request, token b belongs to request
 * b; the reference's decode mode).  *_stride0: leading strides in elements (the reference
 * uses q's for k as well, gdn_state.cpp:163-164; here both are taken).  hv % hk == 0.
 */
MSGL_API int msgl_gdn_state_inplace(const void* q, const void* k, const void* v, const void* g,
                           const void* beta, void* state, const int32_t* slot_ids,
                           const int32_t* qo_indptr, void* y, int64_t tokens, int64_t batch,
                           int64_t hk, int64_t hv, int64_t dk, int64_t dv, int64_t num_slots,
                           int64_t state_stride0, int64_t q_stride0, int64_t k_stride0,
                           int64_t v_stride0, int32_t single_token_mode, void* stream);

/*
 * Tuning knobs, for benchmarking only (0 = built-in heuristic).  One set per HOST THREAD
 * (thread-local): msgl_set_tuning changes the calling thread's later calls only, so a
 * *_workspace_bytes() call and the launch that follows it on the same thread agree whatever
 * other threads set.  Read at launch time; not part of the reference surface.
 *   MSGL_TUNE_SEGMENTS       segments the split-K kernel cuts the visible token stream into
 *   MSGL_TUNE_MIN_SEGMENT    smallest segment length in tokens (multiple of 64; default 128 at
 *                            head_dim 128, 64 at head_dim 256)
 *   MSGL_TUNE_SMALLQ_MAXCOLS largest q_len*group routed to the split-K kernel (up to 64; default
 *                            48 at head_dim 128, 16 at head_dim 256, and up to 64 where the tile
 *                            kernels cannot split a request's keys by its length; negative: never)
 *   MSGL_TUNE_PREFILL_VARIANT head_dim 128 MFMA kernel: 0 the ping-pong kernel (8 waves x 32 rows,
 *                            the two waves of a SIMD alternate between MFMA and softmax phases),
 *                            1 the fused kernel it replaced (8 x 32 rows, every wave a software-
 *                            pipelined mix of MFMA and softmax), kept as its comparison partner
 *   MSGL_TUNE_SPLITKV_WAVES  most waves (adjacent kv heads) per split-K workgroup: 1, 2, 4, 8
 *                            (0 restores the default, 4)
 *   MSGL_TUNE_SPLITKV_BOUNDARY tokens' worth of time a split-K workgroup is charged for starting
 *                            on another request inside its segment (0: default from the shape,
 *                            negative: none)
 *   MSGL_TUNE_GDN_ROWS       state rows per 16-lane group of the gdn_state kernel: 1, 2, 4
 *                            (0: chosen from the problem size)
 *   MSGL_TUNE_PREFILL_KEY_SPLITS  workgroups that share the keys of one query block of the MFMA
 *                            tile kernels (1: never split, up to 32; 0: chosen from the sizes,
 *                            and launches with one query block per request and kv head give each
 *                            request as many shares as its length asks for, up to 128 requests
 *                            or 1024 long ones)
 *   MSGL_TUNE_PREFILL_GANGS  negative: extends with several query blocks per request and kv head
 *                            never use gang ranges (one workgroup per compute unit for the whole
 *                            launch, the units' keys shared out by length); 0: chosen from the sizes;
 *                            positive: whenever the shape allows it, however small the launch
 *   MSGL_TUNE_CLOCK_PROBE    measurement aid: the value is a device pointer to two int64 (0: none).
 *                            Workgroup 0 of every attention kernel launched by this thread then
 *                            leaves there the shader cycles and the 100 MHz wall ticks it lived
 *                            for: cycles / ticks x 0.1 = the shader clock in GHz under that kernel
 */
#define MSGL_TUNE_SEGMENTS 0
#define MSGL_TUNE_MIN_SEGMENT 1
#define MSGL_TUNE_SMALLQ_MAXCOLS 2
#define MSGL_TUNE_PREFILL_VARIANT 3
#define MSGL_TUNE_SPLITKV_WAVES 4
#define MSGL_TUNE_GDN_ROWS 5
#define MSGL_TUNE_PREFILL_KEY_SPLITS 6
#define MSGL_TUNE_SPLITKV_BOUNDARY 7
#define MSGL_TUNE_PREFILL_GANGS 8
#define MSGL_TUNE_CLOCK_PROBE 9
MSGL_API int msgl_set_tuning(int32_t knob, int64_t value);
/* The value the calling thread last set for `knob` (0 if it never did): what its launches and
 * workspace queries use.  Makes the per-thread scope observable: a value set on another thread
 * does not show here.  No counterpart in the reference. */
MSGL_API int msgl_get_tuning(int32_t knob, int64_t* value);

#ifdef __cplusplus
}
#endif
#endif /* MSGL_PAGED_ATTENTION_H */
