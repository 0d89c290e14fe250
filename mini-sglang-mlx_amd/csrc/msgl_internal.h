// Host-side declarations shared by the translation units of libmsgl_paged_attention.so.
#pragma once
#include <hip/hip_runtime.h>
#include <algorithm>
#include <stddef.h>
#include <stdint.h>

#include "../../include/msgl_paged_attention.h"
#include "../../include/msgl_state_pool.h"

namespace msgl {

// ---- store_kv_cache.hip ------------------------------------------------------------
int launch_store_kv_cache(void* k_cache, void* v_cache, const int32_t* indices, const void* k,
                          const void* v, int64_t length, int64_t num_slots, int64_t row_bytes,
                          int64_t k_cache_stride_bytes, int64_t v_cache_stride_bytes,
                          int64_t k_stride_bytes, int64_t v_stride_bytes, hipStream_t stream);

// ---- paged_splitkv.hip -------------------------------------------------------------
// One description serves decode (qo_indptr == nullptr: one query per request, every key
// visible) and the short-query route of prefill (speculative verify / draft proposal).
struct SplitKvArgs {
  const void* q;
  const void* k_cache;
  const void* v_cache;
  const int32_t* kv_indptr;
  const int32_t* kv_indices;
  const int32_t* qo_indptr;    // nullptr for decode
  const int32_t* prefix_lens;  // nullptr for decode
  void* out;
  void* workspace;
  int64_t batch, total_kv, n_q, n_kv, head_dim, num_slots;
  int64_t k_stride0, v_stride0;  // elements
  float sm_scale;
  int32_t max_len_extend;  // 1 for decode; queries per request handled by this launch
  int32_t q_begin;         // first query of every request handled by this launch
  int32_t q_cap;           // cap on a request's query count (0: max_len_extend)
  int32_t f16;             // 1: q / pools / out are IEEE half (decode only), 0: bf16
  int32_t is_cross, window;
  int32_t n_seg;    // segments the visible token stream is cut into
  int32_t min_seg;  // smallest segment length in tokens, multiple of 64
};
// largest q_len * group the split-K kernel is instantiated for
constexpr int kSplitKvMaxCols = 64;
constexpr int kSplitKvMinSegment = 128;
// one resident round of workgroups for this shape, capped so segments keep min_seg tokens
int splitkv_default_segments(int64_t total_kv, int64_t n_kv, int64_t head_dim, int64_t cols,
                             int32_t min_seg);
// benchmarking switch: stream positions charged per request boundary (0: default, negative: none)
void splitkv_set_boundary(int v);
size_t splitkv_workspace_bytes(int64_t batch, int64_t n_q, int64_t n_kv, int64_t head_dim,
                               int64_t max_len_extend, int32_t n_seg);
int launch_splitkv(const SplitKvArgs& a, hipStream_t stream);
// Address (on the current device) and size of the library's built-in split-K scratch, for the
// entry point that takes no workspace.  The first call on a device resolves the address.
int splitkv_scratch(void** ptr, size_t* bytes);
// benchmarking switch: most waves (adjacent kv heads) a split-K workgroup may hold
void splitkv_set_max_waves(int v);

// ---- paged_prefill.hip -------------------------------------------------------------
struct PrefillArgs {
  const void* q;
  const void* k_cache;
  const void* v_cache;
  const int32_t* qo_indptr;
  const int32_t* kv_indptr;
  const int32_t* kv_indices;
  const int32_t* prefix_lens;
  void* out;
  int64_t batch, total_q, total_kv, n_q, n_kv, head_dim, num_slots;
  int64_t k_stride0, v_stride0;  // elements
  float sm_scale;
  int32_t max_len_extend;
  int32_t is_cross, window;
  // key splits (1: none); above 1, `workspace` holds
  // key_splits * total_q * n_q * (head_dim + 1) floats
  int32_t key_splits;
  void* workspace;
  // ragged shares instead (one query block per (request, kv head) only): key tiles per share,
  // 0 = off; `workspace` then holds prefill_ragged_workspace_bytes()
  int32_t ragged_tiles;
  // gang ranges instead (several query blocks per (request, kv head), head_dim 128 only): gangs
  // per XCD, 0 = off; `workspace` then holds prefill_gang_workspace_bytes(); `gang_nonce` is a
  // number no earlier launch on this workspace has used
  int32_t gangs;
  unsigned long long gang_nonce;
};
int launch_prefill_tile(const PrefillArgs& a, hipStream_t stream);     // head_dim 128
// ---- paged_prefill_d256.hip ----------------------------------------------------------
int launch_prefill_tile256(const PrefillArgs& a, hipStream_t stream);  // head_dim 256
// benchmarking switch: head_dim 128 kernel (0: ping-pong kernel, anything else: the fused kernel
// it replaced, 8 waves x 32 rows)
int tile_variant();
void set_tile_variant(int v);
// measurement aid (MSGL_TUNE_CLOCK_PROBE): two device int64 the attention kernels' workgroup 0
// fills with its shader cycles and 100 MHz wall ticks, or nullptr; one value per host thread
long long* clock_probe();

// ---- build_metadata.hip ------------------------------------------------------------
struct MetadataArgs {
  const int32_t* page_table;
  const int32_t* table_rows;
  const int32_t* kv_lens;
  const int32_t* extend_lens;  // nullptr: decode
  int32_t* kv_indptr;
  int32_t* kv_indices;
  int32_t* qo_indptr;
  int32_t* prefix_lens;
  int32_t* positions;
  int32_t* num_kv_splits;
  int64_t table_stride0, batch, n_table_rows, max_seq_len, kv_capacity, q_capacity;
  int32_t max_kv_splits;
};
// largest batch one launch handles (two scanned offset arrays live in LDS)
constexpr int64_t kMetadataMaxBatch = 8000;
int launch_build_metadata(const MetadataArgs& a, hipStream_t stream);

// ---- qk_norm_rope_store.hip ----------------------------------------------------------
struct NormRopeArgs {
  const void* q;
  const void* k;
  const void* v;
  const void* q_weight;
  const void* k_weight;
  const int32_t* positions;
  const int32_t* out_loc;
  void* q_out;
  void* k_cache;
  void* v_cache;
  int64_t q_stride0, k_stride0, v_stride0, kc_stride0, vc_stride0;  // elements
  int64_t n_tokens, n_q, n_kv, head_dim, num_slots;
  float eps, rope_base;
};
int launch_qk_norm_rope_store(const NormRopeArgs& a, hipStream_t stream);

// ---- gdn_state.hip ---------------------------------------------------------------------
struct GdnArgs {
  const void* q;
  const void* k;
  const void* v;
  const void* g;
  const void* beta;
  void* state;
  const int32_t* slot_ids;
  const int32_t* qo_indptr;  // unused in single-token mode
  void* y;
  int64_t tokens, batch, hk, hv;
  int64_t state_stride0, q_stride0, k_stride0, v_stride0;  // elements
  int32_t single_token_mode;
};
int launch_gdn_state(const GdnArgs& a, hipStream_t stream);
// benchmarking switch: state rows per 16-lane group (1, 2, 4; 0 = chosen from the problem size)
void gdn_set_rows(int v);

// ---- state_slots.hip -------------------------------------------------------------------
// src == nullptr: zero fill of the dst slots
int launch_state_slots(void* base, int64_t layer_stride, int64_t slot_stride, int64_t row_bytes,
                       int64_t n_layers, int64_t num_slots, const int32_t* src, const int32_t* dst,
                       int64_t n_pairs, hipStream_t stream);

inline int check_launch() { return hipGetLastError() == hipSuccess ? MSGL_OK : MSGL_ERR_LAUNCH; }

}  // namespace msgl
