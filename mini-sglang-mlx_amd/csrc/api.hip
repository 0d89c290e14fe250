// extern "C" entry points of libmsgl_paged_attention.so: argument checks and routing.
// The checks mirror the reference's host functions (paged_decode_attention.cpp:25-62,
// paged_prefill_attention.cpp:31-76, store_kv_cache.cpp:22-63) as far as raw pointers
// and sizes can express them; rank and dtype-equality checks live in the Python shim.
#include <algorithm>
#include <atomic>

#include "msgl_internal.h"
#include "prefill_params.h"

namespace {

// Benchmarking knobs live per host thread: the thread that sets one changes its own later
// calls only, so a *_workspace_bytes() call and the launch that follows it on the same thread
// always agree on the split, whatever other threads (one per stream) do.
thread_local int64_t t_tune[3] = {0, 0, 0};
thread_local int64_t t_key_splits = 0;
thread_local int64_t t_gangs = 0;  // negative: never use gang ranges
thread_local long long* t_clock_probe = nullptr;
constexpr int kTuneKnobs = 10;
thread_local int64_t t_last_set[kTuneKnobs] = {};  // what this thread last passed to msgl_set_tuning
// launch numbers for the count words of gang ranges (see prefill_gangs()); never 0
std::atomic<unsigned long long> g_gang_nonce{1};

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

int check_common(const void* q, const void* k_cache, const void* v_cache, const void* out,
                 int64_t n_q, int64_t n_kv, int64_t d, int64_t k_stride0, int64_t v_stride0,
                 int32_t dtype, bool f16_ok) {
  if (d != 128 && d != 256) return MSGL_ERR_HEAD_DIM;
  if (n_q <= 0 || n_kv <= 0) return MSGL_ERR_SHAPE;
  if (n_q % n_kv != 0) return MSGL_ERR_HEAD_RATIO;
  // IEEE half exists for decode only, as in the reference (paged_decode_attention.metal:596-604
  // against paged_prefill_attention.metal:646-647)
  if (dtype != MSGL_DTYPE_BF16 && !(f16_ok && dtype == MSGL_DTYPE_F16)) return MSGL_ERR_DTYPE;
  if (k_stride0 < n_kv * d || v_stride0 < n_kv * d) return MSGL_ERR_SHAPE;
  if (!q || !k_cache || !v_cache || !out) return MSGL_ERR_NULL_POINTER;
  // 16-byte row segments are the unit of every load and store
  if (!aligned16(q) || !aligned16(k_cache) || !aligned16(v_cache) || !aligned16(out) ||
      k_stride0 % 8 != 0 || v_stride0 % 8 != 0)
    return MSGL_ERR_ALIGNMENT;
  return MSGL_OK;
}

// Smallest segment: 128 tokens at head_dim 128 (64 changes nothing there), 64 at head_dim 256,
// where a workgroup takes twice as long per token and small launches gain 15-20 % from the
// finer cut.
int32_t min_segment(int64_t head_dim) {
  const int64_t t = t_tune[MSGL_TUNE_MIN_SEGMENT];
  if (t >= 64) return (int32_t)(t / 64 * 64);
  return head_dim == 256 ? 64 : msgl::kSplitKvMinSegment;
}
int32_t segments(int64_t total_kv, int64_t n_kv, int64_t head_dim, int64_t cols) {
  const int64_t t = t_tune[MSGL_TUNE_SEGMENTS];
  if (t >= 1) return (int32_t)(t < (1 << 20) ? t : (1 << 20));
  return msgl::splitkv_default_segments(total_kv, n_kv, head_dim, cols, min_segment(head_dim));
}
// Largest q_len * group that takes the split-K route whatever the launch: at head_dim 128 48 (up
// to three column tiles in one wave; 49-64 columns would run on two waves per kv head that each
// read every K / V row, and the tile kernel with ragged key shares is as fast or faster on them),
// at head_dim 256 16 (one column tile; more would be a wave per tile, each reading every row,
// and the tile kernel with ragged shares is 10-65 % faster from 17 columns on).  Up to 64 columns
// the split-K kernel also takes what the tile kernels cannot give ragged shares to (very many
// or many short requests): its segments are balanced whatever the lengths, and one long request
// among many short ones would otherwise be one long workgroup per kv head.
int64_t smallq_base_cols(int64_t head_dim) { return head_dim == 128 ? 48 : 16; }

}  // namespace

namespace msgl {
long long* clock_probe() { return t_clock_probe; }
}  // namespace msgl

extern "C" {

int msgl_version(void) { return 100; }

const char* msgl_strerror(int code) {
  switch (code) {
    case MSGL_OK: return "ok";
    case MSGL_ERR_NULL_POINTER: return "a required pointer is NULL";
    case MSGL_ERR_HEAD_DIM: return "head_dim must be 128 or 256";
    case MSGL_ERR_HEAD_RATIO: return "num_q_heads must be a multiple of num_kv_heads";
    case MSGL_ERR_GROUP_TOO_LARGE: return "only q_heads/kv_heads <= 16 is supported";
    case MSGL_ERR_DTYPE: return "unsupported dtype";
    case MSGL_ERR_BATCH: return "batch must be > 0";
    case MSGL_ERR_WINDOW: return "sliding_window_size must be >= 0";
    case MSGL_ERR_WORKSPACE: return "workspace missing or too small";
    case MSGL_ERR_SHAPE: return "invalid size or stride";
    case MSGL_ERR_ALIGNMENT: return "pointer or stride not aligned to the vector width";
    case MSGL_ERR_LAUNCH: return "HIP kernel launch failed";
    case MSGL_ERR_HEAD_DIM_MULT4: return "head_dim must be a multiple of 4";
    case MSGL_ERR_GDN_DIMS: return "this specialized kernel requires dk=dv=128";
    case MSGL_ERR_SCRATCH_LIMIT:
      return "sizes need more split-K scratch than the library's built-in 8 MiB; use the entry "
             "point that takes a workspace";
    default: return "unknown error code";
  }
}

int msgl_get_tuning(int32_t knob, int64_t* value) {
  if (!value) return MSGL_ERR_NULL_POINTER;
  if (knob < 0 || knob >= kTuneKnobs) return MSGL_ERR_SHAPE;
  *value = t_last_set[knob];
  return MSGL_OK;
}

int msgl_set_tuning(int32_t knob, int64_t value) {
  if (knob >= 0 && knob < kTuneKnobs) t_last_set[knob] = value;
  if (knob == MSGL_TUNE_SPLITKV_WAVES) {
    msgl::splitkv_set_max_waves((int)value);
    return MSGL_OK;
  }
  if (knob == MSGL_TUNE_SPLITKV_BOUNDARY) {
    msgl::splitkv_set_boundary((int)value);
    return MSGL_OK;
  }
  if (knob == MSGL_TUNE_GDN_ROWS) {
    msgl::gdn_set_rows((int)value);
    return MSGL_OK;
  }
  if (knob == MSGL_TUNE_PREFILL_VARIANT) {
    msgl::set_tile_variant((int)value);
    return MSGL_OK;
  }
  if (knob == MSGL_TUNE_PREFILL_KEY_SPLITS) {
    t_key_splits = value < 0 ? 0 : value;
    return MSGL_OK;
  }
  if (knob == MSGL_TUNE_PREFILL_GANGS) {
    t_gangs = value;
    return MSGL_OK;
  }
  if (knob == MSGL_TUNE_CLOCK_PROBE) {
    t_clock_probe = reinterpret_cast<long long*>(static_cast<intptr_t>(value));
    return MSGL_OK;
  }
  if (knob < 0 || knob > 2) return MSGL_ERR_SHAPE;
  t_tune[knob] = value;
  return MSGL_OK;
}

int msgl_store_kv_cache(void* k_cache, void* v_cache, const int32_t* indices, const void* k,
                        const void* v, int64_t length, int64_t num_kv_heads, int64_t head_dim,
                        int64_t num_slots, int64_t k_cache_stride0, int64_t v_cache_stride0,
                        int64_t k_stride0, int64_t v_stride0, int32_t elem_bytes, void* stream) {
  if (length < 0 || num_kv_heads <= 0 || head_dim <= 0 || num_slots < 0) return MSGL_ERR_SHAPE;
  if (elem_bytes != 2 && elem_bytes != 4) return MSGL_ERR_DTYPE;
  if (head_dim % 4 != 0) return MSGL_ERR_HEAD_DIM_MULT4;  // store_kv_cache.cpp:49-52
  const int64_t row = num_kv_heads * head_dim;
  if (k_cache_stride0 < row || v_cache_stride0 < row || k_stride0 < row || v_stride0 < row)
    return MSGL_ERR_SHAPE;
  if (length == 0) return MSGL_OK;
  if (!k_cache || !v_cache || !indices || !k || !v) return MSGL_ERR_NULL_POINTER;
  return msgl::launch_store_kv_cache(k_cache, v_cache, indices, k, v, length, num_slots, row * elem_bytes,
                                     k_cache_stride0 * elem_bytes, v_cache_stride0 * elem_bytes,
                                     k_stride0 * elem_bytes, v_stride0 * elem_bytes,
                                     static_cast<hipStream_t>(stream));
}

size_t msgl_paged_decode_workspace_bytes(int64_t batch, int64_t total_kv, int64_t num_q_heads,
                                         int64_t num_kv_heads, int64_t head_dim) {
  if (batch <= 0 || total_kv < 0 || num_q_heads <= 0 || num_kv_heads <= 0 ||
      num_q_heads % num_kv_heads != 0)
    return 0;
  const int64_t group = num_q_heads / num_kv_heads;
  return msgl::splitkv_workspace_bytes(batch, num_q_heads, num_kv_heads, head_dim, 1,
                                       segments(total_kv, num_kv_heads, head_dim, group));
}

// Both decode entry points: `builtin_scratch` takes the workspace from the library's own
// per-device array instead of the caller.
static int decode_attention(const void* q, const void* k_cache, const void* v_cache,
                            const int32_t* kv_indptr, const int32_t* kv_indices,
                            const int32_t* num_kv_splits, void* out, void* workspace,
                            size_t workspace_bytes, bool builtin_scratch, int64_t batch,
                            int64_t total_kv, int64_t num_q_heads, int64_t num_kv_heads,
                            int64_t head_dim, int64_t num_slots, int64_t k_cache_stride0,
                            int64_t v_cache_stride0, float sm_scale, int32_t max_kv_splits,
                            int32_t dtype, void* stream) {
  if (batch < 0 || total_kv < 0 || num_slots < 0) return MSGL_ERR_SHAPE;
  if (batch == 0) return MSGL_OK;
  int rc = check_common(q, k_cache, v_cache, out, num_q_heads, num_kv_heads, head_dim,
                        k_cache_stride0, v_cache_stride0, dtype, /*f16_ok=*/true);
  if (rc != MSGL_OK) return rc;
  const int64_t group = num_q_heads / num_kv_heads;
  if (group > 16) return MSGL_ERR_GROUP_TOO_LARGE;  // paged_decode_attention.cpp:54-57
  if (!kv_indptr || !num_kv_splits || (total_kv > 0 && !kv_indices)) return MSGL_ERR_NULL_POINTER;
  (void)max_kv_splits;  // split hints do not steer the cut (result is split-invariant)
  const int32_t n_seg = segments(total_kv, num_kv_heads, head_dim, group);
  const size_t need =
      msgl::splitkv_workspace_bytes(batch, num_q_heads, num_kv_heads, head_dim, 1, n_seg);
  if (builtin_scratch) {
    rc = msgl::splitkv_scratch(&workspace, &workspace_bytes);
    if (rc != MSGL_OK) return rc;
    if (need > workspace_bytes) return MSGL_ERR_SCRATCH_LIMIT;
  }
  if (!workspace || workspace_bytes < need || !aligned16(workspace)) return MSGL_ERR_WORKSPACE;
  msgl::SplitKvArgs a{};
  a.q = q;
  a.k_cache = k_cache;
  a.v_cache = v_cache;
  a.kv_indptr = kv_indptr;
  a.kv_indices = kv_indices;
  a.qo_indptr = nullptr;
  a.prefix_lens = nullptr;
  a.out = out;
  a.workspace = workspace;
  a.batch = batch;
  a.total_kv = total_kv;
  a.n_q = num_q_heads;
  a.n_kv = num_kv_heads;
  a.head_dim = head_dim;
  a.num_slots = num_slots;
  a.k_stride0 = k_cache_stride0;
  a.v_stride0 = v_cache_stride0;
  a.sm_scale = sm_scale;
  a.max_len_extend = 1;
  a.f16 = (dtype == MSGL_DTYPE_F16) ? 1 : 0;
  a.is_cross = 0;
  a.window = 0;
  a.n_seg = n_seg;
  a.min_seg = min_segment(head_dim);
  return msgl::launch_splitkv(a, static_cast<hipStream_t>(stream));
}

int msgl_paged_decode_attention(const void* q, const void* k_cache, const void* v_cache,
                                const int32_t* kv_indptr, const int32_t* kv_indices,
                                const int32_t* num_kv_splits, void* out, void* workspace,
                                size_t workspace_bytes, int64_t batch, int64_t total_kv,
                                int64_t num_q_heads, int64_t num_kv_heads, int64_t head_dim,
                                int64_t num_slots, int64_t k_cache_stride0,
                                int64_t v_cache_stride0, float sm_scale, int32_t max_kv_splits,
                                int32_t dtype, void* stream) {
  return decode_attention(q, k_cache, v_cache, kv_indptr, kv_indices, num_kv_splits, out, workspace,
                          workspace_bytes, false, batch, total_kv, num_q_heads, num_kv_heads,
                          head_dim, num_slots, k_cache_stride0, v_cache_stride0, sm_scale,
                          max_kv_splits, dtype, stream);
}

int msgl_paged_decode_attention_noalloc(const void* q, const void* k_cache, const void* v_cache,
                                        const int32_t* kv_indptr, const int32_t* kv_indices,
                                        const int32_t* num_kv_splits, void* out, int64_t batch,
                                        int64_t total_kv, int64_t num_q_heads,
                                        int64_t num_kv_heads, int64_t head_dim, int64_t num_slots,
                                        int64_t k_cache_stride0, int64_t v_cache_stride0,
                                        float sm_scale, int32_t max_kv_splits, int32_t dtype,
                                        void* stream) {
  return decode_attention(q, k_cache, v_cache, kv_indptr, kv_indices, num_kv_splits, out, nullptr,
                          0, true, batch, total_kv, num_q_heads, num_kv_heads, head_dim, num_slots,
                          k_cache_stride0, v_cache_stride0, sm_scale, max_kv_splits, dtype, stream);
}

// Ragged key shares for the tile kernels (one query block per (request, kv head)): the ping-pong
// kernel and the head_dim 256 kernel know them, the fused head_dim 128 kernels do not.
static int ragged_tiles(int64_t batch, int64_t total_kv, int64_t n_kv, int64_t group,
                        int64_t max_len_extend, int64_t head_dim) {
  if (head_dim == 128 && msgl::tile_variant() != 0) return 0;
  return msgl::prefill_ragged_tiles(batch, total_kv, n_kv, group, max_len_extend,
                                    msgl::prefill_block_rows(head_dim), t_key_splits);
}

// Gang ranges for the head_dim 128 ping-pong kernel (several query blocks per (request, kv head)).
static int gangs_for(int64_t batch, int64_t total_kv, int64_t n_kv, int64_t group, int64_t max_len_extend,
                     int64_t head_dim, int64_t window, int key_splits) {
  if (head_dim != 128 || msgl::tile_variant() != 0 || t_gangs < 0) return 0;
  return msgl::prefill_gangs(batch, total_kv, n_kv, group, max_len_extend, window, msgl::kPrefillBlockRows,
                             t_gangs > 0 ? 1 : key_splits, t_key_splits, /*whatever_the_size=*/t_gangs > 0);
}

static bool use_splitkv_route(int64_t group, int64_t max_len_extend, int64_t head_dim, int64_t batch,
                              int64_t total_kv, int64_t n_kv) {
  const int64_t cols = group * max_len_extend;
  if (max_len_extend < 1 || cols > msgl::kSplitKvMaxCols) return false;
  const int64_t t = t_tune[MSGL_TUNE_SMALLQ_MAXCOLS];
  if (t != 0) return t > 0 && cols <= t;  // set by hand; negative: never
  if (cols <= smallq_base_cols(head_dim)) return true;
  return ragged_tiles(batch, total_kv, n_kv, group, max_len_extend, head_dim) == 0;
}
// Under a sliding window that most requests exceed (mean kv length at least twice the window),
// every request shows about `window` keys, the one case where one workgroup per (request, kv
// head) is balanced: the tile kernel then streams 5-20 % faster than the split-K kernel from
// 17 columns on (shape 5 with a window of 1024: 32 against 36 us).  Only the default routing
// does this; MSGL_TUNE_SMALLQ_MAXCOLS set by hand is obeyed as it stands.
static bool window_prefers_tiles(int64_t batch, int64_t total_kv, int64_t n_kv, int64_t group,
                                 int64_t max_len_extend, int64_t head_dim, int64_t window) {
  if (window <= 0 || head_dim != 128 || t_tune[MSGL_TUNE_SMALLQ_MAXCOLS] != 0) return false;
  if (group * max_len_extend <= 16) return false;
  if (total_kv < 2 * batch * (window + max_len_extend)) return false;
  return ragged_tiles(batch, total_kv, n_kv, group, max_len_extend, head_dim) > 0;
}

size_t msgl_paged_prefill_workspace_bytes(int64_t batch, int64_t total_q, int64_t total_kv,
                                          int64_t num_q_heads, int64_t num_kv_heads,
                                          int64_t head_dim, int64_t max_len_extend) {
  if (batch <= 0 || total_q < 0 || total_kv < 0 || num_q_heads <= 0 || num_kv_heads <= 0 ||
      num_q_heads % num_kv_heads != 0)
    return 0;
  const int64_t group = num_q_heads / num_kv_heads;
  if (!use_splitkv_route(group, max_len_extend, head_dim, batch, total_kv, num_kv_heads)) {
    // tile kernels: partials of a key split, if this launch would use one (a sliding window,
    // unknown here, can only lower the count)
    const int ragged = ragged_tiles(batch, total_kv, num_kv_heads, group, max_len_extend, head_dim);
    if (ragged > 0)
      return msgl::prefill_ragged_workspace_bytes(batch, total_kv, num_kv_heads, group,
                                                  max_len_extend, head_dim, ragged);
    const int k = msgl::prefill_key_splits(batch, total_kv, num_kv_heads, group, max_len_extend, 0,
                                           msgl::prefill_block_rows(head_dim), t_key_splits);
    const int gangs = gangs_for(batch, total_kv, num_kv_heads, group, max_len_extend, head_dim, 0, k);
    const size_t split_need = msgl::prefill_split_workspace_bytes(total_q, num_q_heads, head_dim, k);
    if (gangs > 0)
      return std::max(split_need, msgl::prefill_gang_workspace_bytes(batch, num_kv_heads, group, max_len_extend, gangs));
    return split_need;
  }
  const size_t split_need = msgl::splitkv_workspace_bytes(
      batch, num_q_heads, num_kv_heads, head_dim, max_len_extend,
      segments(total_kv, num_kv_heads, head_dim, group * max_len_extend));
  // a sliding window (unknown here) may send the launch to the tile kernel instead
  const int ragged = ragged_tiles(batch, total_kv, num_kv_heads, group, max_len_extend, head_dim);
  const size_t tile_need = ragged > 0 ? msgl::prefill_ragged_workspace_bytes(batch, total_kv, num_kv_heads, group,
                                                                             max_len_extend, head_dim, ragged)
                                      : 0;
  return std::max(split_need, tile_need);
}

int msgl_paged_prefill_attention(const void* q, const void* k_cache, const void* v_cache,
                                 const int32_t* qo_indptr, const int32_t* kv_indptr,
                                 const int32_t* kv_indices, const int32_t* prefix_lens, void* out,
                                 void* workspace, size_t workspace_bytes, int64_t batch,
                                 int64_t total_q, int64_t total_kv, int64_t num_q_heads,
                                 int64_t num_kv_heads, int64_t head_dim, int64_t num_slots,
                                 int64_t k_cache_stride0, int64_t v_cache_stride0, float sm_scale,
                                 int32_t max_len_extend, int32_t is_cross_attention,
                                 int32_t sliding_window_size, int32_t dtype, void* stream) {
  if (head_dim != 128 && head_dim != 256) return MSGL_ERR_HEAD_DIM;
  if (num_q_heads <= 0 || num_kv_heads <= 0) return MSGL_ERR_SHAPE;
  if (num_q_heads % num_kv_heads != 0) return MSGL_ERR_HEAD_RATIO;
  if (sliding_window_size < 0) return MSGL_ERR_WINDOW;  // paged_prefill_attention.cpp:67-70
  if (batch <= 0) return MSGL_ERR_BATCH;                // :74-77
  if (total_q < 0 || total_kv < 0 || num_slots < 0) return MSGL_ERR_SHAPE;
  if (total_q == 0 || max_len_extend <= 0) return MSGL_OK;
  int rc = check_common(q, k_cache, v_cache, out, num_q_heads, num_kv_heads, head_dim,
                        k_cache_stride0, v_cache_stride0, dtype, /*f16_ok=*/false);
  if (rc != MSGL_OK) return rc;
  if (!qo_indptr || !kv_indptr || !prefix_lens || (total_kv > 0 && !kv_indices))
    return MSGL_ERR_NULL_POINTER;
  const int64_t group = num_q_heads / num_kv_heads;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const bool direct = use_splitkv_route(group, max_len_extend, head_dim, batch, total_kv, num_kv_heads) &&
                      !window_prefers_tiles(batch, total_kv, num_kv_heads, group, max_len_extend, head_dim,
                                            sliding_window_size);
  if (direct) {
    const int32_t n_seg = segments(total_kv, num_kv_heads, head_dim, group * max_len_extend);
    const size_t need = msgl::splitkv_workspace_bytes(batch, num_q_heads, num_kv_heads, head_dim,
                                                      max_len_extend, n_seg);
    if (!workspace || workspace_bytes < need || !aligned16(workspace)) return MSGL_ERR_WORKSPACE;
    msgl::SplitKvArgs a{};
    a.q = q;
    a.k_cache = k_cache;
    a.v_cache = v_cache;
    a.kv_indptr = kv_indptr;
    a.kv_indices = kv_indices;
    a.qo_indptr = qo_indptr;
    a.prefix_lens = prefix_lens;
    a.out = out;
    a.workspace = workspace;
    a.batch = batch;
    a.total_kv = total_kv;
    a.n_q = num_q_heads;
    a.n_kv = num_kv_heads;
    a.head_dim = head_dim;
    a.num_slots = num_slots;
    a.k_stride0 = k_cache_stride0;
    a.v_stride0 = v_cache_stride0;
    a.sm_scale = sm_scale;
    a.max_len_extend = max_len_extend;
    a.q_cap = max_len_extend;
    a.is_cross = is_cross_attention ? 1 : 0;
    a.window = sliding_window_size;
    a.n_seg = n_seg;
    a.min_seg = min_segment(head_dim);
    a.q_begin = 0;
    return msgl::launch_splitkv(a, s);
  }
  msgl::PrefillArgs a{};
  a.q = q;
  a.k_cache = k_cache;
  a.v_cache = v_cache;
  a.qo_indptr = qo_indptr;
  a.kv_indptr = kv_indptr;
  a.kv_indices = kv_indices;
  a.prefix_lens = prefix_lens;
  a.out = out;
  a.batch = batch;
  a.total_q = total_q;
  a.total_kv = total_kv;
  a.n_q = num_q_heads;
  a.n_kv = num_kv_heads;
  a.head_dim = head_dim;
  a.num_slots = num_slots;
  a.k_stride0 = k_cache_stride0;
  a.v_stride0 = v_cache_stride0;
  a.sm_scale = sm_scale;
  a.max_len_extend = max_len_extend;
  a.is_cross = is_cross_attention ? 1 : 0;
  a.window = sliding_window_size;
  a.key_splits = 1;
  a.ragged_tiles = ragged_tiles(batch, total_kv, num_kv_heads, group, max_len_extend, head_dim);
  if (a.ragged_tiles > 0) {
    // ragged shares need room for their partials; without it the keys go in one pass
    const size_t need = msgl::prefill_ragged_workspace_bytes(batch, total_kv, num_kv_heads, group,
                                                             max_len_extend, head_dim, a.ragged_tiles);
    if (need > 0 && (!workspace || workspace_bytes < need || !aligned16(workspace))) a.ragged_tiles = 0;
    else a.workspace = workspace;
  } else {
    a.key_splits = msgl::prefill_key_splits(batch, total_kv, num_kv_heads, group, max_len_extend,
                                            sliding_window_size, msgl::prefill_block_rows(head_dim),
                                            t_key_splits);
  }
  if (a.key_splits > 1) {
    // the split is an optimisation: without room for its partials the keys go in one pass
    const size_t need = msgl::prefill_split_workspace_bytes(total_q, num_q_heads, head_dim, a.key_splits);
    if (!workspace || workspace_bytes < need || !aligned16(workspace)) a.key_splits = 1;
    else a.workspace = workspace;
  }
  a.gangs = 0;
  if (t_gangs > 0 && a.ragged_tiles == 0) a.key_splits = 1;  // forced for a test: gang ranges instead
  if (a.ragged_tiles == 0 && a.key_splits == 1) {
    const int gangs = gangs_for(batch, total_kv, num_kv_heads, group, max_len_extend, head_dim,
                                sliding_window_size, a.key_splits);
    // so are gang ranges: without room for their slots every unit goes to one workgroup per query block
    if (gangs > 0 && workspace && aligned16(workspace) &&
        workspace_bytes >= msgl::prefill_gang_workspace_bytes(batch, num_kv_heads, group, max_len_extend, gangs)) {
      a.gangs = gangs;
      a.workspace = workspace;
      a.gang_nonce = g_gang_nonce.fetch_add(1, std::memory_order_relaxed) & ((1ull << 47) - 1);
      if (a.gang_nonce == 0) a.gang_nonce = g_gang_nonce.fetch_add(1, std::memory_order_relaxed);
    }
  }
  return head_dim == 256 ? msgl::launch_prefill_tile256(a, s) : msgl::launch_prefill_tile(a, s);
}

int msgl_copy_state_slots(void* slab, int64_t layer_stride_bytes, int64_t slot_stride_bytes,
                          int64_t row_bytes, int64_t n_layers, int64_t num_slots, const int32_t* src,
                          const int32_t* dst, int64_t n_pairs, void* stream) {
  if (n_layers < 0 || num_slots < 0 || n_pairs < 0 || row_bytes < 0 || slot_stride_bytes < row_bytes ||
      (n_layers > 1 && layer_stride_bytes < num_slots * slot_stride_bytes))
    return MSGL_ERR_SHAPE;
  if (n_layers == 0 || n_pairs == 0 || row_bytes == 0) return MSGL_OK;
  if (!slab || !dst) return MSGL_ERR_NULL_POINTER;
  return msgl::launch_state_slots(slab, layer_stride_bytes, slot_stride_bytes, row_bytes, n_layers,
                                  num_slots, src, dst, n_pairs, static_cast<hipStream_t>(stream));
}

int msgl_build_attention_metadata(const int32_t* page_table, int64_t table_stride0,
                                  int64_t n_table_rows, int64_t max_seq_len,
                                  const int32_t* table_rows, const int32_t* kv_lens,
                                  const int32_t* extend_lens, int64_t batch, int32_t* kv_indptr,
                                  int32_t* kv_indices, int64_t kv_capacity, int32_t* qo_indptr,
                                  int32_t* prefix_lens, int32_t* positions, int64_t q_capacity,
                                  int32_t* num_kv_splits, int32_t max_kv_splits, void* stream) {
  if (batch < 0 || batch > msgl::kMetadataMaxBatch || n_table_rows <= 0 || max_seq_len < 0 ||
      table_stride0 < max_seq_len || kv_capacity < 0 || q_capacity < 0 ||
      kv_capacity > 0x7fffffffLL || q_capacity > 0x7fffffffLL || max_seq_len > 0x7fffffffLL ||
      n_table_rows > 0x7fffffffLL)
    return MSGL_ERR_SHAPE;
  if (!kv_indptr) return MSGL_ERR_NULL_POINTER;
  if (batch > 0 && (!page_table || !table_rows || !kv_lens)) return MSGL_ERR_NULL_POINTER;
  if (kv_capacity > 0 && !kv_indices) return MSGL_ERR_NULL_POINTER;
  msgl::MetadataArgs a{};
  a.page_table = page_table;
  a.table_rows = table_rows;
  a.kv_lens = kv_lens;
  a.extend_lens = extend_lens;
  a.kv_indptr = kv_indptr;
  a.kv_indices = kv_indices;
  a.qo_indptr = qo_indptr;
  a.prefix_lens = prefix_lens;
  a.positions = positions;
  a.num_kv_splits = num_kv_splits;
  a.table_stride0 = table_stride0;
  a.batch = batch;
  a.n_table_rows = n_table_rows;
  a.max_seq_len = max_seq_len;
  a.kv_capacity = kv_capacity;
  a.q_capacity = positions ? q_capacity : 0;
  a.max_kv_splits = max_kv_splits;
  return msgl::launch_build_metadata(a, static_cast<hipStream_t>(stream));
}

int msgl_qk_norm_rope_store(const void* q, const void* k, const void* v, int64_t q_stride0,
                            int64_t k_stride0, int64_t v_stride0, const void* q_weight,
                            const void* k_weight, const int32_t* positions,
                            const int32_t* out_loc, void* q_out, void* k_cache, void* v_cache,
                            int64_t k_cache_stride0, int64_t v_cache_stride0, int64_t num_slots,
                            int64_t n_tokens, int64_t num_q_heads, int64_t num_kv_heads,
                            int64_t head_dim, float rms_norm_eps, float rope_base, int32_t dtype,
                            void* stream) {
  if (head_dim != 128 && head_dim != 256) return MSGL_ERR_HEAD_DIM;
  if (dtype != MSGL_DTYPE_BF16) return MSGL_ERR_DTYPE;
  if (n_tokens < 0 || num_q_heads <= 0 || num_kv_heads <= 0 || num_slots < 0) return MSGL_ERR_SHAPE;
  if (!(rope_base > 1.0f) || !(rms_norm_eps >= 0.0f)) return MSGL_ERR_SHAPE;
  if (q_stride0 < num_q_heads * head_dim || k_stride0 < num_kv_heads * head_dim ||
      v_stride0 < num_kv_heads * head_dim || k_cache_stride0 < num_kv_heads * head_dim ||
      v_cache_stride0 < num_kv_heads * head_dim)
    return MSGL_ERR_SHAPE;
  if (n_tokens == 0) return MSGL_OK;
  if (!q || !k || !v || !q_weight || !k_weight || !positions || !out_loc || !q_out || !k_cache ||
      !v_cache)
    return MSGL_ERR_NULL_POINTER;
  if (!aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(q_weight) ||
      !aligned16(k_weight) || !aligned16(q_out) || !aligned16(k_cache) || !aligned16(v_cache) ||
      q_stride0 % 8 || k_stride0 % 8 || v_stride0 % 8 || k_cache_stride0 % 8 || v_cache_stride0 % 8)
    return MSGL_ERR_ALIGNMENT;
  msgl::NormRopeArgs a{};
  a.q = q;
  a.k = k;
  a.v = v;
  a.q_weight = q_weight;
  a.k_weight = k_weight;
  a.positions = positions;
  a.out_loc = out_loc;
  a.q_out = q_out;
  a.k_cache = k_cache;
  a.v_cache = v_cache;
  a.q_stride0 = q_stride0;
  a.k_stride0 = k_stride0;
  a.v_stride0 = v_stride0;
  a.kc_stride0 = k_cache_stride0;
  a.vc_stride0 = v_cache_stride0;
  a.n_tokens = n_tokens;
  a.num_slots = num_slots;
  a.n_q = num_q_heads;
  a.n_kv = num_kv_heads;
  a.head_dim = head_dim;
  a.eps = rms_norm_eps;
  a.rope_base = rope_base;
  return msgl::launch_qk_norm_rope_store(a, static_cast<hipStream_t>(stream));
}

int msgl_gdn_state_inplace(const void* q, const void* k, const void* v, const void* g,
                           const void* beta, void* state, const int32_t* slot_ids,
                           const int32_t* qo_indptr, void* y, int64_t tokens, int64_t batch,
                           int64_t hk, int64_t hv, int64_t dk, int64_t dv, int64_t num_slots,
                           int64_t state_stride0, int64_t q_stride0, int64_t k_stride0,
                           int64_t v_stride0, int32_t single_token_mode, void* stream) {
  if (dk != 128 || dv != 128) return MSGL_ERR_GDN_DIMS;  // gdn_state.cpp:80-83
  if (tokens < 0 || batch < 0 || hk <= 0 || hv <= 0 || num_slots < 0) return MSGL_ERR_SHAPE;
  if (hv % hk != 0) return MSGL_ERR_HEAD_RATIO;          // gdn_state.cpp:76-79
  if (single_token_mode && tokens != batch) return MSGL_ERR_SHAPE;  // :107-111
  if (state_stride0 < hv * dv * dk || q_stride0 < hk * dk || k_stride0 < hk * dk ||
      v_stride0 < hv * dv)
    return MSGL_ERR_SHAPE;
  if (tokens == 0 || batch == 0) return MSGL_OK;
  if (!q || !k || !v || !g || !beta || !state || !slot_ids || !y) return MSGL_ERR_NULL_POINTER;
  if (!single_token_mode && !qo_indptr) return MSGL_ERR_NULL_POINTER;
  if (!aligned16(q) || !aligned16(k) || !aligned16(state) || q_stride0 % 8 || k_stride0 % 8 ||
      state_stride0 % 4)
    return MSGL_ERR_ALIGNMENT;
  msgl::GdnArgs a{};
  a.q = q;
  a.k = k;
  a.v = v;
  a.g = g;
  a.beta = beta;
  a.state = state;
  a.slot_ids = slot_ids;
  a.qo_indptr = qo_indptr;
  a.y = y;
  a.tokens = tokens;
  a.batch = batch;
  a.hk = hk;
  a.hv = hv;
  a.state_stride0 = state_stride0;
  a.q_stride0 = q_stride0;
  a.k_stride0 = k_stride0;
  a.v_stride0 = v_stride0;
  a.single_token_mode = single_token_mode;
  return msgl::launch_gdn_state(a, static_cast<hipStream_t>(stream));
}

}  // extern "C"
