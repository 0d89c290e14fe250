// Kernel parameter block and launch geometry shared by the prefill tile kernels.
#pragma once
#include "msgl_internal.h"

namespace msgl {

struct PrefillParams {
  const uint16_t* q;
  const uint16_t* k_cache;
  const uint16_t* v_cache;
  const int32_t* qo_indptr;
  const int32_t* kv_indptr;
  const int32_t* kv_indices;
  const int32_t* prefix_lens;
  uint16_t* out;
  int64_t k_stride0, v_stride0;
  int32_t batch, n_q, n_kv, group;
  int32_t n_qblk, n_pairs;  // q blocks per (request, kv head); batch * n_kv
  int32_t xcds_per_unit;    // see prefill_xcds_per_unit()
  int32_t max_len_extend, is_cross, window;
  float scale_log2e;
  uint32_t max_slot;  // num_slots - 1: slot ids are clamped to it before they become addresses
  // key splits: each workgroup takes one contiguous share of its rows' visible keys
  // and leaves a normalised fp32 partial and a base-2 log-sum-exp per row for the merge kernel
  int32_t n_ksplit;
  int64_t part_rows;  // total_q * n_q: rows of one split's partial
  float* part_o;      // [n_ksplit][part_rows][head_dim]
  float* part_lse;    // [n_ksplit][part_rows]
  // ragged shares (see prefill_ragged_tiles()): a request's keys in shares of `ragged_tiles` tiles,
  // as many as it needs; partials are then [unit][kv head][row of the block], a unit being one
  // (request, share), and req_units[2 b], [2 b + 1] = request b's first unit and unit count
  int32_t ragged_tiles, ragged_units, ragged_rows;
  int32_t* req_units;
  // gang ranges (see prefill_gangs()): `gangs` per XCD, 0 = off; cuts closer than `gang_snap`
  // tiles to either end of a (request, kv head) move to that end; a workgroup that ends up with
  // part of a unit's keys leaves its rows in `gang_slots` and counts itself in `gang_counts`
  int32_t gangs, gang_snap;
  float* gang_slots;
  unsigned long long* gang_counts;
  unsigned long long gang_nonce;
  long long* clock_probe;  // measurement aid, see ClockProbe; nullptr: off
};

constexpr int kBN = 64;  // keys per tile
// A stale row max is kept until the new one exceeds it by this much (base-2 exponent):
// P stays below 2^kLazy, far inside bf16 / fp32 range, and O is rescaled rarely.
constexpr float kLazy = 8.0f;
// Requests are processed longest first only up to this batch size: every workgroup ranks the
// requests itself (batch^2 comparisons spread over its threads), which stops paying when there
// are many of them.
constexpr int kRankedBatch = 128;
constexpr int kPrefillBlockRows = 256;      // rows per workgroup, head_dim 128
constexpr int kPrefillBlockRows256 = 128;   // head_dim 256
// Key splits: when (requests x kv heads x query blocks) cannot fill the chip, the keys of every
// query block are shared out over several workgroups.
constexpr int kComputeUnits = 256;
constexpr int kMaxKeySplits = 32;
constexpr int kMinKeysPerSplit = 1024;

inline int prefill_block_rows(int64_t head_dim) {
  return head_dim == 256 ? kPrefillBlockRows256 : kPrefillBlockRows;
}

// Workgroup ids go round the 8 XCDs.  A (request, kv head, key split) unit keeps all its query
// blocks on one XCD (they read the same keys: one L2 holds them), so units are dealt to the XCDs
// eight at a time.  The units left over when their number is no multiple of 8 would leave XCDs
// without work (a single request with 2 kv heads: 6 of 8), so up to 4 left-over units spread
// their query blocks over 8 / (their number rounded up to a power of two) XCDs each.
inline int prefill_xcds_per_unit(int64_t n_units) {
  const int64_t left = n_units % 8;
  if (left == 0 || left >= 5) return 1;
  return left == 1 ? 8 : (left == 2 ? 4 : 2);
}
// workgroups on the busiest XCD
inline int64_t prefill_blocks_per_xcd(int64_t n_units, int64_t n_qblk) {
  const int x = prefill_xcds_per_unit(n_units);
  const int64_t last_row = n_units % 8 == 0 ? 0 : (n_qblk + x - 1) / x;
  return n_units / 8 * n_qblk + last_row;
}

// Number of key splits for a launch, from sizes the host knows (the per-request lengths stay on
// the device: the average visible length stands for all of them).  Cost model: the (request, kv
// head, split) units are dealt round-robin to the 8 XCDs, a unit brings its query blocks, and an
// XCD runs its workgroups in rounds of one per compute unit; a split costs a few percent (its
// partial, the merge).  The count minimises rounds(k) / k * (1 + 0.03 (k - 1)); launches of more
// than four rounds are left alone.  `forced` > 0 overrides (clamped to kMaxKeySplits).
inline int prefill_key_splits(int64_t batch, int64_t total_kv, int64_t n_kv, int64_t group,
                              int64_t max_len_extend, int64_t window, int block_rows,
                              int64_t forced) {
  if (forced > 0) return (int)(forced < kMaxKeySplits ? forced : kMaxKeySplits);
  if (batch <= 0) return 1;
  constexpr int64_t kXcds = 8, kUnitsPerXcd = kComputeUnits / kXcds;
  const int64_t n_qblk = (max_len_extend * group + block_rows - 1) / block_rows;
  const int64_t pairs = batch * n_kv;
  auto rounds = [&](int64_t k) {
    const int64_t blocks = prefill_blocks_per_xcd(pairs * k, n_qblk);  // on the busiest XCD
    return (blocks + kUnitsPerXcd - 1) / kUnitsPerXcd;
  };
  if (n_qblk <= 0 || rounds(1) > 4) return 1;
  int64_t keys = total_kv / batch;
  if (window > 0 && keys > window + max_len_extend) keys = window + max_len_extend;
  int64_t most = keys / kMinKeysPerSplit;
  if (most > kMaxKeySplits) most = kMaxKeySplits;
  int best = 1;
  double best_cost = (double)rounds(1);
  for (int64_t k = 2; k <= most; ++k) {
    const double cost = (double)rounds(k) / (double)k * (1.0 + 0.03 * (double)(k - 1));
    if (cost < best_cost) {
      best_cost = cost;
      best = (int)k;
    }
  }
  return best;
}

// Ragged shares, for launches with one query block per (request, kv head) (short query blocks:
// their cost is reading the keys).  Cutting every request's keys the same number of times makes
// the workgroups of a long request long; instead a share is `tiles` key tiles for every request,
// a request gets as many shares as it needs, and the workgroups find their (request, share) by a
// prefix sum over the requests' share counts, so the grid holds no empty workgroups beyond the
// rounding.  tiles = what gives about one workgroup per compute unit, at least kRaggedMinTiles.
// Returns 0 when the launch does not qualify.
// Every workgroup scans the share counts of all requests (LDS): up to 128 requests that is free,
// beyond it costs a workgroup 1.5-5 us, which pays only when the requests are long enough
// (mean of kRaggedLongMean keys or more: 512 requests of 1 K keys +5 %, but -40 % when one of
// them has 60 K; 1000 requests of 100 keys would lose 33 %).
constexpr int kRaggedFreeBatch = 128;
constexpr int kRaggedMaxBatch = 1024;
constexpr int kRaggedLongMean = 1024;
constexpr int kRaggedMinTiles = 8;  // 512 keys: 4-16 % faster than 16 on launches that leave CUs idle, 4 and 2 slower
inline int64_t prefill_tiles_bound(int64_t batch, int64_t total_kv) {
  return (total_kv + kBN - 1) / kBN + 2 * batch;  // sum over requests of their key tiles, at most
}
inline int prefill_ragged_tiles(int64_t batch, int64_t total_kv, int64_t n_kv, int64_t group,
                                int64_t max_len_extend, int block_rows, int64_t forced_splits) {
  if (forced_splits > 0 || batch <= 0 || batch > kRaggedMaxBatch) return 0;
  if (batch > kRaggedFreeBatch && total_kv < (int64_t)kRaggedLongMean * batch) return 0;
  if (max_len_extend * group > block_rows) return 0;
  int64_t t = (prefill_tiles_bound(batch, total_kv) * n_kv + kComputeUnits - 1) / kComputeUnits;
  if (t < kRaggedMinTiles) t = kRaggedMinTiles;
  return (int)(t < (1 << 20) ? t : (1 << 20));
}
// (request, share) units a launch can have at most
inline int64_t prefill_ragged_units(int64_t batch, int64_t total_kv, int tiles) {
  return prefill_tiles_bound(batch, total_kv) / tiles + batch;
}
// no request can need a second share: nothing to merge, no workspace
inline bool prefill_ragged_never_splits(int64_t batch, int64_t total_kv, int tiles) {
  return prefill_tiles_bound(batch, total_kv) <= tiles;
}
inline size_t prefill_ragged_workspace_bytes(int64_t batch, int64_t total_kv, int64_t n_kv, int64_t group,
                                             int64_t max_len_extend, int64_t head_dim, int tiles) {
  if (tiles <= 0 || prefill_ragged_never_splits(batch, total_kv, tiles)) return 0;
  const size_t rows = (size_t)prefill_ragged_units(batch, total_kv, tiles) * (size_t)n_kv *
                      (size_t)(max_len_extend * group);
  return rows * (size_t)(head_dim + 1) * sizeof(float) + (size_t)batch * 2 * sizeof(int32_t);
}

// Gang ranges, for launches with several query blocks per (request, kv head) (chunked extends on
// long prefixes: their cost is the MFMA work, and it differs from unit to unit with the prefix).
// One workgroup per compute unit stays for the whole launch.  The 32 workgroups on an XCD form
// 32 / n_qblk gangs; a gang's workgroups take the query blocks of one unit side by side (they read
// the same keys at the same time: one L2 serves them) and the gangs share the XCD's units by
// length: the units' key tiles, laid end to end, are cut into equal ranges, one per gang, so
// every gang has the same MFMA work whatever the prefix lengths are.  A unit that a cut goes
// through is finished by the gang that gets there last: each of its parts leaves unnormalised
// rows, row maxima and row sums in its slot and counts itself; the part that counts last adds the
// others to its registers and writes the result.  Returns gangs per XCD, 0 when the launch does
// not qualify (the host knows sizes, not lengths).
constexpr int kGangMaxUnits = 256;   // units per XCD
constexpr int kGangMinTiles = 48;    // key tiles per gang below which one pass per unit is kept
inline int prefill_gangs(int64_t batch, int64_t total_kv, int64_t n_kv, int64_t group,
                         int64_t max_len_extend, int64_t window, int block_rows, int key_splits,
                         int64_t forced_splits, bool whatever_the_size = false) {
  if (forced_splits > 0 || key_splits > 1 || window > 0 || batch <= 0 || batch > kRankedBatch) return 0;
  const int64_t n_qblk = (max_len_extend * group + block_rows - 1) / block_rows;
  constexpr int64_t kUnitsPerXcd = kComputeUnits / 8;
  if (n_qblk < 2 || n_qblk > 16 || kUnitsPerXcd % n_qblk != 0) return 0;
  const int64_t n_pairs = batch * n_kv;
  if (n_pairs % 8 != 0 || n_pairs / 8 > kGangMaxUnits) return 0;
  const int64_t gangs = kUnitsPerXcd / n_qblk;
  if (whatever_the_size) return (int)gangs;
  if (n_pairs / 8 < gangs) return 0;  // fewer units than gangs: key splits are the tool
  const int64_t tiles_per_xcd = prefill_tiles_bound(batch, total_kv) * n_kv / 8;
  if (tiles_per_xcd < gangs * kGangMinTiles) return 0;
  return (int)gangs;
}
constexpr size_t kGangSlotBytes = (size_t)kPrefillBlockRows * 128 * sizeof(float) + 8 * 64 * 2 * sizeof(float);
inline size_t prefill_gang_workspace_bytes(int64_t batch, int64_t n_kv, int64_t group,
                                           int64_t max_len_extend, int gangs) {
  if (gangs <= 0) return 0;
  const int64_t n_qblk = (max_len_extend * group + kPrefillBlockRows - 1) / kPrefillBlockRows;
  const size_t slots = (size_t)8 * gangs * 2 * n_qblk;
  const size_t counts = (size_t)batch * n_kv * n_qblk;
  return slots * kGangSlotBytes + (counts * sizeof(unsigned long long) + 255) / 256 * 256;
}

inline size_t prefill_split_workspace_bytes(int64_t total_q, int64_t n_q, int64_t head_dim, int n_ksplit) {
  if (n_ksplit <= 1) return 0;
  return (size_t)n_ksplit * (size_t)total_q * (size_t)n_q * (size_t)(head_dim + 1) * sizeof(float);
}

// Combines the partials of a key-split launch into `out` (defined beside the head_dim 128 kernel).
int launch_prefill_merge(const struct PrefillParams& p, int head_dim, hipStream_t stream);

// Fills `p` and the grid size; returns MSGL_OK, or an error, or sets n_blocks = 0 for an
// empty problem.  wide: some pool byte offset needs more than 32 bits.
inline int make_prefill_params(const PrefillArgs& a, PrefillParams& p, int64_t& n_blocks, bool& wide,
                               int block_rows = kPrefillBlockRows) {
  p.q = static_cast<const uint16_t*>(a.q);
  p.k_cache = static_cast<const uint16_t*>(a.k_cache);
  p.v_cache = static_cast<const uint16_t*>(a.v_cache);
  p.qo_indptr = a.qo_indptr;
  p.kv_indptr = a.kv_indptr;
  p.kv_indices = a.kv_indices;
  p.prefix_lens = a.prefix_lens;
  p.out = static_cast<uint16_t*>(a.out);
  p.k_stride0 = a.k_stride0;
  p.v_stride0 = a.v_stride0;
  p.batch = (int32_t)a.batch;
  p.n_q = (int32_t)a.n_q;
  p.n_kv = (int32_t)a.n_kv;
  p.group = (int32_t)(a.n_q / a.n_kv);
  p.max_len_extend = a.max_len_extend;
  p.is_cross = a.is_cross;
  p.window = a.window;
  p.scale_log2e = a.sm_scale * 1.4426950408889634f;
  p.max_slot = (uint32_t)(a.num_slots > 0 ? a.num_slots - 1 : 0);
  p.n_ksplit = a.key_splits > 1 ? a.key_splits : 1;
  p.part_rows = a.total_q * a.n_q;
  p.part_o = static_cast<float*>(a.workspace);
  p.part_lse = p.part_o ? p.part_o + (int64_t)p.n_ksplit * p.part_rows * a.head_dim : nullptr;
  if (p.n_ksplit > 1 && !p.part_o) return MSGL_ERR_WORKSPACE;
  const int64_t rows = (int64_t)a.max_len_extend * p.group;
  const int64_t n_qblk = (rows + block_rows - 1) / block_rows;
  const int64_t n_pairs = a.batch * a.n_kv;
  p.ragged_tiles = 0;
  p.ragged_units = 0;
  p.ragged_rows = 0;
  p.req_units = nullptr;
  p.gangs = 0;
  p.gang_snap = 0;
  p.gang_slots = nullptr;
  p.gang_counts = nullptr;
  p.gang_nonce = 0;
  p.clock_probe = clock_probe();
  if (a.ragged_tiles > 0 && n_qblk == 1) {
    const int64_t units = prefill_ragged_units(a.batch, a.total_kv, a.ragged_tiles);
    p.n_ksplit = 1;
    p.ragged_tiles = a.ragged_tiles;
    p.ragged_units = (int32_t)units;
    p.ragged_rows = (int32_t)rows;
    if (!prefill_ragged_never_splits(a.batch, a.total_kv, a.ragged_tiles)) {
      if (!a.workspace) return MSGL_ERR_WORKSPACE;
      const int64_t part_rows = units * a.n_kv * rows;
      p.part_rows = part_rows;
      p.part_o = static_cast<float*>(a.workspace);
      p.part_lse = p.part_o + part_rows * a.head_dim;
      p.req_units = reinterpret_cast<int32_t*>(p.part_lse + part_rows);
    }
    n_blocks = units * a.n_kv;
    if (n_blocks > 0x7fffffffLL) return MSGL_ERR_SHAPE;
    p.n_qblk = 1;
    p.n_pairs = (int32_t)n_pairs;
    p.xcds_per_unit = 1;
    wide = (uint64_t)a.num_slots * (uint64_t)a.k_stride0 * 2u >= (1ull << 32) ||
           (uint64_t)a.num_slots * (uint64_t)a.v_stride0 * 2u >= (1ull << 32) ||
           a.num_slots >= (1 << 24) || a.k_stride0 * 2 >= (1 << 24) || a.v_stride0 * 2 >= (1 << 24);
    return MSGL_OK;
  }
  p.xcds_per_unit = prefill_xcds_per_unit(n_pairs * p.n_ksplit);
  n_blocks = 8 * prefill_blocks_per_xcd(n_pairs * p.n_ksplit, n_qblk);
  if (n_qblk <= 0 || n_blocks <= 0) {
    n_blocks = 0;
    return MSGL_OK;
  }
  if (n_blocks > 0x7fffffffLL) return MSGL_ERR_SHAPE;
  p.n_qblk = (int32_t)n_qblk;
  p.n_pairs = (int32_t)n_pairs;
  if (a.gangs > 0 && p.n_ksplit == 1 && block_rows == kPrefillBlockRows) {
    if (!a.workspace) return MSGL_ERR_WORKSPACE;
    p.gangs = a.gangs;
    // the last rows' diagonal lies in the last ceil(extend / 64) tiles of a unit: no cut goes there,
    // so every part of a unit holds keys that every row of every query block sees
    p.gang_snap = (int32_t)((a.max_len_extend + kBN - 1) / kBN + 2);
    const size_t slots = (size_t)8 * a.gangs * 2 * n_qblk;
    p.gang_slots = static_cast<float*>(a.workspace);
    p.gang_counts = reinterpret_cast<unsigned long long*>(static_cast<char*>(a.workspace) + slots * kGangSlotBytes);
    p.gang_nonce = a.gang_nonce;
    n_blocks = kComputeUnits;  // one workgroup per compute unit, 32 per XCD
  }
  // narrow offsets: slot * row_bytes fits 32 bits and both factors fit 24 bits (one
  // full-rate 24-bit multiply per row)
  wide = (uint64_t)a.num_slots * (uint64_t)a.k_stride0 * 2u >= (1ull << 32) ||
         (uint64_t)a.num_slots * (uint64_t)a.v_stride0 * 2u >= (1ull << 32) ||
         a.num_slots >= (1 << 24) || a.k_stride0 * 2 >= (1 << 24) || a.v_stride0 * 2 >= (1 << 24);
  return MSGL_OK;
}

}  // namespace msgl
