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
  int32_t max_len_extend, is_cross, window;
  float scale_log2e;
#ifdef MSGL_PROFILE_PHASES
  long long* prof;  // [blocks][waves][8] cycle totals
#endif
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
  const int64_t rows = (int64_t)a.max_len_extend * p.group;
  const int64_t n_qblk = (rows + block_rows - 1) / block_rows;
  const int64_t n_pairs = a.batch * a.n_kv;
  n_blocks = (n_pairs + 7) / 8 * 8 * n_qblk;
  if (n_qblk <= 0 || n_blocks <= 0) {
    n_blocks = 0;
    return MSGL_OK;
  }
  if (n_blocks > 0x7fffffffLL) return MSGL_ERR_SHAPE;
  p.n_qblk = (int32_t)n_qblk;
  p.n_pairs = (int32_t)n_pairs;
  // narrow offsets: slot * row_bytes fits 32 bits and both factors fit 24 bits (one
  // full-rate 24-bit multiply per row)
  wide = (uint64_t)a.num_slots * (uint64_t)a.k_stride0 * 2u >= (1ull << 32) ||
         (uint64_t)a.num_slots * (uint64_t)a.v_stride0 * 2u >= (1ull << 32) ||
         a.num_slots >= (1 << 24) || a.k_stride0 * 2 >= (1 << 24) || a.v_stride0 * 2 >= (1 << 24);
  return MSGL_OK;
}

}  // namespace msgl
