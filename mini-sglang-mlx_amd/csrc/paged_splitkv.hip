// Bandwidth-bound paged attention for short query blocks on gfx950: single-token GQA
// decode (paged_decode_attention) and the q_len <= a-few-tokens route of
// paged_prefill_attention (speculative verify, draft proposal).
//
// Replaces paged_decode_attention_stage1 / _stage2
// (mini-sglang-mlx-kernel/csrc/paged_decode_attention.metal:313-586) and, for short
// extends, paged_prefill_attention (paged_prefill_attention.metal:382-640).
//
// Work decomposition
//   The visible keys of all requests, in CSR order, form one token stream.  It is cut
//   into `n_seg` equal segments (the count is chosen on the host: workgroups for 13 of every
//   16 CUs, all resident at once, one round, no tail; the HBM system, not the CUs, is the limit).
//   A workgroup owns one segment and `nwh` adjacent kv heads, one wave64 per head; all
//   waves walk the same tokens, so the workgroup touches nwh*256-byte stretches of every
//   slot row together.  A wave holds up to two tiles of 16 columns; shapes with more
//   columns add a second wave per head (measured: a second wave re-reading the rows costs
//   about as much as reading them from HBM, so columns stay in one wave when they fit).
//   A segment may
//   cross request boundaries: the wave finishes one request's share (writing bf16 output
//   directly if it covered the whole request, otherwise a normalised fp32 partial + base-2
//   LSE) and continues with the next.  splitkv_merge_kernel combines the partials.
//   The host never reads device metadata: every wave derives its segment from kv_indptr
//   (and qo_indptr / prefix_lens) with a wave-wide prefix sum.
//
// Inner product shapes (one wave, one kv head)
//   columns    = the q rows sharing this kv head: col = q_idx * group + head_in_group,
//                padded to NCT tiles of 16 (the MFMA N dimension).  Every K / V row is
//                read once per kv head, whatever the group size or q_len.
//   S^T        = K_tile (16 tokens x D) * Q^T        -> mfma 16x16x32, tokens on M
//   O^T       += V_tile^T (D x 32 tokens) * P^T      -> mfma 16x16x32, tokens on K
//   Both products keep "column" on l%16 of the accumulator, so the softmax state, the
//   P operand and the O rescale stay lane-local; the only cross-lane traffic per tile is
//   the column max (two xor-shuffles).
//   V rows are loaded as whole 16-byte segments (16 lanes cover one 256-byte row) and
//   turned into the token-contiguous MFMA operand by an in-lane 8x8 transpose of 16-bit
//   values (v_perm_b32); the token order inside an MFMA is chosen so that it matches the
//   accumulator layout of S^T, which is legal because the contraction is a sum.
//
// Algorithmic HBM bytes per visible token and kv head: 2 * D * 2 (one K row + one V row)
// plus 4 bytes of kv_indices per token.
#include <atomic>
#include <type_traits>

#include "msgl_device.h"
#include "msgl_internal.h"

namespace msgl {
namespace {

struct SplitKvParams {
  const uint16_t* q;
  const uint16_t* k_cache;
  const uint16_t* v_cache;
  const int32_t* kv_indptr;
  const int32_t* kv_indices;
  const int32_t* qo_indptr;
  const int32_t* prefix_lens;
  uint16_t* out;
  float* part_o;        // [n_seg + batch][n_kv][D / 8][cols][8], fp32 or IEEE half: see partial_offset()
  float* part_lse;      // [n_seg + batch][n_kv][cols]
  int32_t* req_items;   // [batch][2] first segment holding the request, number of segments sharing it
  int64_t k_stride0, v_stride0;
  int32_t batch, n_q, n_kv, group;
  int32_t nwh;          // kv heads per workgroup
  int32_t head_groups;  // n_kv / nwh
  int32_t n_seg, min_seg, cols, max_len_extend;
  int32_t boundary;  // stream positions a request boundary is charged with (see stream_length)
  int32_t q_begin, q_cap;  // first query of every request in this launch; cap on a request's queries
  int32_t f16;             // elements are IEEE half instead of bf16
  int32_t is_cross, window;
  int32_t wide;  // pool byte offsets need 64 bits
  uint32_t max_slot;  // num_slots - 1: slot ids are clamped to it before they become addresses
  float scale_log2e;
  long long* clock_probe;  // measurement aid, see ClockProbe; nullptr: off
};

// Visible key range and query geometry of one request.
struct ReqInfo {
  int32_t kv_start, kv_len;  // CSR segment
  int32_t q_start, q_len;    // rows of q / out
  int32_t prefix;            // position of query 0
  int32_t lo, hi;            // keys [lo, hi) can be visible to some query of the request
};

__device__ __forceinline__ ReqInfo request_info(const SplitKvParams& p, int b) {
  ReqInfo r;
  r.kv_start = p.kv_indptr[b];
  r.kv_len = p.kv_indptr[b + 1] - r.kv_start;
  if (r.kv_len < 0) r.kv_len = 0;
  if (p.qo_indptr == nullptr) {
    r.q_start = b;
    r.q_len = 1;
    r.prefix = r.kv_len - 1;
  } else {
    // this launch covers queries q_begin .. q_begin + max_len_extend - 1 of every request
    const int q0 = p.qo_indptr[b];
    const int q_all = min(p.qo_indptr[b + 1] - q0, p.q_cap);
    r.q_start = q0 + p.q_begin;
    r.q_len = max(min(q_all - p.q_begin, p.max_len_extend), 0);
    r.prefix = p.prefix_lens[b] + p.q_begin;
  }
  // first query has the lowest window floor, last query the highest causal limit
  r.lo = (p.window > 0) ? max(0, r.prefix - p.window + 1) : 0;
  r.lo &= ~15;
  r.hi = p.is_cross ? r.kv_len : min(r.kv_len, r.prefix + r.q_len);
  if (r.q_len <= 0 || r.hi <= r.lo) {
    r.lo = 0;
    r.hi = 0;
  }
  return r;
}

// Element type of the partials.  bf16 launches keep them as IEEE half: a normalised partial row is
// a weighted mean of V rows, every bf16 value of ordinary size is a half value exactly (a share
// that holds all of a row's weight hands the V row on unchanged), and half's 11 significant bits
// are 8 times finer than the bf16 result the merge rounds to.  Values are clamped to half's range,
// far beyond any V a bf16 cache holds in practice.  The partials are 2.5 % of the bytes at eight
// queries a request but 7 % of the time (their stores compete with everybody's reads); halved,
// the verify shape gains 3 %.  (16-bit fixed point against the row's largest element is finer on
// rows that average many keys and coarser on a row's small elements: a copied V row then is no
// longer exact.)  IEEE-half launches, whose results are as fine as such a partial, keep fp32.
typedef _Float16 f16x8s_t __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2s_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pack_half2_clamped(float lo, float hi) {
  f16x2s_t v;
  v[0] = (_Float16)__builtin_fminf(__builtin_fmaxf(lo, -65504.f), 65504.f);
  v[1] = (_Float16)__builtin_fminf(__builtin_fmaxf(hi, -65504.f), 65504.f);
  return __builtin_bit_cast(uint32_t, v);
}

// Where dim `dim` of column `col` of the partial of (item, kv head) number `block` lives.  Blocks
// of 8 dims are the outer index and columns the inner one: in the attention kernel's accumulator
// layout the 16 lanes of a row group hold the same 8 dims of 16 consecutive columns, so one store
// instruction writes 32 contiguous bytes per lane and 512 contiguous bytes per row group.  (With
// the column as the outer index every lane of a store wrote 16 bytes of a different 512-byte row:
// 64 partial cache lines per instruction, and the partial stores of a share cost as much as
// several microseconds of streaming.)
__device__ __forceinline__ int64_t partial_offset(int64_t block, int cols, int col, int dim, int D) {
  return (block * cols * (int64_t)D) + ((int64_t)(dim >> 3) * cols + col) * 8 + (dim & 7);
}

// A request with visible keys takes their number of positions in the stream plus `boundary`
// positions without tokens behind them.  Starting on the next request costs a workgroup a fixed
// time (its geometry, Q rows, slot ids and first tiles are three dependent memory round trips, and
// the load pipeline drains and refills): measured 8-9 us, the time of about a hundred tokens, and the
// kernel ends when its slowest workgroup does.  Charging the boundary to the segment that crosses it
// gives that workgroup fewer tokens; a segment that ends or starts inside the empty positions just
// has less to do or starts at the next request.
__device__ __forceinline__ int stream_length(const SplitKvParams& p, int visible) {
  return visible > 0 ? visible + p.boundary : 0;
}

// Segments are a multiple of 64 positions long, one trip of the tile loop.  (Multiples of 16 or 32
// fill the last few segments that rounding up to 64 leaves without work, but give every share a
// partly filled trip: measured 0.5-1 % slower on the decode and verify shapes.)
__device__ __forceinline__ int segment_length(int total, int n_seg, int min_seg) {
  const int even = ((total + n_seg - 1) / n_seg + 63) / 64 * 64;
  return max(even, min_seg);
}

// Wave-cooperative: length of the stream, and the request that holds stream position
// `seg * seg_len` (its keys or the empty positions behind them) together with the stream position
// of that request's first key.
// Returns false when the segment starts beyond the stream.  All lanes must call.
__device__ __forceinline__ bool locate_segment(const SplitKvParams& p, int seg, int* seg_len,
                                               int* total_out, int* req, int* req_vstart) {
  const int lane = lane_id();
  int total = 0, n = 0, incl = 0;
  for (int b0 = 0; b0 < p.batch; b0 += kWave) {
    const int b = b0 + lane;
    n = 0;
    if (b < p.batch) {
      const ReqInfo r = request_info(p, b);
      n = stream_length(p, r.hi - r.lo);
    }
    incl = wave_inclusive_scan(n);
    total += __shfl(incl, kWave - 1, kWave);
  }
  total = max(total - p.boundary, 0);  // nothing follows the last request: its empty positions go
  const int len = segment_length(total, p.n_seg, p.min_seg);
  *seg_len = len;
  *total_out = total;
  const int pos = seg * len;
  if (pos >= total) return false;
  int base = 0;
  for (int b0 = 0; b0 < p.batch; b0 += kWave) {
    if (p.batch > kWave) {  // more than one batch of requests: recompute this batch
      const int b = b0 + lane;
      n = 0;
      if (b < p.batch) {
        const ReqInfo r = request_info(p, b);
        n = stream_length(p, r.hi - r.lo);
      }
      incl = wave_inclusive_scan(n);
    }
    const int batch_total = __shfl(incl, kWave - 1, kWave);
    if (pos < base + batch_total) {
      const int first = base + incl - n;
      const bool hit = (pos >= first) && (pos < first + n);
      const int src = __ffsll((long long)__ballot(hit)) - 1;
      *req = b0 + src;
      *req_vstart = __shfl(first, src, kWave);
      return true;
    }
    base += batch_total;
  }
  return false;
}

template <int D>
struct KvTile {
  u32x4_t k[2][D / 32];   // [16-token sub-tile][32-wide slice of D]: MFMA A operand of S^T
  u32x4_t v[D / 128][8];  // [128-wide half of D][token j of the lane group]: raw V segments
};

// NCT = tiles of 16 columns per wave, NW = waves per workgroup (launch bound only).  One
// column tile at head dim 128 fits 256 VGPRs, so two such waves per SIMD can be resident.
// WIDE: pool byte offsets need 64 bits (a pool of 4 GiB or more); otherwise a row's offset is
// one 32-bit multiply instead of a 64-bit multiply-add per load.
template <int D, int NCT, int NW, bool WIDE, bool F16>
__global__ __launch_bounds__(64 * NW, ((D == 128 && NCT == 1) ? 2 : 1)) void splitkv_attention_kernel(SplitKvParams p) {
  constexpr int KS = D / 32;   // k-steps of the QK product
  constexpr int VH = D / 128;  // 128-wide halves of D in the PV product
  const ClockProbe clock_probe_(p.clock_probe);
  const int lane = lane_id();
  const int t16 = lane & 15;
  const int g = lane >> 4;

  const int seg = blockIdx.x / p.head_groups;
  const int wave = threadIdx.x >> 6;
  const int cw = wave / p.nwh;  // which share of the columns this wave owns
  const int ct0 = cw * NCT;     // first of its tiles of 16 columns
  const int kvh = (blockIdx.x - seg * p.head_groups) * p.nwh + (wave - cw * p.nwh);
  int seg_len, total, cur_b, vs;
  if (!locate_segment(p, seg, &seg_len, &total, &cur_b, &vs)) return;
  cur_b = __builtin_amdgcn_readfirstlane(cur_b);
  vs = __builtin_amdgcn_readfirstlane(vs);
  int vpos = seg * seg_len;
  const int seg_end = min(vpos + seg_len, total);

  const unsigned char* kbase =
      reinterpret_cast<const unsigned char*>(p.k_cache + (int64_t)kvh * D + g * 8);
  const unsigned char* vbase =
      reinterpret_cast<const unsigned char*>(p.v_cache + (int64_t)kvh * D + t16 * 8);
  const uint32_t k_row_bytes = (uint32_t)p.k_stride0 * 2u;
  const uint32_t v_row_bytes = (uint32_t)p.v_stride0 * 2u;
  auto row_offset = [](int slot_id, uint32_t row_bytes) -> uint64_t {
    if constexpr (WIDE) return (uint64_t)(uint32_t)slot_id * row_bytes;
    else return (uint64_t)((uint32_t)slot_id * row_bytes);
  };

  while (vpos < seg_end && cur_b < p.batch) {
    const ReqInfo r = request_info(p, cur_b);
    const int vlen = r.hi - r.lo;
    if (vpos >= vs + vlen) {  // no keys, or past them in the empty positions: on to the next request
      vs += stream_length(p, vlen);
      vpos = max(vpos, vs);
      ++cur_b;
      continue;
    }
    const int t_begin = r.lo + (vpos - vs);
    const int t_end = min(r.hi, t_begin + (seg_end - vpos));
    const bool whole = (t_begin == r.lo) && (t_end == r.hi);
    if (t_begin == r.lo && kvh == 0 && ct0 == 0 && lane == 0) {
      // the wave that starts a request tells the merge kernel where its partials are
      const int s_first = vs / seg_len;
      p.req_items[2 * cur_b] = s_first;
      p.req_items[2 * cur_b + 1] = (vs + vlen - 1) / seg_len - s_first + 1;
    }
    const int ncols = r.q_len * p.group;

    // ---- Q operand and per-column visibility bounds --------------------------------
    u32x4_t qreg[NCT][KS];
    int col_lo[NCT], col_hi[NCT];
    int all_lo = 0, all_hi = 0x7fffffff;  // tile is mask-free iff inside [all_lo, all_hi]
#pragma unroll
    for (int ct = 0; ct < NCT; ++ct) {
      const int col = (ct0 + ct) * 16 + t16;
      const bool valid = col < ncols;
      const int qi = valid ? col / p.group : 0;
      const int hh = valid ? col - qi * p.group : 0;
      const uint16_t* qrow =
          p.q + ((int64_t)(r.q_start + qi) * p.n_q + kvh * p.group + hh) * D + g * 8;
#pragma unroll
      for (int c = 0; c < KS; ++c) {
        u32x4_t raw = {0u, 0u, 0u, 0u};
        if (valid) raw = ld_global_b128(qrow + c * 32);
        qreg[ct][c] = raw;
      }
      const int qpos = r.prefix + qi;
      int lo = (p.window > 0) ? qpos - p.window + 1 : 0;
      int hi = p.is_cross ? r.kv_len - 1 : min(qpos, r.kv_len - 1);
      hi = min(hi, t_end - 1);
      if (valid) {
        all_lo = max(all_lo, lo);
        all_hi = min(all_hi, hi);
      } else {
        lo = 1;
        hi = 0;
      }
      col_lo[ct] = lo;
      col_hi[ct] = hi;
    }
#pragma unroll
    for (int off = 1; off < 16; off <<= 1) {
      all_lo = max(all_lo, __shfl_xor(all_lo, off, kWave));
      all_hi = min(all_hi, __shfl_xor(all_hi, off, kWave));
    }
    all_lo = __builtin_amdgcn_readfirstlane(all_lo);
    all_hi = __builtin_amdgcn_readfirstlane(all_hi);

    // ---- accumulators ----------------------------------------------------------------
    f32x4_t oacc[NCT][VH][8];
    float m_run[NCT], l_run[NCT];
#pragma unroll
    for (int ct = 0; ct < NCT; ++ct) {
      m_run[ct] = kNegInf;
      l_run[ct] = 0.f;
#pragma unroll
      for (int hf = 0; hf < VH; ++hf)
#pragma unroll
        for (int n = 0; n < 8; ++n) oacc[ct][hf][n] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    }

    const int32_t* idx_base = p.kv_indices + r.kv_start;
    const int last_tok = t_end - 1;

    // slot ids of the two K rows this lane loads in a 32-token tile starting at tb
    auto load_idx = [&](int tb, int& s0, int& s1) {
      s0 = (int)min((uint32_t)idx_base[min(tb + t16, last_tok)], p.max_slot);
      s1 = (int)min((uint32_t)idx_base[min(tb + 16 + t16, last_tok)], p.max_slot);
    };
    auto load_tile = [&](KvTile<D>& t, int s0, int s1) {
#pragma unroll
      for (int c = 0; c < KS; ++c) {
        t.k[0][c] = ld_global_b128(kbase + row_offset(s0, k_row_bytes) + c * 64);
        t.k[1][c] = ld_global_b128(kbase + row_offset(s1, k_row_bytes) + c * 64);
      }
      // V rows of this lane group: tokens 4g+j (j<4) of sub-tile 0, then of sub-tile 1;
      // their slot ids sit in lanes 4g+j of the K index registers.
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int src = 4 * g + (j & 3);
        const int slot = __shfl(j < 4 ? s0 : s1, src, kWave);
        const unsigned char* vrow = vbase + row_offset(slot, v_row_bytes);
#pragma unroll
        for (int hf = 0; hf < VH; ++hf) t.v[hf][j] = ld_global_b128(vrow + hf * 256);
      }
    };

    auto compute_tile = [&](const KvTile<D>& t, int tb) {
      // S^T[token][col] for the two 16-token sub-tiles
      f32x4_t s[2][NCT];
#pragma unroll
      for (int sub = 0; sub < 2; ++sub)
#pragma unroll
        for (int ct = 0; ct < NCT; ++ct) {
          f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int c = 0; c < KS; ++c)
            acc = mfma_16x16x32_raw<F16>(t.k[sub][c], qreg[ct][c], acc);
          s[sub][ct] = acc;
        }
      const bool need_mask = (tb < all_lo) || (tb + 31 > all_hi);
      uint32_t pb[NCT][4];
#pragma unroll
      for (int ct = 0; ct < NCT; ++ct) {
        float x[2][4];
#pragma unroll
        for (int sub = 0; sub < 2; ++sub)
#pragma unroll
          for (int i = 0; i < 4; ++i) x[sub][i] = s[sub][ct][i] * p.scale_log2e;
        if (need_mask) {
#pragma unroll
          for (int sub = 0; sub < 2; ++sub)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              const int tok = tb + sub * 16 + 4 * g + i;
              if (tok < col_lo[ct] || tok > col_hi[ct]) x[sub][i] = kNegInf;
            }
        }
        float mx = fmaxf(fmaxf(fmaxf(x[0][0], x[0][1]), fmaxf(x[0][2], x[0][3])),
                         fmaxf(fmaxf(x[1][0], x[1][1]), fmaxf(x[1][2], x[1][3])));
        mx = wave_max_xor(mx, 16);
        mx = wave_max_xor(mx, 32);
        const float m_new = fmaxf(m_run[ct], mx);
        const float m_safe = (m_new == kNegInf) ? 0.f : m_new;
        const float alpha = fast_exp2(m_run[ct] - m_safe);
        m_run[ct] = m_new;
        float psum = 0.f;
#pragma unroll
        for (int sub = 0; sub < 2; ++sub)
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            x[sub][i] = fast_exp2(x[sub][i] - m_safe);
            psum += x[sub][i];
          }
        l_run[ct] = l_run[ct] * alpha + psum;
        pb[ct][0] = pack_16x2<F16>(x[0][0], x[0][1]);
        pb[ct][1] = pack_16x2<F16>(x[0][2], x[0][3]);
        pb[ct][2] = pack_16x2<F16>(x[1][0], x[1][1]);
        pb[ct][3] = pack_16x2<F16>(x[1][2], x[1][3]);
        if (__any(alpha != 1.0f)) {
#pragma unroll
          for (int hf = 0; hf < VH; ++hf)
#pragma unroll
            for (int n = 0; n < 8; ++n) oacc[ct][hf][n] *= alpha;
        }
      }
      // O^T += V^T P^T.  MFMA n of half hf produces d = hf*128 + 8*row + n on row = l%16.
#pragma unroll
      for (int hf = 0; hf < VH; ++hf)
#pragma unroll
        for (int n = 0; n < 8; ++n) {
          u32x4_t vt;
#pragma unroll
          for (int qd = 0; qd < 4; ++qd) {
            const uint32_t a = t.v[hf][2 * qd][n >> 1];
            const uint32_t c = t.v[hf][2 * qd + 1][n >> 1];
            vt[qd] = (n & 1) ? pack_hi16(a, c) : pack_lo16(a, c);
          }
#pragma unroll
          for (int ct = 0; ct < NCT; ++ct) {
            const u32x4_t pv = {pb[ct][0], pb[ct][1], pb[ct][2], pb[ct][3]};
            oacc[ct][hf][n] = mfma_16x16x32_raw<F16>(vt, pv, oacc[ct][hf][n]);
          }
        }
    };

    // ---- tile loop: two register tiles, slot ids fetched two tiles ahead.  Every load in
    // the loop body is unconditional (tokens past the range clamp to its last token and
    // are masked), so the number of loads in flight at each wait is a compile-time
    // constant and the next tile stays in flight while the current one is computed. ----
    const int n_pairs = (t_end - t_begin + 63) / 64;
    KvTile<D> ta, tb_;
    int i0a, i0b, i1a, i1b;
    load_idx(t_begin, i0a, i0b);
    load_idx(t_begin + 32, i1a, i1b);
    load_tile(ta, i0a, i0b);
    load_idx(t_begin + 64, i0a, i0b);
    for (int pr = 0; pr < n_pairs; ++pr) {
      const int tok = t_begin + pr * 64;
      load_tile(tb_, i1a, i1b);
      load_idx(tok + 96, i1a, i1b);
      compute_tile(ta, tok);
      load_tile(ta, i0a, i0b);
      load_idx(tok + 128, i0a, i0b);
      compute_tile(tb_, tok + 32);
    }

    // ---- this request's share is done: write output or partial -------------------------
#pragma unroll
    for (int ct = 0; ct < NCT; ++ct) {
      float l = l_run[ct];
      l += __shfl_xor(l, 16, kWave);
      l += __shfl_xor(l, 32, kWave);
      const float inv = (l > 0.f) ? 1.0f / l : 0.f;
      const int col = (ct0 + ct) * 16 + t16;
      if (col >= ncols) continue;
      const int qi = col / p.group;
      const int hh = col - qi * p.group;
      if (whole) {
        uint16_t* orow = p.out + ((int64_t)(r.q_start + qi) * p.n_q + kvh * p.group + hh) * D;
#pragma unroll
        for (int hf = 0; hf < VH; ++hf)
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            u32x4_t w;
#pragma unroll
            for (int n = 0; n < 4; ++n)
              w[n] = pack_16x2<F16>(oacc[ct][hf][2 * n][i] * inv, oacc[ct][hf][2 * n + 1][i] * inv);
            st_global_b128(orow + hf * 128 + (4 * g + i) * 8, w);
          }
      } else {
        const int64_t block = (int64_t)(seg + cur_b) * p.n_kv + kvh;
        if constexpr (F16) {
#pragma unroll
          for (int hf = 0; hf < VH; ++hf)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              f32x4_t w0, w1;
#pragma unroll
              for (int n = 0; n < 4; ++n) {
                w0[n] = oacc[ct][hf][n][i] * inv;
                w1[n] = oacc[ct][hf][4 + n][i] * inv;
              }
              float* dst = p.part_o + partial_offset(block, p.cols, col, hf * 128 + (4 * g + i) * 8, D);
              *reinterpret_cast<f32x4_t*>(dst) = w0;
              *reinterpret_cast<f32x4_t*>(dst + 4) = w1;
            }
        } else {
#pragma unroll
          for (int hf = 0; hf < VH; ++hf)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              u32x4_t w;
#pragma unroll
              for (int n = 0; n < 4; ++n)
                w[n] = pack_half2_clamped(oacc[ct][hf][2 * n][i] * inv, oacc[ct][hf][2 * n + 1][i] * inv);
              _Float16* dst = reinterpret_cast<_Float16*>(p.part_o) +
                              partial_offset(block, p.cols, col, hf * 128 + (4 * g + i) * 8, D);
              *reinterpret_cast<u32x4_t*>(dst) = w;
            }
        }
        if (g == 0) p.part_lse[block * p.cols + col] = (l > 0.f) ? m_run[ct] + __log2f(l) : kNegInf;
      }
    }

    vpos += t_end - t_begin;  // the request's end, or the segment's: the loop head sorts it out
  }
}

// One workgroup of NW waves per (request, query, q head): merge the partials of the segments
// that share the request, by base-2 LSE.  Requests without visible keys get zeros; requests
// that sat inside one segment were written by the attention kernel itself.
// Up to kMergeSmall items (a request cut a few times: the usual case) one wave reads whole rows
// and nothing crosses lanes.  Beyond that a partial row is taken as D / 8 chunks of 8 floats,
// one chunk per lane, so a wave holds 64 / (D / 8) rows side by side and a workgroup
// NG = NW * that many; each of these lane groups takes every NG-th item, one in the first trip
// and kMergeUnroll per trip after it, with all their loads in flight together.  A request cut
// into a hundred segments (one long request alone on the chip) thus needs three or four memory
// round trips where a loop over its items needs a hundred.
constexpr int kMergeUnroll = 3;
constexpr int kMergeSmall = 8;
template <int D, bool F16, int NW>
__global__ __launch_bounds__(64 * NW) void splitkv_merge_kernel(SplitKvParams p) {
  constexpr int LPI = D / 8;          // lanes per item
  constexpr int GPW = kWave / LPI;    // items side by side in a wave
  constexpr int NG = GPW * NW;        // ... and in the workgroup
  constexpr int U = kMergeUnroll;
  const int b = blockIdx.x / p.max_len_extend;
  const int qi = blockIdx.x - b * p.max_len_extend;
  const int hq = blockIdx.y;
  const int lane = lane_id();
  const int wave = threadIdx.x >> 6;
  const int grp = wave * GPW + lane / LPI;
  const int dl = lane % LPI;  // this lane's chunk: dims dl * 8 .. dl * 8 + 7
  // every exit below, and the choice between the two ways, is the same for the whole workgroup
  const int s_first = p.req_items[2 * b];
  const int n_items = p.req_items[2 * b + 1];
  const ReqInfo r = request_info(p, b);
  if (qi >= r.q_len) return;
  uint16_t* orow = p.out + ((int64_t)(r.q_start + qi) * p.n_q + hq) * D + dl * 8;
  if (r.hi - r.lo == 0) {  // no visible key: nobody wrote req_items, the row is zero
    if (threadIdx.x < LPI) st_global_b128(orow, u32x4_t{0u, 0u, 0u, 0u});
    return;
  }
  if (n_items == 1) return;  // written by the attention kernel itself
  const int kvh = hq / p.group;
  const int col = qi * p.group + (hq - kvh * p.group);
  const int64_t stride = (int64_t)p.n_kv * p.cols;                               // rows per item
  const int64_t row0 = ((int64_t)(s_first + b) * p.n_kv + kvh) * p.cols + col;  // LSE of item 0
  const int64_t block0 = (int64_t)(s_first + b) * p.n_kv + kvh;                 // partial of item 0

  if (n_items <= kMergeSmall) {
    // one wave, a whole row per load, every lane reads the few LSEs itself: one memory round
    // trip after the geometry's
    if (wave > 0) return;
    constexpr int PER = D / kWave;  // consecutive floats per lane
    float ls[kMergeSmall], v[kMergeSmall][PER];
#pragma unroll
    for (int u = 0; u < kMergeSmall; ++u) {
      ls[u] = kNegInf;
#pragma unroll
      for (int e = 0; e < PER; ++e) v[u][e] = 0.f;
      if (u < n_items) {
        ls[u] = p.part_lse[row0 + u * stride];
        const int64_t at = partial_offset(block0 + (int64_t)u * p.n_kv, p.cols, col, lane * PER, D);
        if constexpr (F16) {
          const float* src = p.part_o + at;
#pragma unroll
          for (int e = 0; e < PER; ++e) v[u][e] = src[e];
        } else {
          const _Float16* src = reinterpret_cast<const _Float16*>(p.part_o) + at;
#pragma unroll
          for (int e = 0; e < PER; ++e) v[u][e] = (float)src[e];
        }
      }
    }
    float mx = ls[0];
#pragma unroll
    for (int u = 1; u < kMergeSmall; ++u) mx = fmaxf(mx, ls[u]);
    float acc[PER];
#pragma unroll
    for (int e = 0; e < PER; ++e) acc[e] = 0.f;
    float wsum = 0.f;
    if (mx > kNegInf) {
#pragma unroll
      for (int u = 0; u < kMergeSmall; ++u) {
        const float wu = fast_exp2(ls[u] - mx);  // 0 for an item that is not there
#pragma unroll
        for (int e = 0; e < PER; ++e) acc[e] += wu * v[u][e];
        wsum += wu;
      }
    }
    const float inv = (wsum > 0.f) ? 1.0f / wsum : 0.f;
    uint16_t* dst = p.out + ((int64_t)(r.q_start + qi) * p.n_q + hq) * D + lane * PER;
#pragma unroll
    for (int e = 0; e < PER; e += 2)
      *reinterpret_cast<uint32_t*>(dst + e) = pack_16x2<F16>(acc[e] * inv, acc[e + 1] * inv);
    return;
  }

  float acc[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) acc[e] = 0.f;
  float wsum = 0.f;
  float lse[U];
  f32x4_t va[U][2];
  // items base, base + NG, ... (`n` of them); lanes past the last item load nothing and
  // contribute weight 0 to a row of zeros
  auto fetch = [&](int base, auto n) {
#pragma unroll
    for (int u = 0; u < decltype(n)::value; ++u) {
      const int it = base + u * NG;
      lse[u] = kNegInf;
      va[u][0] = va[u][1] = f32x4_t{0.f, 0.f, 0.f, 0.f};
      if (it < n_items) {
        lse[u] = p.part_lse[row0 + it * stride];
        const int64_t at = partial_offset(block0 + (int64_t)it * p.n_kv, p.cols, col, dl * 8, D);
        if constexpr (F16) {
          const float* src = p.part_o + at;
          va[u][0] = *reinterpret_cast<const f32x4_t*>(src);
          va[u][1] = *reinterpret_cast<const f32x4_t*>(src + 4);
        } else {
          const f16x8s_t hv = *reinterpret_cast<const f16x8s_t*>(reinterpret_cast<const _Float16*>(p.part_o) + at);
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            va[u][0][e] = (float)hv[e];
            va[u][1][e] = (float)hv[4 + e];
          }
        }
      }
    }
  };
  auto consume = [&](float mx, auto n) {
#pragma unroll
    for (int u = 0; u < decltype(n)::value; ++u) {
      const float wu = fast_exp2(lse[u] - mx);  // 0 for an item that is not there
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        acc[e] += wu * va[u][0][e];
        acc[4 + e] += wu * va[u][1][e];
      }
      wsum += wu;
    }
  };
  using One = std::integral_constant<int, 1>;
  using Trip = std::integral_constant<int, U>;
  // Two memory round trips for up to NG items: geometry and place of the partials above, then
  // every LSE (for the maximum) and one row per lane group together.  The rest in trips of
  // NG * U items.
  fetch(grp, One{});
  float mx = kNegInf;
  for (int it = lane; it < n_items; it += kWave) mx = fmaxf(mx, p.part_lse[row0 + it * stride]);
#pragma unroll
  for (int off = 1; off < kWave; off <<= 1) mx = fmaxf(mx, __shfl_xor(mx, off, kWave));
  if (mx > kNegInf) {
    consume(mx, One{});
    for (int base = grp + NG; base < n_items; base += NG * U) {
      fetch(base, Trip{});
      consume(mx, Trip{});
    }
  }
  // fold the lane groups of a wave, then the waves
#pragma unroll
  for (int off = LPI; off < kWave; off <<= 1) {
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] += __shfl_xor(acc[e], off, kWave);
    wsum += __shfl_xor(wsum, off, kWave);
  }
  if constexpr (NW > 1) {
    __shared__ float fold[NW - 1][LPI][9];
    if (wave > 0 && lane < LPI) {
#pragma unroll
      for (int e = 0; e < 8; ++e) fold[wave - 1][lane][e] = acc[e];
      fold[wave - 1][lane][8] = wsum;
    }
    __syncthreads();
    if (wave > 0) return;
    if (lane < LPI) {
#pragma unroll
      for (int w = 0; w < NW - 1; ++w) {
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[e] += fold[w][lane][e];
        wsum += fold[w][lane][8];
      }
    }
  }
  if (lane >= LPI) return;
  const float inv = (wsum > 0.f) ? 1.0f / wsum : 0.f;
  u32x4_t w;
#pragma unroll
  for (int e = 0; e < 4; ++e) w[e] = pack_16x2<F16>(acc[2 * e] * inv, acc[2 * e + 1] * inv);
  st_global_b128(orow, w);
}

int nct_for(int64_t cols) { return (int)((cols + 15) / 16); }

thread_local int t_max_waves = 4;  // benchmarking switch, one value per host thread
int heads_per_group(int64_t n_kv) {
  const int cap = t_max_waves;
  if (cap >= 8 && n_kv % 8 == 0) return 8;
  if (cap >= 4 && n_kv % 4 == 0) return 4;
  return (cap >= 2 && n_kv % 2 == 0) ? 2 : 1;
}

int device_cus() {
  static std::atomic<int> cache{0};
  int v = cache.load();
  if (v > 0) return v;
  int dev = 0, cus = 0;
  if (hipGetDevice(&dev) != hipSuccess ||
      hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess ||
      cus <= 0) {
    (void)hipGetLastError();
    return 256;  // MI355X
  }
  cache.store(cus);
  return cus;
}

template <int D, int NCT, int NW>
void launch_attn(const SplitKvParams& p, hipStream_t stream) {
  const dim3 grid((unsigned)(p.n_seg * p.head_groups)), block(64 * NW);
  if constexpr (NCT == 1) {  // IEEE half exists for decode only (one column tile)
    if (p.f16) {
      if (p.wide) hipLaunchKernelGGL((splitkv_attention_kernel<D, NCT, NW, true, true>), grid, block, 0, stream, p);
      else hipLaunchKernelGGL((splitkv_attention_kernel<D, NCT, NW, false, true>), grid, block, 0, stream, p);
      return;
    }
  }
  if (p.wide) hipLaunchKernelGGL((splitkv_attention_kernel<D, NCT, NW, true, false>), grid, block, 0, stream, p);
  else hipLaunchKernelGGL((splitkv_attention_kernel<D, NCT, NW, false, false>), grid, block, 0, stream, p);
}

template <int D, int NCT>
int launch_dn(const SplitKvParams& p, int waves, hipStream_t stream) {
  if (p.f16 && NCT != 1) return MSGL_ERR_DTYPE;
  switch (waves) {
    case 1: launch_attn<D, NCT, 1>(p, stream); break;
    case 2: launch_attn<D, NCT, 2>(p, stream); break;
    case 4: launch_attn<D, NCT, 4>(p, stream); break;
    case 8:
      if constexpr (D == 128 && NCT == 1) launch_attn<D, NCT, 8>(p, stream);
      else return MSGL_ERR_SHAPE;
      break;
    default: return MSGL_ERR_SHAPE;
  }
  int rc = check_launch();
  if (rc != MSGL_OK) return rc;
  const dim3 mgrid((unsigned)(p.batch * p.max_len_extend), (unsigned)p.n_q);
  // four waves per row when a request can be cut into more items than one wave takes in a trip
  // and the rows are few enough that the extra waves cost nothing
  constexpr int kItemsPerTrip = kWave / (D / 8) * (1 + kMergeUnroll);
  const bool wide_merge = p.n_seg > kItemsPerTrip && (int64_t)mgrid.x * mgrid.y <= 1024;
  if (wide_merge) {
    if (p.f16) hipLaunchKernelGGL((splitkv_merge_kernel<D, true, 4>), mgrid, dim3(256), 0, stream, p);
    else hipLaunchKernelGGL((splitkv_merge_kernel<D, false, 4>), mgrid, dim3(256), 0, stream, p);
  } else {
    if (p.f16) hipLaunchKernelGGL((splitkv_merge_kernel<D, true, 1>), mgrid, dim3(64), 0, stream, p);
    else hipLaunchKernelGGL((splitkv_merge_kernel<D, false, 1>), mgrid, dim3(64), 0, stream, p);
  }
  return check_launch();
}

// How a shape's column tiles map onto waves: tiles per wave and waves per kv head.
struct ColSplit { int nct_wave; int col_waves; };
ColSplit col_split(int nct, int64_t head_dim) {
  // head dim 256: one tile per wave (two would spill); three tiles take four waves, the last
  // of which finds no valid column (workgroups come in 1, 2, 4 or 8 waves)
  if (head_dim != 128) return ColSplit{1, nct == 3 ? 4 : nct};
  // head dim 128: up to three tiles in one wave (487 VGPRs; 33-48 columns run 22-26 % faster
  // than on two waves per kv head, which read every K / V row twice); four tiles spill, and with
  // the Q operand parked in LDS to avoid that they are no faster than two waves of two
  return nct <= 3 ? ColSplit{nct, 1} : ColSplit{2, 2};
}

template <int D>
int launch_d(const SplitKvParams& p, int nct, hipStream_t stream) {
  const ColSplit cs = col_split(nct, D);
  const int waves = p.nwh * cs.col_waves;
  if (cs.nct_wave == 1) return launch_dn<D, 1>(p, waves, stream);
  if constexpr (D == 128) {
    if (cs.nct_wave == 2) return launch_dn<D, 2>(p, waves, stream);
    if (cs.nct_wave == 3) return launch_dn<D, 3>(p, waves, stream);
  }
  return MSGL_ERR_SHAPE;
}

}  // namespace

// ---- built-in scratch for callers that cannot allocate --------------------------------------
// One array per GPU, part of the loaded code object, held until the process ends.  In host code
// the array's name is only a handle for hipGetSymbolAddress: the address that kernels and copies
// use is looked up once per device, with that device current, and kept.
constexpr size_t kScratchBytes = (size_t)MSGL_DECODE_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kScratchBytes];

int splitkv_scratch(void** ptr, size_t* bytes) {
  constexpr int kMaxDevices = 64;
  static std::atomic<void*> addr[kMaxDevices];
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
    (void)hipGetLastError();
    return MSGL_ERR_LAUNCH;
  }
  void* p = addr[dev].load(std::memory_order_acquire);
  if (p == nullptr) {
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || p == nullptr) {
      (void)hipGetLastError();
      return MSGL_ERR_LAUNCH;
    }
    addr[dev].store(p, std::memory_order_release);  // every thread resolves the same address
  }
  *ptr = p;
  *bytes = kScratchBytes;
  return MSGL_OK;
}

void splitkv_set_max_waves(int v) { t_max_waves = v > 0 ? v : 4; }  // 0 restores the default

// benchmarking switch, one value per host thread: stream positions charged per request boundary
// (0: chosen from the shape, below; negative: none)
static thread_local int t_boundary = 0;
void splitkv_set_boundary(int v) { t_boundary = v; }
// A boundary costs a workgroup about 8 us (measured on the benchmark shapes, one and eight
// queries per request); in that time it would stream 8 us x (what the chip reads per us) /
// (workgroups x bytes of one token's K and V rows for the workgroup's kv heads) tokens.
// A workgroup with the chip to itself streams about 40 GB/s (its own chain of loads, not the
// memory system, is the limit), so a small launch charges what one workgroup reads in that time.
static int boundary_tokens(int64_t n_wgs, int nwh, int64_t head_dim) {
  if (t_boundary != 0) return t_boundary > 0 ? (t_boundary < 4096 ? t_boundary : 4096) : 0;
  const double bytes_per_token = (double)nwh * 2.0 * (double)head_dim * 2.0;
  const double wg_bytes_per_us = std::min(6.2e6 / (double)(n_wgs > 0 ? n_wgs : 1), 40e3);
  const double tokens = 8.0 * wg_bytes_per_us / bytes_per_token;
  const int64_t t = ((int64_t)tokens + 8) / 16 * 16;
  return (int)(t < 0 ? 0 : (t > 1024 ? 1024 : t));
}

// kv heads per workgroup for this shape: up to 4, halved when a second wave per head is
// needed for the columns (a workgroup of the wide variants holds at most 4 waves: they
// need more than 256 VGPRs, one wave per SIMD)
static int nwh_for(int64_t n_kv, int nct, int64_t head_dim) {
  int nwh = heads_per_group(n_kv);
  const int col_waves = col_split(nct, head_dim).col_waves;
  const int max_waves = (nct == 1 && head_dim == 128) ? 8 : 4;
  while (nwh * col_waves > max_waves && nwh > 1) nwh /= 2;
  return nwh;
}

int splitkv_default_segments(int64_t total_kv, int64_t n_kv, int64_t head_dim, int64_t cols,
                             int32_t min_seg) {
  const int nct = nct_for(cols);
  const int nwh = nwh_for(n_kv, nct, head_dim);
  const int waves = nwh * col_split(nct, head_dim).col_waves;
  const int64_t head_groups = n_kv / nwh;
  // Workgroups for 13 of every 16 CUs, at most one per CU (small workgroups are doubled up until
  // a CU holds four waves): the memory system is saturated well before every CU streams, and
  // fewer, longer segments mean fewer partials and fewer request boundaries inside a segment.
  // Measured at 256 CUs, segments per head group 80 .. 128: fastest at 96 .. 112 on every
  // benchmark shape (1-2 % under 128), slower again below 88.
  const int64_t blocks = (int64_t)device_cus() * 13 / 16 * (waves >= 4 ? 1 : 4 / waves);
  int64_t n_seg = blocks / head_groups;
  const int64_t by_len = (total_kv + min_seg - 1) / min_seg;
  if (n_seg > by_len) n_seg = by_len;
  if (n_seg < 1) n_seg = 1;
  return (int)n_seg;
}

size_t splitkv_workspace_bytes(int64_t batch, int64_t n_q, int64_t n_kv, int64_t head_dim,
                               int64_t max_len_extend, int32_t n_seg) {
  const int64_t cols = n_q / n_kv * max_len_extend;
  const int64_t rows = ((int64_t)n_seg + batch) * n_kv * cols;
  size_t bytes = (size_t)rows * (size_t)head_dim * sizeof(float);  // part_o
  bytes += (size_t)rows * sizeof(float);                           // part_lse
  bytes += (size_t)(2 * batch + 4) * sizeof(int32_t);              // req_items
  return (bytes + 255) / 256 * 256 + 256;
}

int launch_splitkv(const SplitKvArgs& a, hipStream_t stream) {
  const int64_t group = a.n_q / a.n_kv;
  const int64_t cols = group * a.max_len_extend;
  if (cols < 1 || cols > kSplitKvMaxCols || a.n_seg < 1 || a.min_seg < 64 || a.min_seg % 64 != 0)
    return MSGL_ERR_SHAPE;
  if (a.batch * a.max_len_extend > 0x7fffffffLL || a.total_kv > 0x7fffffffLL) return MSGL_ERR_SHAPE;
  if (a.batch == 0) return MSGL_OK;
  const int nct = nct_for(cols);
  const int nwh = nwh_for(a.n_kv, nct, a.head_dim);

  SplitKvParams p;
  p.q = static_cast<const uint16_t*>(a.q);
  p.k_cache = static_cast<const uint16_t*>(a.k_cache);
  p.v_cache = static_cast<const uint16_t*>(a.v_cache);
  p.kv_indptr = a.kv_indptr;
  p.kv_indices = a.kv_indices;
  p.qo_indptr = a.qo_indptr;
  p.prefix_lens = a.prefix_lens;
  p.out = static_cast<uint16_t*>(a.out);
  p.cols = (int32_t)cols;
  const int64_t rows = ((int64_t)a.n_seg + a.batch) * a.n_kv * cols;
  char* ws = static_cast<char*>(a.workspace);
  p.part_o = reinterpret_cast<float*>(ws);
  p.part_lse = reinterpret_cast<float*>(ws + (size_t)rows * a.head_dim * sizeof(float));
  p.req_items = reinterpret_cast<int32_t*>(ws + (size_t)rows * (a.head_dim + 1) * sizeof(float));
  p.k_stride0 = a.k_stride0;
  p.v_stride0 = a.v_stride0;
  p.batch = (int32_t)a.batch;
  p.n_q = (int32_t)a.n_q;
  p.n_kv = (int32_t)a.n_kv;
  p.group = (int32_t)group;
  p.max_slot = (uint32_t)(a.num_slots > 0 ? a.num_slots - 1 : 0);
  p.nwh = nwh;
  p.head_groups = (int32_t)(a.n_kv / nwh);
  p.n_seg = a.n_seg;
  p.boundary = boundary_tokens((int64_t)a.n_seg * (a.n_kv / nwh), nwh, a.head_dim);
  p.min_seg = a.min_seg;
  p.max_len_extend = a.max_len_extend;
  p.f16 = a.f16;
  p.q_begin = a.q_begin;
  p.q_cap = a.q_cap > 0 ? a.q_cap : a.max_len_extend;
  p.is_cross = a.is_cross;
  p.window = a.window;
  p.scale_log2e = a.sm_scale * kLog2e;
  p.clock_probe = clock_probe();
  p.wide = ((uint64_t)a.num_slots * (uint64_t)a.k_stride0 * 2u >= (1ull << 32) ||
            (uint64_t)a.num_slots * (uint64_t)a.v_stride0 * 2u >= (1ull << 32)) ? 1 : 0;
  if ((int64_t)p.n_seg * p.head_groups > 0x7fffffffLL) return MSGL_ERR_SHAPE;
  if (a.head_dim == 128) return launch_d<128>(p, nct, stream);
  if (a.head_dim == 256) return launch_d<256>(p, nct, stream);
  return MSGL_ERR_HEAD_DIM;
}

}  // namespace msgl
