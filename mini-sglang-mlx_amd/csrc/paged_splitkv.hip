// Bandwidth-bound paged attention for short query blocks on gfx950: single-token GQA
// decode (paged_decode_attention) and the q_len <= a-few-tokens route of
// paged_prefill_attention (speculative verify, draft proposal).
//
// Replaces paged_decode_attention_stage1 / _stage2
// (mini-sglang-mlx-kernel/csrc/paged_decode_attention.metal:313-586) and, for short
// extends, paged_prefill_attention (paged_prefill_attention.metal:382-640).
//
// Shape of the computation
//   work item  = (request, kv head, chunk of `chunk` consecutive visible tokens), one wave64.
//   columns    = the q rows that share this kv head: col = q_idx * group + head_in_group,
//                padded to NCT tiles of 16 (the MFMA N dimension).  Every K / V row is
//                therefore read once per kv head, whatever the group size or q_len.
//   S^T        = K_tile (16 tokens x D) * Q^T        -> mfma 16x16x32, tokens on M
//   O^T       += V_tile^T (D x 32 tokens) * P^T      -> mfma 16x16x32, tokens on K
//   Both products keep "column" on l%16 of the accumulator, so the softmax state, the
//   P operand and the O rescale stay lane-local; the only cross-lane traffic per tile is
//   the column max (two xor-shuffles).
//   V rows are loaded as whole 16-byte segments (16 lanes cover one 256-byte row) and
//   turned into the token-contiguous MFMA operand by an in-lane 8x8 transpose of 16-bit
//   values (v_perm_b32); the token order inside an MFMA is chosen so that it matches the
//   accumulator layout of S^T, which is legal because the contraction is a sum.
//   Item -> (request, chunk) is recomputed by every wave from kv_indptr with a wave-wide
//   prefix sum: the host never reads device metadata, so the grid is the host-known upper
//   bound ceil(total_kv / chunk) + batch and surplus waves exit.
//   Requests that fit one chunk write bf16 output directly; others write a normalised fp32
//   partial + base-2 LSE, merged by splitkv_merge_kernel.
//
// Algorithmic HBM bytes per visible token and kv head: 2 * D * 2 (one K row + one V row)
// plus 4 bytes of kv_indices per token.
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
  float* part_o;           // [max_items][n_kv][cols_pad][D]
  float* part_lse;         // [max_items][n_kv][cols_pad]
  int32_t* req_item_base;  // [batch] first item of a request (written by its chunk 0)
  int64_t k_stride0, v_stride0;
  int32_t batch, n_q, n_kv, group;
  int32_t max_items, cols_pad, max_len_extend, chunk;
  int32_t is_cross, window;
  float scale_log2e;
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
    r.q_start = p.qo_indptr[b];
    r.q_len = min(p.qo_indptr[b + 1] - r.q_start, p.max_len_extend);
    r.prefix = p.prefix_lens[b];
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

__device__ __forceinline__ int32_t num_chunks(const ReqInfo& r, int chunk) {
  return (r.hi - r.lo + chunk - 1) / chunk;
}

// Wave-cooperative search: which request owns work item `item`?  Returns false when the
// item lies beyond the last request.  All lanes must call.
__device__ __forceinline__ bool locate_item(const SplitKvParams& p, int item, int* req,
                                            int* chunk_idx, int* item_base) {
  const int lane = lane_id();
  int base = 0;
  for (int b0 = 0; b0 < p.batch; b0 += kWave) {
    const int b = b0 + lane;
    int n = 0;
    if (b < p.batch) n = num_chunks(request_info(p, b), p.chunk);
    const int incl = wave_inclusive_scan(n);
    const int total = __shfl(incl, kWave - 1, kWave);
    if (item < base + total) {
      const int first = base + incl - n;
      const bool hit = (item >= first) && (item < first + n);
      const unsigned long long m = __ballot(hit);
      const int src = __ffsll((long long)m) - 1;
      *req = b0 + src;
      *item_base = __shfl(first, src, kWave);
      *chunk_idx = item - *item_base;
      return true;
    }
    base += total;
  }
  return false;
}

template <int D>
struct KvTile {
  u32x4_t k[2][D / 32];   // [16-token sub-tile][32-wide slice of D]: MFMA A operand of S^T
  u32x4_t v[D / 128][8];  // [128-wide half of D][token j of the lane group]: raw V segments
};

template <int D, int NCT>
__global__ __launch_bounds__(64) void splitkv_attention_kernel(SplitKvParams p) {
  constexpr int KS = D / 32;   // k-steps of the QK product
  constexpr int VH = D / 128;  // 128-wide halves of D in the PV product
  const int lane = lane_id();
  const int t16 = lane & 15;
  const int g = lane >> 4;

  const int item = blockIdx.x / p.n_kv;
  const int kvh = blockIdx.x - item * p.n_kv;
  int b, chunk_idx, item_base;
  if (!locate_item(p, item, &b, &chunk_idx, &item_base)) return;
  const ReqInfo r = request_info(p, b);
  const int n_items = num_chunks(r, p.chunk);
  if (chunk_idx == 0 && kvh == 0 && lane == 0) p.req_item_base[b] = item_base;

  const int t_begin = r.lo + chunk_idx * p.chunk;
  const int t_end = min(r.hi, t_begin + p.chunk);
  const int ncols = r.q_len * p.group;

  // ---- Q operand and per-column visibility bounds --------------------------------
  bf16x8_t qreg[NCT][KS];
  int col_lo[NCT], col_hi[NCT];
  int all_lo = 0, all_hi = 0x7fffffff;  // tile is mask-free iff inside [all_lo, all_hi]
#pragma unroll
  for (int ct = 0; ct < NCT; ++ct) {
    const int col = ct * 16 + t16;
    const bool valid = col < ncols;
    const int qi = valid ? col / p.group : 0;
    const int hh = valid ? col - qi * p.group : 0;
    const uint16_t* qrow =
        p.q + ((int64_t)(r.q_start + qi) * p.n_q + kvh * p.group + hh) * D + g * 8;
#pragma unroll
    for (int c = 0; c < KS; ++c) {
      u32x4_t raw = {0u, 0u, 0u, 0u};
      if (valid) raw = ld_global_b128(qrow + c * 32);
      qreg[ct][c] = as_bf16x8(raw);
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

  // ---- accumulators ------------------------------------------------------------------
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
  const uint16_t* kbase = p.k_cache + (int64_t)kvh * D + g * 8;
  const uint16_t* vbase = p.v_cache + (int64_t)kvh * D + t16 * 8;
  const int last_tok = t_end - 1;

  // slot ids of the two K rows this lane loads in a 32-token tile starting at tb
  auto load_idx = [&](int tb, int& s0, int& s1) {
    s0 = idx_base[min(tb + t16, last_tok)];
    s1 = idx_base[min(tb + 16 + t16, last_tok)];
  };
  auto load_tile = [&](KvTile<D>& t, int s0, int s1) {
#pragma unroll
    for (int c = 0; c < KS; ++c) {
      t.k[0][c] = ld_global_b128(kbase + (int64_t)s0 * p.k_stride0 + c * 32);
      t.k[1][c] = ld_global_b128(kbase + (int64_t)s1 * p.k_stride0 + c * 32);
    }
    // V rows of this lane group: tokens 4g+j (j<4) of sub-tile 0, then of sub-tile 1;
    // their slot ids sit in lanes 4g+j of the K index registers.
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int src = 4 * g + (j & 3);
      const int slot = __shfl(j < 4 ? s0 : s1, src, kWave);
      const uint16_t* vrow = vbase + (int64_t)slot * p.v_stride0;
#pragma unroll
      for (int hf = 0; hf < VH; ++hf) t.v[hf][j] = ld_global_b128(vrow + hf * 128);
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
          acc = mfma_16x16x32(as_bf16x8(t.k[sub][c]), qreg[ct][c], acc);
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
      pb[ct][0] = pack_bf16x2(x[0][0], x[0][1]);
      pb[ct][1] = pack_bf16x2(x[0][2], x[0][3]);
      pb[ct][2] = pack_bf16x2(x[1][0], x[1][1]);
      pb[ct][3] = pack_bf16x2(x[1][2], x[1][3]);
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
          oacc[ct][hf][n] = mfma_16x16x32(as_bf16x8(vt), as_bf16x8(pv), oacc[ct][hf][n]);
        }
      }
  };

  // ---- main loop: two register tiles; slot ids are fetched two tiles ahead so that
  // issuing the next tile's loads never waits on the tile still in flight ----------------
  const int n_tiles = (t_end - t_begin + 31) / 32;
  KvTile<D> ta, tb_;
  int i0a, i0b, i1a, i1b;
  load_idx(t_begin, i0a, i0b);
  load_idx(t_begin + 32, i1a, i1b);
  load_tile(ta, i0a, i0b);
  load_idx(t_begin + 64, i0a, i0b);
  for (int t = 0; t < n_tiles; t += 2) {
    const int tok = t_begin + t * 32;
    if (t + 1 < n_tiles) load_tile(tb_, i1a, i1b);
    load_idx(tok + 96, i1a, i1b);
    compute_tile(ta, tok);
    if (t + 1 < n_tiles) {
      if (t + 2 < n_tiles) load_tile(ta, i0a, i0b);
      load_idx(tok + 128, i0a, i0b);
      compute_tile(tb_, tok + 32);
    }
  }

  // ---- epilogue ----------------------------------------------------------------------
  const bool direct = (n_items == 1);
#pragma unroll
  for (int ct = 0; ct < NCT; ++ct) {
    float l = l_run[ct];
    l += __shfl_xor(l, 16, kWave);
    l += __shfl_xor(l, 32, kWave);
    const float inv = (l > 0.f) ? 1.0f / l : 0.f;
    const int col = ct * 16 + t16;
    if (col >= ncols) continue;
    const int qi = col / p.group;
    const int hh = col - qi * p.group;
    if (direct) {
      uint16_t* orow = p.out + ((int64_t)(r.q_start + qi) * p.n_q + kvh * p.group + hh) * D;
#pragma unroll
      for (int hf = 0; hf < VH; ++hf)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          u32x4_t w;
#pragma unroll
          for (int n = 0; n < 4; ++n)
            w[n] = pack_bf16x2(oacc[ct][hf][2 * n][i] * inv, oacc[ct][hf][2 * n + 1][i] * inv);
          st_global_b128(orow + hf * 128 + (4 * g + i) * 8, w);
        }
    } else {
      const int64_t prow = ((int64_t)item * p.n_kv + kvh) * p.cols_pad + col;
      float* po = p.part_o + prow * D;
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
          float* dst = po + hf * 128 + (4 * g + i) * 8;
          *reinterpret_cast<f32x4_t*>(dst) = w0;
          *reinterpret_cast<f32x4_t*>(dst + 4) = w1;
        }
      if (g == 0) p.part_lse[prow] = (l > 0.f) ? m_run[ct] + __log2f(l) : kNegInf;
    }
  }
}

// One wave per (request, query, q head): merge the request's partials by base-2 LSE.
// Requests without visible keys (or empty) get zeros; single-item requests were written
// by the attention kernel itself.
template <int D>
__global__ __launch_bounds__(64) void splitkv_merge_kernel(SplitKvParams p) {
  const int b = blockIdx.x / p.max_len_extend;
  const int qi = blockIdx.x - b * p.max_len_extend;
  const int hq = blockIdx.y;
  const int lane = lane_id();
  const ReqInfo r = request_info(p, b);
  if (qi >= r.q_len) return;
  const int n_items = num_chunks(r, p.chunk);
  if (n_items == 1) return;
  constexpr int PER = D / kWave;  // consecutive floats per lane
  uint16_t* orow = p.out + ((int64_t)(r.q_start + qi) * p.n_q + hq) * D + lane * PER;
  if (n_items == 0) {
#pragma unroll
    for (int e = 0; e < PER; ++e) orow[e] = 0;
    return;
  }
  const int kvh = hq / p.group;
  const int col = qi * p.group + (hq - kvh * p.group);
  const int base = p.req_item_base[b];
  const int64_t stride = (int64_t)p.n_kv * p.cols_pad;
  const int64_t row0 = ((int64_t)base * p.n_kv + kvh) * p.cols_pad + col;

  float mx = kNegInf;
  for (int it = lane; it < n_items; it += kWave) mx = fmaxf(mx, p.part_lse[row0 + it * stride]);
#pragma unroll
  for (int off = 1; off < kWave; off <<= 1) mx = fmaxf(mx, __shfl_xor(mx, off, kWave));
  float acc[PER];
#pragma unroll
  for (int e = 0; e < PER; ++e) acc[e] = 0.f;
  float wsum = 0.f;
  if (mx > kNegInf) {
    for (int it = 0; it < n_items; ++it) {
      const float w = fast_exp2(p.part_lse[row0 + it * stride] - mx);
      const float* src = p.part_o + (row0 + it * stride) * D + lane * PER;
#pragma unroll
      for (int e = 0; e < PER; ++e) acc[e] += w * src[e];
      wsum += w;
    }
  }
  const float inv = (wsum > 0.f) ? 1.0f / wsum : 0.f;
#pragma unroll
  for (int e = 0; e < PER; e += 2)
    *reinterpret_cast<uint32_t*>(orow + e) = pack_bf16x2(acc[e] * inv, acc[e + 1] * inv);
}

int64_t max_items_for(int64_t batch, int64_t total_kv, int32_t chunk) {
  return (total_kv + chunk - 1) / chunk + batch;
}
int cols_pad_for(int64_t cols) { return (int)((cols + 15) / 16 * 16); }

template <int D>
int launch_d(const SplitKvParams& p, int nct, int64_t n_blocks, hipStream_t stream) {
  const dim3 grid((unsigned)n_blocks), block(64);
  switch (nct) {
    case 1: hipLaunchKernelGGL((splitkv_attention_kernel<D, 1>), grid, block, 0, stream, p); break;
    case 2: hipLaunchKernelGGL((splitkv_attention_kernel<D, 2>), grid, block, 0, stream, p); break;
    case 3: hipLaunchKernelGGL((splitkv_attention_kernel<D, 3>), grid, block, 0, stream, p); break;
    case 4: hipLaunchKernelGGL((splitkv_attention_kernel<D, 4>), grid, block, 0, stream, p); break;
    default: return MSGL_ERR_SHAPE;
  }
  int rc = check_launch();
  if (rc != MSGL_OK) return rc;
  const dim3 mgrid((unsigned)(p.batch * p.max_len_extend), (unsigned)p.n_q);
  hipLaunchKernelGGL((splitkv_merge_kernel<D>), mgrid, block, 0, stream, p);
  return check_launch();
}

}  // namespace

int splitkv_default_chunk(int64_t total_kv, int64_t n_kv, int64_t cols) {
  // Enough waves to fill 256 CUs several times over, while the fp32 partial a chunk
  // writes (cols * D * 4 bytes per kv head) stays a few percent of the KV bytes it reads.
  const int64_t target_waves = 8192;
  int64_t chunk = (total_kv * n_kv + target_waves - 1) / target_waves;
  const int64_t floor_for_partials = 32 * cols;  // partial bytes <= ~3 % of KV bytes
  if (chunk < floor_for_partials) chunk = floor_for_partials;
  if (chunk < 64) chunk = 64;
  if (chunk > 4096) chunk = 4096;
  return (int)((chunk + 31) / 32 * 32);
}

size_t splitkv_workspace_bytes(int64_t batch, int64_t total_kv, int64_t n_q, int64_t n_kv,
                               int64_t head_dim, int64_t max_len_extend, int32_t chunk) {
  const int64_t group = n_q / n_kv;
  const int64_t items = max_items_for(batch, total_kv, chunk);
  const int64_t rows = items * n_kv * cols_pad_for(group * max_len_extend);
  size_t bytes = (size_t)rows * (size_t)head_dim * sizeof(float);  // part_o
  bytes += (size_t)rows * sizeof(float);                           // part_lse
  bytes += (size_t)batch * sizeof(int32_t);                        // req_item_base
  return (bytes + 255) / 256 * 256 + 256;
}

int launch_splitkv(const SplitKvArgs& a, hipStream_t stream) {
  const int64_t group = a.n_q / a.n_kv;
  const int64_t cols = group * a.max_len_extend;
  if (cols < 1 || cols > kSplitKvMaxCols || a.chunk < 32 || a.chunk % 32 != 0)
    return MSGL_ERR_SHAPE;
  const int64_t items = max_items_for(a.batch, a.total_kv, a.chunk);
  const int64_t n_blocks = items * a.n_kv;
  if (n_blocks > 0x7fffffffLL || a.batch * a.max_len_extend > 0x7fffffffLL)
    return MSGL_ERR_SHAPE;
  if (a.batch == 0) return MSGL_OK;

  SplitKvParams p;
  p.q = static_cast<const uint16_t*>(a.q);
  p.k_cache = static_cast<const uint16_t*>(a.k_cache);
  p.v_cache = static_cast<const uint16_t*>(a.v_cache);
  p.kv_indptr = a.kv_indptr;
  p.kv_indices = a.kv_indices;
  p.qo_indptr = a.qo_indptr;
  p.prefix_lens = a.prefix_lens;
  p.out = static_cast<uint16_t*>(a.out);
  p.cols_pad = cols_pad_for(cols);
  const int64_t rows = items * a.n_kv * p.cols_pad;
  char* ws = static_cast<char*>(a.workspace);
  p.part_o = reinterpret_cast<float*>(ws);
  p.part_lse = reinterpret_cast<float*>(ws + (size_t)rows * a.head_dim * sizeof(float));
  p.req_item_base = reinterpret_cast<int32_t*>(ws + (size_t)rows * (a.head_dim + 1) * sizeof(float));
  p.k_stride0 = a.k_stride0;
  p.v_stride0 = a.v_stride0;
  p.batch = (int32_t)a.batch;
  p.n_q = (int32_t)a.n_q;
  p.n_kv = (int32_t)a.n_kv;
  p.group = (int32_t)group;
  p.max_items = (int32_t)items;
  p.max_len_extend = a.max_len_extend;
  p.chunk = a.chunk;
  p.is_cross = a.is_cross;
  p.window = a.window;
  p.scale_log2e = a.sm_scale * kLog2e;
  const int nct = p.cols_pad / 16;
  if (a.head_dim == 128) return launch_d<128>(p, nct, n_blocks, stream);
  if (a.head_dim == 256) return launch_d<256>(p, nct, n_blocks, stream);
  return MSGL_ERR_HEAD_DIM;
}

}  // namespace msgl
