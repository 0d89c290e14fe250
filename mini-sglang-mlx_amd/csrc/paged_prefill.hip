// MFMA tile kernel for paged prefill / chunked extend attention on gfx950.
// Replaces paged_prefill_attention (mini-sglang-mlx-kernel/csrc/paged_prefill_attention.metal:382-640).
//
// Shape of the computation
//   workgroup  = 4 waves, 256 "rows" of one (request, kv head): row = q_idx * group + head,
//                so the `group` query heads that share a kv head sit in the same tile and
//                every K / V tile is fetched once per group (the reference fetches it once
//                per q head).  Each wave owns 64 rows = two 32-wide MFMA column tiles.
//   K/V tiles  = 64 keys, gathered through kv_indices into LDS, double buffered; one
//                barrier per tile.  K is stored row-major (padded rows); V is transposed
//                on the way in (4 keys x 8 dims per thread, v_perm_b32) so that the PV
//                operand is one 16-byte LDS read.
//   S^T        = K_tile * Q^T          mfma 32x32x16, keys on M, rows on N
//   O^T       += V_tile^T * P^T        mfma 32x32x16, dims on M, rows on N, keys on K
//   With rows on N in both products the softmax state, the bf16 P operand and the O
//   rescale are lane-local; per tile and row tile the only cross-lane step is one
//   xor-32 max.  Key order inside a PV k-step and the order of V's dims in LDS are
//   permuted (legal: one is a contraction index, the other only labels output rows) so
//   that P feeds the MFMA straight from the S accumulators and LDS writes are
//   conflict-free; the epilogue un-permutes through LDS and stores whole 256-byte rows.
//   The KV loop starts at the window floor and stops at the causal limit of the block;
//   waves skip tiles none of their rows can see.
//
// Algorithmic flops: 4 * D per visible (query, key) pair and q head (QK^T + PV).
#include <atomic>

#include "msgl_device.h"
#include "msgl_internal.h"

namespace msgl {
namespace {

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
};

constexpr int kBN = 64;  // keys per tile
// A stale row max is kept until the new one exceeds it by this much (base-2 exponent):
// P stays below 2^kLazy, far inside bf16 / fp32 range, and O is rescaled rarely.
constexpr float kLazy = 8.0f;

template <int D, int ROWS>
struct Smem {
  static constexpr int KROW = D + 8;    // bf16 elements per K row (16 B pad)
  static constexpr int VROW = kBN + 8;  // bf16 elements per V^T row
  static constexpr int K_BYTES = kBN * KROW * 2;
  static constexpr int V_BYTES = D * VROW * 2;
  static constexpr int STAGE_BYTES = K_BYTES + V_BYTES;
  static constexpr int OROW = D + 8;
  static constexpr int O_BYTES = ROWS * OROW * 2;
  static constexpr int TOTAL = (2 * STAGE_BYTES > O_BYTES) ? 2 * STAGE_BYTES : O_BYTES;
};

// RT = 32-row tiles per wave, NW = waves per workgroup; the workgroup covers NW*RT*32 rows.
template <int D, int RT, int NW>
__global__ __launch_bounds__(NW * 64) void prefill_tile_kernel(PrefillParams p) {
  static_assert(D == 128, "tile kernel is instantiated for head_dim 128");
  constexpr int kRows = NW * RT * 32;
  constexpr int KPT = kBN * 16 / (NW * 64);  // keys staged per thread (16 threads per row)
  static_assert(KPT == 4 || KPT == 2, "staging assumes 256 or 512 threads");
  using S = Smem<D, kRows>;
  constexpr int KSTEPS = D / 16;  // k-steps of QK^T
  constexpr int DT = D / 32;      // 32-row tiles of O^T
  __shared__ __attribute__((aligned(16))) unsigned char smem[S::TOTAL];

  const int tid = threadIdx.x;
  const int w = tid >> 6;
  const int lane = tid & 63;
  const int h = lane >> 5;
  const int c32 = lane & 31;

  // ---- block -> (request, kv head, q block).  Consecutive block ids go to different
  // XCDs; the q blocks of one (request, kv head) share an XCD (and its L2) and are
  // issued back to back, heaviest (latest rows) first.
  const int xcd = blockIdx.x & 7;
  const int seq = blockIdx.x >> 3;
  const int pair = (seq / p.n_qblk) * 8 + xcd;
  if (pair >= p.n_pairs) return;
  const int qblk = p.n_qblk - 1 - (seq % p.n_qblk);
  const int b = pair / p.n_kv;
  const int kvh = pair - b * p.n_kv;

  const int q_start = p.qo_indptr[b];
  const int q_len = min(p.qo_indptr[b + 1] - q_start, p.max_len_extend);
  const int kv_start = p.kv_indptr[b];
  const int kn = max(p.kv_indptr[b + 1] - kv_start, 0);
  const int prefix = p.prefix_lens[b];
  const int rows_total = q_len * p.group;
  const int row0 = qblk * kRows;
  if (row0 >= rows_total) return;

  const int qi_lo = row0 / p.group;
  const int qi_hi = min(rows_total - 1, row0 + kRows - 1) / p.group;
  int k_hi = p.is_cross ? kn : min(kn, prefix + qi_hi + 1);
  int k_lo = (p.window > 0) ? max(0, prefix + qi_lo - p.window + 1) : 0;
  k_lo &= ~(kBN - 1);
  if (k_hi < k_lo) k_hi = k_lo;
  const int n_tiles = (k_hi - k_lo + kBN - 1) / kBN;

  // ---- per-lane rows: Q operand, visibility bounds ---------------------------------
  bf16x8_t qreg[RT][KSTEPS];
  int row_lo[RT], row_hi[RT];
  int w_lo_min = 0x7fffffff, w_lo_max = -0x7fffffff, w_hi_min = 0x7fffffff, w_hi_max = -1;
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    const int row = row0 + (w * RT + rt) * 32 + c32;
    const bool valid = row < rows_total;
    const int qi = valid ? row / p.group : 0;
    const int hh = valid ? row - qi * p.group : 0;
    const int64_t off = ((int64_t)(q_start + qi) * p.n_q + kvh * p.group + hh) * D;
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) {
      u32x4_t raw = {0u, 0u, 0u, 0u};
      if (valid) raw = ld_global_b128(p.q + off + ks * 16 + h * 8);
      qreg[rt][ks] = as_bf16x8(raw);
    }
    const int qpos = prefix + qi;
    int lo = (p.window > 0) ? qpos - p.window + 1 : 0;
    int hi = p.is_cross ? kn - 1 : min(qpos, kn - 1);
    if (valid) {
      w_lo_min = min(w_lo_min, lo);
      w_lo_max = max(w_lo_max, lo);
      w_hi_min = min(w_hi_min, hi);
      w_hi_max = max(w_hi_max, hi);
    } else {
      lo = 1;
      hi = 0;
    }
    row_lo[rt] = lo;
    row_hi[rt] = hi;
  }
#pragma unroll
  for (int off = 1; off < kWave; off <<= 1) {
    w_lo_min = min(w_lo_min, __shfl_xor(w_lo_min, off, kWave));
    w_lo_max = max(w_lo_max, __shfl_xor(w_lo_max, off, kWave));
    w_hi_min = min(w_hi_min, __shfl_xor(w_hi_min, off, kWave));
    w_hi_max = max(w_hi_max, __shfl_xor(w_hi_max, off, kWave));
  }
  w_lo_min = __builtin_amdgcn_readfirstlane(w_lo_min);
  w_lo_max = __builtin_amdgcn_readfirstlane(w_lo_max);
  w_hi_min = __builtin_amdgcn_readfirstlane(w_hi_min);
  w_hi_max = __builtin_amdgcn_readfirstlane(w_hi_max);

  f32x16_t oacc[DT][RT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
      for (int i = 0; i < 16; ++i) oacc[dt][rt][i] = 0.f;
  float m_run[RT], l_run[RT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    m_run[rt] = kNegInf;
    l_run[rt] = 0.f;
  }

  // ---- staging: thread (kg, c) moves keys KPT*kg .. KPT*kg+KPT-1, dims 8c..8c+7 -------
  const int kg = tid >> 4;
  const int c = tid & 15;
  const int key0 = kg * KPT;
  const int pos0 = (key0 & ~12) | ((key0 & 4) << 1) | ((key0 & 8) >> 1);  // key bits 2 <-> 3
  const int32_t* idx_base = p.kv_indices + kv_start;
  const uint16_t* kbase = p.k_cache + (int64_t)kvh * D + c * 8;
  const uint16_t* vbase = p.v_cache + (int64_t)kvh * D + c * 8;
  u32x4_t kr[KPT], vr[KPT];
  int32_t slot[KPT];  // slot ids of the NEXT tile to load, fetched one tile ahead
  auto slot_load = [&](int tb) {
#pragma unroll
    for (int i = 0; i < KPT; ++i) slot[i] = idx_base[min(tb + key0 + i, kn - 1)];
  };
  auto stage_load = [&]() {
#pragma unroll
    for (int i = 0; i < KPT; ++i) {
      kr[i] = ld_global_b128(kbase + (int64_t)slot[i] * p.k_stride0);
      vr[i] = ld_global_b128(vbase + (int64_t)slot[i] * p.v_stride0);
    }
  };
  auto stage_store = [&](int buf) {
    unsigned char* ks = smem + buf * S::STAGE_BYTES;
    unsigned char* vs = ks + S::K_BYTES;
#pragma unroll
    for (int i = 0; i < KPT; ++i)
      *reinterpret_cast<u32x4_t*>(ks + ((key0 + i) * S::KROW + c * 8) * 2) = kr[i];
    // V^T row of dim 8c+n is 16n+c: the 16 lanes of one write hit consecutive rows
#pragma unroll
    for (int n = 0; n < 8; ++n) {
      unsigned char* dst = vs + ((16 * n + c) * S::VROW + pos0) * 2;
      const uint32_t t0 = (n & 1) ? pack_hi16(vr[0][n >> 1], vr[1][n >> 1])
                                  : pack_lo16(vr[0][n >> 1], vr[1][n >> 1]);
      if constexpr (KPT == 4) {
        u32x2_t t;
        t[0] = t0;
        t[1] = (n & 1) ? pack_hi16(vr[2][n >> 1], vr[3][n >> 1])
                       : pack_lo16(vr[2][n >> 1], vr[3][n >> 1]);
        *reinterpret_cast<u32x2_t*>(dst) = t;
      } else {
        *reinterpret_cast<uint32_t*>(dst) = t0;
      }
    }
  };

  auto compute_tile = [&](int buf, int tb) {
    const unsigned char* ks = smem + buf * S::STAGE_BYTES;
    const unsigned char* vs = ks + S::K_BYTES;
    // S^T[key][row]: lane holds key = tb + 32kt + 8(i/4) + 4h + i%4, row = 32rt + c32
    f32x16_t s[2][RT];
#pragma unroll
    for (int kt = 0; kt < 2; ++kt)
#pragma unroll
      for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int i = 0; i < 16; ++i) s[kt][rt][i] = 0.f;
#pragma unroll
    for (int kstep = 0; kstep < KSTEPS; ++kstep)
#pragma unroll
      for (int kt = 0; kt < 2; ++kt) {
        const bf16x8_t a = as_bf16x8(*reinterpret_cast<const u32x4_t*>(
            ks + ((kt * 32 + c32) * S::KROW + kstep * 16 + h * 8) * 2));
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) s[kt][rt] = mfma_32x32x16(a, qreg[rt][kstep], s[kt][rt]);
      }

    const bool need_mask = (tb < w_lo_max) || (tb + kBN - 1 > w_hi_min);
    bf16x8_t pb[RT][4];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
      if (need_mask) {
#pragma unroll
        for (int kt = 0; kt < 2; ++kt)
#pragma unroll
          for (int i = 0; i < 16; ++i) {
            const int key = tb + kt * 32 + 8 * (i >> 2) + 4 * h + (i & 3);
            const float x = s[kt][rt][i] * p.scale_log2e;
            s[kt][rt][i] = (key < row_lo[rt] || key > row_hi[rt]) ? kNegInf : x;
          }
      }
      float mx = kNegInf;
#pragma unroll
      for (int kt = 0; kt < 2; ++kt)
#pragma unroll
        for (int i = 0; i < 16; ++i) mx = fmaxf(mx, s[kt][rt][i]);
      // unmasked tiles keep raw scores: max commutes with a non-negative scale
      if (!need_mask) {
        if (p.scale_log2e < 0.f) {
          mx = -kNegInf;
#pragma unroll
          for (int kt = 0; kt < 2; ++kt)
#pragma unroll
            for (int i = 0; i < 16; ++i) mx = fminf(mx, s[kt][rt][i]);
        }
        mx *= p.scale_log2e;
      }
      mx = wave_max_xor(mx, 32);
      const float m_old = m_run[rt];
      const float m_new = fmaxf(m_old, mx);
      const float m_use = (m_new - m_old > kLazy) ? m_new : m_old;
      const float m_safe = (m_use == kNegInf) ? 0.f : m_use;
      const float alpha = fast_exp2(m_old - m_safe);
      m_run[rt] = m_use;
      const float mul = need_mask ? 1.0f : p.scale_log2e;
      float psum = 0.f;
#pragma unroll
      for (int kt = 0; kt < 2; ++kt)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const float e = fast_exp2(__builtin_fmaf(s[kt][rt][i], mul, -m_safe));
          s[kt][rt][i] = e;
          psum += e;
        }
      l_run[rt] = l_run[rt] * alpha + psum;
      if (__any(alpha != 1.0f)) {
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
          for (int i = 0; i < 16; ++i) oacc[dt][rt][i] *= alpha;
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        u32x4_t pk;
#pragma unroll
        for (int j = 0; j < 4; ++j)
          pk[j] = pack_bf16x2(s[u >> 1][rt][8 * (u & 1) + 2 * j], s[u >> 1][rt][8 * (u & 1) + 2 * j + 1]);
        pb[rt][u] = as_bf16x8(pk);
      }
    }
    // O^T[dim row][row] += V^T * P^T ; k-step u covers key positions 16u .. 16u+15
#pragma unroll
    for (int u = 0; u < 4; ++u)
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) {
        const bf16x8_t a = as_bf16x8(*reinterpret_cast<const u32x4_t*>(
            vs + ((dt * 32 + c32) * S::VROW + 16 * u + 8 * h) * 2));
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) oacc[dt][rt] = mfma_32x32x16(a, pb[rt][u], oacc[dt][rt]);
      }
  };

  // ---- main loop ---------------------------------------------------------------------
  // Every load and LDS store below is unconditional (tiles past the end clamp to the last
  // key and are never read), so the loop body has one fixed sequence of memory operations:
  // the next tile's rows are in flight during the whole compute phase and the slot ids of
  // the tile after it were fetched a full iteration earlier.
  if (n_tiles > 0) {
    slot_load(k_lo);
    stage_load();
    slot_load(k_lo + kBN);
    stage_store(0);
    __syncthreads();
    for (int t = 0; t < n_tiles; ++t) {
      const int tb = k_lo + t * kBN;
      stage_load();                // rows of tile t+1
      slot_load(tb + 2 * kBN);     // slot ids of tile t+2
      if (tb <= w_hi_max && tb + kBN - 1 >= w_lo_min) compute_tile(t & 1, tb);
      stage_store((t + 1) & 1);
      __syncthreads();
    }
  }

  // ---- epilogue: normalise, un-permute through LDS, store whole rows -----------------
  // O^T row R = 32dt + 8(i/4) + 4h + i%4 holds dim 8(R%16) + R/16, so for fixed i < 8 the
  // eight values {oacc[dt][i], oacc[dt][i+8]}, dt = 0..3, are dims 8X .. 8X+7 with
  // X = 8((i/4)&1) + 4h + i%4.
  unsigned char* os = smem;
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    float l = l_run[rt];
    l += __shfl_xor(l, 32, kWave);
    const float inv = (l > 0.f) ? 1.0f / l : 0.f;
    const int lrow = (w * RT + rt) * 32 + c32;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      u32x4_t wv;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
        wv[dt] = pack_bf16x2(oacc[dt][rt][i] * inv, oacc[dt][rt][i + 8] * inv);
      const int X = 8 * ((i >> 2) & 1) + 4 * h + (i & 3);
      *reinterpret_cast<u32x4_t*>(os + (lrow * S::OROW + 8 * X) * 2) = wv;
    }
  }
  __syncthreads();
  constexpr int ROWS_PER_PASS = NW * 4;
#pragma unroll 4
  for (int pass = 0; pass < kRows / ROWS_PER_PASS; ++pass) {
    const int lrow = pass * ROWS_PER_PASS + (tid >> 4);
    const int row = row0 + lrow;
    if (row < rows_total) {
      const int qi = row / p.group;
      const int hh = row - qi * p.group;
      const u32x4_t v = *reinterpret_cast<const u32x4_t*>(os + (lrow * S::OROW + c * 8) * 2);
      st_global_b128(p.out + ((int64_t)(q_start + qi) * p.n_q + kvh * p.group + hh) * D + c * 8, v);
    }
  }
}

}  // namespace

static std::atomic<int> g_tile_variant{0};
int tile_variant() { return g_tile_variant.load(); }
void set_tile_variant(int v) { g_tile_variant.store(v); }

int launch_prefill_tile(const PrefillArgs& a, hipStream_t stream) {
  if (a.head_dim != 128) return MSGL_ERR_HEAD_DIM;
  PrefillParams p;
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
  p.scale_log2e = a.sm_scale * kLog2e;
  const int variant = tile_variant();
  const int64_t block_rows = 256;
  const int64_t rows = (int64_t)a.max_len_extend * p.group;
  const int64_t n_qblk = (rows + block_rows - 1) / block_rows;
  const int64_t n_pairs = a.batch * a.n_kv;
  const int64_t n_blocks = (n_pairs + 7) / 8 * 8 * n_qblk;
  if (n_qblk <= 0 || n_blocks <= 0) return MSGL_OK;
  if (n_blocks > 0x7fffffffLL) return MSGL_ERR_SHAPE;
  p.n_qblk = (int32_t)n_qblk;
  p.n_pairs = (int32_t)n_pairs;
  if (variant == 1)
    hipLaunchKernelGGL((prefill_tile_kernel<128, 2, 4>), dim3((unsigned)n_blocks), dim3(256), 0,
                       stream, p);
  else
    hipLaunchKernelGGL((prefill_tile_kernel<128, 1, 8>), dim3((unsigned)n_blocks), dim3(512), 0,
                       stream, p);
  return check_launch();
}

}  // namespace msgl
