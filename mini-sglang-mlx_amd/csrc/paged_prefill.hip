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
#include <type_traits>

#include "msgl_device.h"
#include "msgl_internal.h"

namespace msgl {
namespace {

#ifdef MSGL_PROFILE_PHASES
#define MSGL_TICK(i) do { const long long t_ = clock64(); prof_acc[i] += t_ - prof_t; prof_t = t_; } while (0)
#else
#define MSGL_TICK(i) do { } while (0)
#endif

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
  long long* prof;  // [blocks][8] cycle totals of wave 0
#endif
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
  static constexpr int STAGES = 4;
  static constexpr int TOTAL = (STAGES * STAGE_BYTES > O_BYTES) ? STAGES * STAGE_BYTES : O_BYTES;
};

// RT = 32-row tiles per wave, NW = waves per workgroup; the workgroup covers NW*RT*32 rows.
// WIDE: pool byte offsets need 64 bits (pool of 4 GiB or more); otherwise a row's offset
// is one 32-bit multiply instead of a 64-bit multiply-add per load.
template <int D, int RT, int NW, bool WIDE>
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
  // issued back to back, heaviest (latest rows) first.  Requests are taken in order of
  // decreasing kv length (longest-processing-time-first: the dispatcher hands out blocks
  // in id order, so long requests start first and short ones fill the tail); each block
  // finds "the request of rank r" itself from kv_indptr, the host never sees the lengths.
  const int xcd = blockIdx.x & 7;
  const int seq = blockIdx.x >> 3;
  const int pair = (seq / p.n_qblk) * 8 + xcd;
  if (pair >= p.n_pairs) return;
  const int qblk = p.n_qblk - 1 - (seq % p.n_qblk);
  const int want_rank = pair / p.n_kv;
  const int kvh = pair - want_rank * p.n_kv;
  __shared__ int ranked_request;
  for (int i = tid; i < p.batch; i += NW * 64) {
    const int len_i = p.kv_indptr[i + 1] - p.kv_indptr[i];
    int rank = 0;
    for (int j = 0; j < p.batch; ++j) {
      const int len_j = p.kv_indptr[j + 1] - p.kv_indptr[j];
      rank += (len_j > len_i) || (len_j == len_i && j < i);
    }
    if (rank == want_rank) ranked_request = i;
  }
  __syncthreads();
  const int b = ranked_request;

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
  const unsigned char* kbase = reinterpret_cast<const unsigned char*>(p.k_cache + (int64_t)kvh * D + c * 8);
  const unsigned char* vbase = reinterpret_cast<const unsigned char*>(p.v_cache + (int64_t)kvh * D + c * 8);
  const uint32_t k_row_bytes = (uint32_t)p.k_stride0 * 2u;
  const uint32_t v_row_bytes = (uint32_t)p.v_stride0 * 2u;
  auto row_offset = [](uint32_t slot_id, uint32_t row_bytes) -> uint64_t {
    if constexpr (WIDE) return (uint64_t)slot_id * row_bytes;
    else return (uint64_t)(slot_id * row_bytes);
  };
  u32x4_t kr[KPT], vr[KPT];
  int32_t slot[KPT];  // slot ids of the NEXT tile to load, fetched one tile ahead
  auto slot_load = [&](int tb) {
#pragma unroll
    for (int i = 0; i < KPT; ++i) slot[i] = idx_base[min(tb + key0 + i, kn - 1)];
  };
  auto stage_load = [&]() {
#pragma unroll
    for (int i = 0; i < KPT; ++i) {
      kr[i] = ld_global_b128(kbase + row_offset((uint32_t)slot[i], k_row_bytes));
      vr[i] = ld_global_b128(vbase + row_offset((uint32_t)slot[i], v_row_bytes));
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

  // ---- the three pieces of one half tile (32 keys) --------------------------------------
  struct Scores {
    f32x16_t s[RT];  // S^T[key][row]: key = base + 8(i/4) + 4h + i%4, row = 32rt + c32
  };
  auto qk_half = [&](int buf, int kt, Scores& sc) {
    const unsigned char* ks = smem + buf * S::STAGE_BYTES + (kt * 32 + c32) * S::KROW * 2 + h * 16;
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
      for (int i = 0; i < 16; ++i) sc.s[rt][i] = 0.f;
#pragma unroll
    for (int kstep = 0; kstep < KSTEPS; ++kstep) {
      const bf16x8_t a = as_bf16x8(*reinterpret_cast<const u32x4_t*>(ks + kstep * 32));
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) sc.s[rt] = mfma_32x32x16(a, qreg[rt][kstep], sc.s[rt]);
    }
  };
  // Online softmax step over 32 keys starting at `base`.  MASKED halves scale and mask
  // explicitly; interior halves keep raw scores and fold the scale into the exp2 argument
  // (max commutes with a positive scale).
  auto softmax_half = [&](Scores& sc, int base, auto masked_tag, bf16x8_t (&pb)[RT][2],
                          float (&alpha)[RT]) {
    constexpr bool MASKED = decltype(masked_tag)::value;
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
      if constexpr (MASKED) {
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const int key = base + 8 * (i >> 2) + 4 * h + (i & 3);
          const float x = sc.s[rt][i] * p.scale_log2e;
          sc.s[rt][i] = (key < row_lo[rt] || key > row_hi[rt]) ? kNegInf : x;
        }
      }
      float mx = fmaxf(sc.s[rt][0], sc.s[rt][1]);
#pragma unroll
      for (int i = 2; i < 16; ++i) mx = fmaxf(mx, sc.s[rt][i]);
      if constexpr (!MASKED) mx *= p.scale_log2e;
      mx = wave_max_xor(mx, 32);
      const float m_old = m_run[rt];
      const float m_new = fmaxf(m_old, mx);
      const float m_use = (m_new - m_old > kLazy) ? m_new : m_old;
      const float m_safe = (m_use == kNegInf) ? 0.f : m_use;
      alpha[rt] = fast_exp2(m_old - m_safe);
      m_run[rt] = m_use;
      const float mul = MASKED ? 1.0f : p.scale_log2e;
      float psum = 0.f;
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const float e = fast_exp2(__builtin_fmaf(sc.s[rt][i], mul, -m_safe));
        sc.s[rt][i] = e;
        psum += e;
      }
      l_run[rt] = l_run[rt] * alpha[rt] + psum;
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        u32x4_t pk;
#pragma unroll
        for (int j = 0; j < 4; ++j)
          pk[j] = pack_bf16x2(sc.s[rt][8 * u + 2 * j], sc.s[rt][8 * u + 2 * j + 1]);
        pb[rt][u] = as_bf16x8(pk);
      }
    }
  };
  // O^T[dim row][row] += V^T * P^T over key positions 32kt .. 32kt+31 (two k-steps of 16)
  auto pv_half = [&](int buf, int kt, const bf16x8_t (&pb)[RT][2]) {
    const unsigned char* vs =
        smem + buf * S::STAGE_BYTES + S::K_BYTES + c32 * S::VROW * 2 + (32 * kt + 8 * h) * 2;
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) {
        const bf16x8_t a = as_bf16x8(
            *reinterpret_cast<const u32x4_t*>(vs + dt * 32 * S::VROW * 2 + u * 32));
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) oacc[dt][rt] = mfma_32x32x16(a, pb[rt][u], oacc[dt][rt]);
      }
  };
  // O *= alpha where some row's lazy max moved (rare)
  auto rescale = [&](const float (&alpha)[RT]) {
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
      if (__any(alpha[rt] != 1.0f)) {
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
          for (int i = 0; i < 16; ++i) oacc[dt][rt][i] *= alpha[rt];
      }
    }
  };
  // One pipeline step over half tiles i-1, i, i+1: the matrix pipe computes the scores of
  // half i+1 and adds P V of half i-1 while the VALU turns the scores of half i into P.
  // The three pieces are independent.  The step is cut into four slices, each holding a
  // quarter of the MFMAs (two K operands, two V operands) and a quarter of the softmax, with
  // a scheduling barrier between slices: inside a slice the compiler interleaves MFMA, LDS
  // reads and VALU freely, across slices nothing moves, which bounds operand live ranges.
  // `mul` is the factor still to be applied to the scores: the softmax scale on interior
  // halves (raw scores; max commutes with a positive scale), 1 on halves that apply_mask
  // already scaled.
  auto fused_half = [&](Scores& cur, float mul, Scores& nxt, int k_buf, int k_kt, int v_buf,
                        int v_kt, const bf16x8_t (&pb_prev)[RT][2], bf16x8_t (&pb_cur)[RT][2],
                        float (&alpha_cur)[RT]) {
    const unsigned char* ks =
        smem + k_buf * S::STAGE_BYTES + (k_kt * 32 + c32) * S::KROW * 2 + h * 16;
    const unsigned char* vs =
        smem + v_buf * S::STAGE_BYTES + S::K_BYTES + c32 * S::VROW * 2 + (32 * v_kt + 8 * h) * 2;
    // MFMA operands of one slice: two K rows-of-16-dims and two V^T rows-of-16-keys per lane
    struct Ops {
      bf16x8_t k[2], v[2];
    };
    auto load_ops = [&](int sl) {
      Ops o;
      const int u = sl >> 1;
#pragma unroll
      for (int e = 0; e < 2; ++e) {
        o.k[e] = as_bf16x8(*reinterpret_cast<const u32x4_t*>(ks + (2 * sl + e) * 32));
        o.v[e] = as_bf16x8(*reinterpret_cast<const u32x4_t*>(
            vs + (2 * (sl & 1) + e) * 32 * S::VROW * 2 + u * 32));
      }
      return o;
    };
    auto mfma_slice = [&](int sl, const Ops& o) {
      // alternate the two products: consecutive score MFMAs extend the same accumulator
      // chain, the P V ones go to different accumulators
      const int u = sl >> 1;
#pragma unroll
      for (int e = 0; e < 2; ++e) {
        const int kstep = 2 * sl + e;
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) nxt.s[rt] = mfma_32x32x16(o.k[e], qreg[rt][kstep], nxt.s[rt]);
        const int dt = 2 * (sl & 1) + e;
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) oacc[dt][rt] = mfma_32x32x16(o.v[e], pb_prev[rt][u], oacc[dt][rt]);
      }
    };
    float m_safe[RT], psum[RT];
    // pin(): the value must exist at this point of the instruction stream.  Without it the
    // optimiser sinks the softmax arithmetic out of its slice, next to its first use in the
    // following step, and the MFMAs of this step run with the VALU idle.
    auto exp_slice = [&](int first) {  // elements first .. first+7
#pragma unroll
      for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int i = first; i < first + 8; ++i) {
          float e = fast_exp2(__builtin_fmaf(cur.s[rt][i], mul, -m_safe[rt]));
          pin(e);
          cur.s[rt][i] = e;
          psum[rt] += e;
        }
    };
    auto pack_slice = [&](int u) {
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) {
        u32x4_t pk;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          uint32_t w = pack_bf16x2(cur.s[rt][8 * u + 2 * j], cur.s[rt][8 * u + 2 * j + 1]);
          pin(w);
          pk[j] = w;
        }
        pb_cur[rt][u] = as_bf16x8(pk);
      }
    };
    // slice 0: row max, lazy-max decision.  Each slice first requests the operands of the
    // next one, so LDS latency is covered by a slice of MFMA + VALU work.
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
      for (int i = 0; i < 16; ++i) nxt.s[rt][i] = 0.f;
    const Ops o0 = load_ops(0);
    const Ops o1 = load_ops(1);
    mfma_slice(0, o0);
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
      float mx = fmaxf(cur.s[rt][0], cur.s[rt][1]);
#pragma unroll
      for (int i = 2; i < 16; ++i) mx = fmaxf(mx, cur.s[rt][i]);
      mx = wave_max_xor(mx * mul, 32);
      const float m_old = m_run[rt];
      const float m_new = fmaxf(m_old, mx);
      const float m_use = (m_new - m_old > kLazy) ? m_new : m_old;
      m_safe[rt] = (m_use == kNegInf) ? 0.f : m_use;
      alpha_cur[rt] = fast_exp2(m_old - m_safe[rt]);
      m_run[rt] = m_use;
      psum[rt] = 0.f;
      pin(m_safe[rt]);
      pin(alpha_cur[rt]);
    }
    __builtin_amdgcn_sched_barrier(0);
    const Ops o2 = load_ops(2);
    mfma_slice(1, o1);
    exp_slice(0);
    __builtin_amdgcn_sched_barrier(0);
    const Ops o3 = load_ops(3);
    mfma_slice(2, o2);
    exp_slice(8);
    pack_slice(0);
    __builtin_amdgcn_sched_barrier(0);
    mfma_slice(3, o3);
    pack_slice(1);
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) l_run[rt] = l_run[rt] * alpha_cur[rt] + psum[rt];
    __builtin_amdgcn_sched_barrier(0);
  };
  auto half_step = [&](Scores& cur, int cur_base, bool need_mask, Scores& nxt, int k_buf, int k_kt,
                       int v_buf, int v_kt, const bf16x8_t (&pb_prev)[RT][2],
                       const float (&alpha_prev)[RT], bf16x8_t (&pb_cur)[RT][2],
                       float (&alpha_cur)[RT]) {
    rescale(alpha_prev);
    float mul = p.scale_log2e;
    if (need_mask) {  // boundary halves: scale and mask in place, in a block of their own
#pragma unroll
      for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const int key = cur_base + 8 * (i >> 2) + 4 * h + (i & 3);
          const float x = cur.s[rt][i] * p.scale_log2e;
          cur.s[rt][i] = (key < row_lo[rt] || key > row_hi[rt]) ? kNegInf : x;
        }
      mul = 1.0f;
    }
    fused_half(cur, mul, nxt, k_buf, k_kt, v_buf, v_kt, pb_prev, pb_cur, alpha_cur);
  };

  // ---- main loop ---------------------------------------------------------------------
  // Four LDS stages: tiles j-1 (V of its second half), j, j+1 (K of its first half) and the
  // stage being filled with tile j+2.  Every load and LDS store is unconditional (tiles past
  // the end clamp to the last key and are fully masked), so each wait is a compile-time
  // partial wait.  Rows travel HBM -> registers -> LDS with a full iteration in flight:
  // requested in the middle of iteration j-1, parked in LDS in the middle of iteration j,
  // first read in iteration j+1.
  const bool general_scale = p.scale_log2e <= 0.f;  // fast path needs a positive scale
  if (n_tiles > 0) {
    slot_load(k_lo);
    stage_load();
    slot_load(k_lo + kBN);
    stage_store(0);
    stage_load();
    slot_load(k_lo + 2 * kBN);
    stage_store(1);
    stage_load();               // rows of tile 2 stay in registers into the first iteration
    slot_load(k_lo + 3 * kBN);
    __syncthreads();
    Scores sa, sb;
    qk_half(0, 0, sa);
    bf16x8_t pb_a[RT][2], pb_b[RT][2];
    float alpha_a[RT], alpha_b[RT];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
      alpha_b[rt] = 1.0f;
#pragma unroll
      for (int u = 0; u < 2; ++u) pb_b[rt][u] = as_bf16x8(u32x4_t{0u, 0u, 0u, 0u});
    }
    // stage indices of tiles j-1, j, j+1, j+2 (the first P is zero, so "tile -1" may alias 0)
    int b_prev = 0, b_cur = 0, b_next = 1, b_fill = 2, b_spare = 3;
#ifdef MSGL_PROFILE_PHASES
    long long prof_acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    long long prof_t = clock64();
    const long long prof_c0 = prof_t, prof_w0 = wall_clock64();
#endif
    for (int j = 0; j < n_tiles; ++j) {
      const int tb = k_lo + j * kBN;
      const bool m0 = general_scale || (tb < w_lo_max) || (tb + 31 > w_hi_min);
      const bool m1 = general_scale || (tb + 32 < w_lo_max) || (tb + 63 > w_hi_min);
      // half (j,0): scores of (j,1) from K stage j, P V of (j-1,1) from V stage j-1
      half_step(sa, tb, m0, sb, b_cur, 1, b_prev, 1, pb_b, alpha_b, pb_a, alpha_a);
      MSGL_TICK(1);
      // rows of tile j+2 were requested an iteration ago: park them in the free stage, then
      // request tile j+3 (its slot ids were fetched an iteration ago as well)
      stage_store(b_fill);
      MSGL_TICK(3);
      stage_load();
      slot_load(tb + 4 * kBN);
      MSGL_TICK(0);
      // half (j,1): scores of (j+1,0) from K stage j+1, P V of (j,0) from V stage j
      half_step(sb, tb + 32, m1, sa, b_next, 0, b_cur, 0, pb_a, alpha_a, pb_b, alpha_b);
      MSGL_TICK(2);
      __syncthreads();
      MSGL_TICK(4);
      const int freed = (j == 0) ? b_spare : b_prev;  // stage of tile j-1 is free after this barrier
      b_prev = b_cur;
      b_cur = b_next;
      b_next = b_fill;
      b_fill = freed;
    }
    // the last half's P V is still owed
    rescale(alpha_b);
    pv_half(b_prev, 1, pb_b);
    __syncthreads();  // the epilogue reuses the stages as its output staging area
#ifdef MSGL_PROFILE_PHASES
    if (lane == 0) {
      long long* dst = p.prof + ((long long)blockIdx.x * 8 + w) * 8;
      for (int i = 0; i < 5; ++i) dst[i] = prof_acc[i];
      dst[5] = n_tiles;
      dst[6] = clock64() - prof_c0;
      dst[7] = wall_clock64() - prof_w0;
    }
#endif
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

#ifdef MSGL_PROFILE_PHASES
static long long* g_prof_buf = nullptr;
extern "C" __attribute__((visibility("default"))) long long* msgl_debug_prof_buffer() { return g_prof_buf; }
#endif
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
#ifdef MSGL_PROFILE_PHASES
  static long long* prof_buf = nullptr;
  if (!prof_buf) (void)hipMalloc(&prof_buf, 8192 * 64 * sizeof(long long));
  p.prof = prof_buf;
  g_prof_buf = prof_buf;
#endif
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
  const bool wide = (uint64_t)a.num_slots * (uint64_t)a.k_stride0 * 2u >= (1ull << 32) ||
                    (uint64_t)a.num_slots * (uint64_t)a.v_stride0 * 2u >= (1ull << 32);
  const dim3 grid((unsigned)n_blocks);
  if (variant == 1) {
    if (wide) hipLaunchKernelGGL((prefill_tile_kernel<128, 2, 4, true>), grid, dim3(256), 0, stream, p);
    else hipLaunchKernelGGL((prefill_tile_kernel<128, 2, 4, false>), grid, dim3(256), 0, stream, p);
  } else {
    if (wide) hipLaunchKernelGGL((prefill_tile_kernel<128, 1, 8, true>), grid, dim3(512), 0, stream, p);
    else hipLaunchKernelGGL((prefill_tile_kernel<128, 1, 8, false>), grid, dim3(512), 0, stream, p);
  }
  return check_launch();
}

}  // namespace msgl
