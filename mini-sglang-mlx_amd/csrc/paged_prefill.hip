// MFMA tile kernel for paged prefill / chunked extend attention on gfx950, with K and V
// rows moved HBM -> LDS by the memory pipeline itself (no staging registers, no VALU work).
// Replaces paged_prefill_attention (mini-sglang-mlx-kernel/csrc/paged_prefill_attention.metal:382-640).
//
// Shape of the computation
//   workgroup  = NW waves, 256 "rows" of one (request, kv head): row = q_idx * group + head,
//                so the `group` query heads that share a kv head sit in the same tile and
//                every K / V tile is fetched once per group (the reference fetches it once
//                per q head).  A wave owns RT 32-row tiles.
//   K/V tiles  = 64 keys gathered through kv_indices.  One global_load_lds_dwordx4 moves four
//                whole 256-byte rows (64 lanes x 16 B) into 1 KiB of LDS; the four rows of
//                "unit" u are keys u, u+16, u+32, u+48 of the tile and consecutive units sit
//                1040 B (K) or 1088 B (V) apart, so that the 16 lanes of one LDS read phase,
//                which want the same 16 B of 16 consecutive keys (K) or 32 B of 4 consecutive
//                keys at two dim offsets (V), fall into different banks.
//   S^T        = K_tile * Q^T          mfma 32x32x16, keys on M, rows on N
//   O^T       += V_tile^T * P^T        mfma 32x32x16, dims on M, rows on N, keys on K;
//                the V^T operand (8 keys of one dim per lane) comes from row-major V through
//                two ds_read_b64_tr_b16, which transpose 4 keys x 16 dims across 16 lanes.
//   With rows on N in both products the softmax state, the bf16 P operand and the O
//   rescale are lane-local; per half tile and row tile the only cross-lane step is one
//   xor-32 max.  Key order inside a PV k-step follows the S^T accumulator layout (legal:
//   it is a contraction index), so P feeds the MFMA straight from the S accumulators.
//   The KV loop starts at the window floor and stops at the causal limit of the block;
//   boundary half tiles are scaled and masked in place before their softmax.
//
// Algorithmic flops: 4 * D per visible (query, key) pair and q head (QK^T + PV).
#include <type_traits>

#include "msgl_device.h"
#include "msgl_internal.h"
#include "prefill_params.h"
#include "prefill_tile_common.h"

namespace msgl {
namespace {

constexpr int kUnitRows = 4;                 // rows moved by one LDS-direct load
constexpr int kUnits = kBN / kUnitRows;      // 16 per tile
constexpr int kKUnit = 1024 + 16;            // bytes between K units
constexpr int kVUnit = 1024 + 64;            // bytes between V units
constexpr int kKStage = kUnits * kKUnit;     // 16640
constexpr int kVStage = kUnits * kVUnit;     // 17408
constexpr int kKStages = 3, kVStages = 3;
constexpr int kVBase = kKStages * kKStage;
constexpr int kStageTotal = kVBase + kVStages * kVStage;

// RT = 32-row tiles per wave, NW = waves per workgroup; the workgroup covers NW*RT*32 rows.
// WIDE: pool byte offsets need 64 bits (pool of 4 GiB or more).
template <int D, int RT, int NW, bool WIDE>
__global__ __launch_bounds__(NW * 64) void prefill_tile_kernel(PrefillParams p) {
  static_assert(D == 128, "tile kernel is instantiated for head_dim 128");
  constexpr int kRows = NW * RT * 32;
  constexpr int UPW = kUnits / NW;  // units each wave moves per tile
  static_assert(UPW * NW == kUnits, "waves must divide the units of a tile");
  constexpr int KSTEPS = D / 16;  // k-steps of QK^T
  constexpr int DT = D / 32;      // 32-row tiles of O^T
  constexpr int OROW = D + 8;
  constexpr int O_BYTES = kRows * OROW * 2;
  constexpr int SMEM_BYTES = kStageTotal > O_BYTES ? kStageTotal : O_BYTES;
  __shared__ __attribute__((aligned(16))) unsigned char smem[SMEM_BYTES];
  using OffT = typename std::conditional<WIDE, uint64_t, uint32_t>::type;

  const int tid = threadIdx.x;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63;
  const int h = lane >> 5;
  const int c32 = lane & 31;

  // ---- block -> (request, kv head, key split, q block).  Consecutive block ids go to
  // different XCDs; the q blocks of one (request, kv head, key split) read the same keys,
  // share an XCD (and its L2) and are issued back to back, heaviest (latest rows) first.  Requests are taken in order of
  // decreasing kv length (longest-processing-time-first: the dispatcher hands out blocks
  // in id order, so long requests start first and short ones fill the tail); each block
  // finds "the request of rank r" itself from kv_indptr, the host never sees the lengths.
  // Beyond kRankedBatch requests the order is the batch order.
  const BlockWork work = prefill_block_work(p);
  if (!work.ok) return;
  const int unit = work.unit;  // (request, kv head, key split)
  const int pair = unit / p.n_ksplit;
  const int split = unit - pair * p.n_ksplit;
  const int qblk = work.qblk;
  const int want_rank = pair / p.n_kv;
  const int kvh = pair - want_rank * p.n_kv;
  const int b = request_of_rank<NW * 64>(p.kv_indptr, p.batch, want_rank, tid);

  const int q_start = p.qo_indptr[b];
  const int q_len = min(p.qo_indptr[b + 1] - q_start, p.max_len_extend);
  const int kv_start = p.kv_indptr[b];
  const int kn = max(p.kv_indptr[b + 1] - kv_start, 0);
  const int prefix = p.prefix_lens[b];
  const int rows_total = q_len * p.group;
  const int row0 = qblk * kRows;
  if (row0 >= rows_total) return;

  // A wave all of whose rows lie past the end of the request's rows (possible in its last query
  // block) takes part in moving tiles and in every barrier but computes nothing: its SIMD's
  // matrix pipe is left to the wave that shares it.
  const bool idle = __builtin_amdgcn_readfirstlane(row0 + w * RT * 32 >= rows_total ? 1 : 0) != 0;
  const int qi_lo = row0 / p.group;
  const int qi_hi = min(rows_total - 1, row0 + kRows - 1) / p.group;
  int k_hi = p.is_cross ? kn : min(kn, prefix + qi_hi + 1);
  int k_lo = (p.window > 0) ? max(0, prefix + qi_lo - p.window + 1) : 0;
  k_lo &= ~(kBN - 1);
  if (k_hi < k_lo) k_hi = k_lo;
  // key split `split` of n_ksplit: a whole number of tiles each, the last takes the ragged end;
  // shares past the end are empty (they still leave their "nothing seen" partial)
  if (p.n_ksplit > 1) {
    const int all_tiles = (k_hi - k_lo + kBN - 1) / kBN;
    const int share = (all_tiles + p.n_ksplit - 1) / p.n_ksplit * kBN;
    k_lo = min(k_lo + split * share, k_hi);
    k_hi = min(k_hi, k_lo + share);
  }
  const int n_tiles = (k_hi - k_lo + kBN - 1) / kBN;

  // ---- per-lane rows: Q operand, visibility bounds ---------------------------------
  bf16x8_t qreg[RT][KSTEPS];
  int row_lo[RT], row_hi[RT];
  int w_lo_max = -0x7fffffff, w_hi_min = 0x7fffffff;
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
    // k_hi - 1 only binds under a key split: the pipeline looks one half tile past its share
    int hi = min(p.is_cross ? kn - 1 : min(qpos, kn - 1), k_hi - 1);
    if (valid) {
      w_lo_max = max(w_lo_max, lo);
      w_hi_min = min(w_hi_min, hi);
    } else {
      lo = 1;
      hi = 0;
    }
    row_lo[rt] = lo;
    row_hi[rt] = hi;
  }
#pragma unroll
  for (int off = 1; off < kWave; off <<= 1) {
    w_lo_max = max(w_lo_max, __shfl_xor(w_lo_max, off, kWave));
    w_hi_min = min(w_hi_min, __shfl_xor(w_hi_min, off, kWave));
  }
  w_lo_max = __builtin_amdgcn_readfirstlane(w_lo_max);
  w_hi_min = __builtin_amdgcn_readfirstlane(w_hi_min);

  f32x16_t oacc[DT][RT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
      for (int i = 0; i < 16; ++i) oacc[dt][rt][i] = 0.f;
  float m_run[RT], l_run[RT], m_safe_run[RT];  // m_safe_run: m_run, or 0 while m_run is -inf
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    m_run[rt] = kNegInf;
    l_run[rt] = 0.f;
    m_safe_run[rt] = 0.f;
  }

  // ---- moving a tile: wave w owns units w*UPW .. w*UPW+UPW-1; in a unit, lane l fetches
  // 16-byte chunk l%16 of key (unit + 16 (l/16)) ------------------------------------------
  const uint32_t lds0 = (uint32_t)(uintptr_t)MSGL_LDS_PTR(unsigned char, smem);
  const int32_t* idx_base = p.kv_indices + kv_start;
  const unsigned char* k_src = reinterpret_cast<const unsigned char*>(p.k_cache + (int64_t)kvh * D);
  const unsigned char* v_src = reinterpret_cast<const unsigned char*>(p.v_cache + (int64_t)kvh * D);
  const uint32_t k_row_bytes = (uint32_t)p.k_stride0 * 2u;
  const uint32_t v_row_bytes = (uint32_t)p.v_stride0 * 2u;
  const uint32_t chunk_off = (uint32_t)(lane & 15) * 16u;
  const int unit_key = w * UPW + 16 * (lane >> 4);  // + i for unit i of this wave
  // slot ids are clamped to the pool before they become addresses
  auto row_offset = [&](int32_t slot_id, uint32_t row_bytes) -> OffT {
    const uint32_t id = min((uint32_t)slot_id, p.max_slot);
    if constexpr (WIDE) return (uint64_t)id * row_bytes + chunk_off;
    else return __umul24(id, row_bytes) + chunk_off;  // both below 2^24 here
  };
  int32_t slot[UPW];  // slot ids of the tile whose K moves next, fetched one iteration ahead
  OffT k_off[UPW];    // K row offsets of that tile
  OffT v_off[UPW];    // V row offsets of the tile whose K went out one iteration ago
  OffT v_off_next[UPW];
  auto slot_load = [&](int tb) {
#pragma unroll
    for (int i = 0; i < UPW; ++i) slot[i] = idx_base[min(tb + unit_key + i, kn - 1)];
  };
  auto offsets_from_slots = [&]() {
#pragma unroll
    for (int i = 0; i < UPW; ++i) {
      k_off[i] = row_offset(slot[i], k_row_bytes);
      v_off_next[i] = row_offset(slot[i], v_row_bytes);
    }
  };
  auto rotate_v_offsets = [&]() {
#pragma unroll
    for (int i = 0; i < UPW; ++i) v_off[i] = v_off_next[i];
  };
  // move number n of an iteration: the V units first, then the K units
  auto move = [&](int n, uint32_t k_stage, uint32_t v_stage) {
    if (n < UPW)
      lds_direct_b128(lds0 + v_stage + (uint32_t)(w * UPW + n) * kVUnit, v_src, v_off[n]);
    else
      lds_direct_b128(lds0 + k_stage + (uint32_t)(w * UPW + n - UPW) * kKUnit, k_src, k_off[n - UPW]);
  };

  // per-lane LDS read offsets inside a stage
  //   K operand of MFMA row c32 (key 32kt + c32): unit c32 % 16, row 2kt + c32/16
  const uint32_t k_lane = (uint32_t)(c32 & 15) * kKUnit + (uint32_t)(c32 >> 4) * 256u + (uint32_t)h * 16u;
  //   V^T operand: group g = lane/16 reads dims 16 (g%2) .. +15 of keys 4h .. 4h+3 (+8)
  const uint32_t v_lane = (uint32_t)(4 * h + ((lane & 15) >> 2)) * kVUnit +
                          (uint32_t)((lane >> 4) & 1) * 32u + (uint32_t)(lane & 3) * 8u;

  // ---- the pieces of one half tile (32 keys) ----------------------------------------------
  struct Scores {
    f32x16_t s[RT];  // S^T[key][row]: key = base + 8(i/4) + 4h + i%4, row = 32rt + c32
  };
  auto k_operand = [&](const unsigned char* ks, int kstep) {
    return as_bf16x8(*reinterpret_cast<const u32x4_t*>(ks + kstep * 32));
  };
  // keys {16u + 4h + e} and {16u + 8 + 4h + e}, e = 0..3, of the half: the S^T rows that the
  // lane's accumulators 8u .. 8u+7 hold
  auto v_operand = [&](const unsigned char* vs, int u, int dt) {
    const u32x2_t lo = lds_read_tr16(vs + u * 256 + dt * 64);
    const u32x2_t hi = lds_read_tr16(vs + u * 256 + dt * 64 + 8 * kVUnit);
    return as_bf16x8(u32x4_t{lo[0], lo[1], hi[0], hi[1]});
  };
  auto qk_half = [&](uint32_t k_stage, int kt, Scores& sc) {
    const unsigned char* ks = smem + k_stage + k_lane + kt * 512;
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
      for (int i = 0; i < 16; ++i) sc.s[rt][i] = 0.f;
#pragma unroll
    for (int kstep = 0; kstep < KSTEPS; ++kstep) {
      const bf16x8_t a = k_operand(ks, kstep);
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) sc.s[rt] = mfma_32x32x16(a, qreg[rt][kstep], sc.s[rt]);
    }
  };
  auto pv_half = [&](uint32_t v_stage, int kt, const bf16x8_t (&pb)[RT][2]) {
    const unsigned char* vs = smem + v_stage + v_lane + kt * 512;
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) {
        const bf16x8_t a = v_operand(vs, u, dt);
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
  // Softmax state of one half tile, decided as soon as its scores exist:
  //   mul    factor still to be applied to the scores: the softmax scale on interior halves
  //          (raw scores; max commutes with a positive scale), 1 on boundary halves, which
  //          are scaled and masked in place
  //   m_safe the (lazy) running row max the half's exponentials are taken against
  //   alpha  exp2(previous max - m_safe): what O and l must be multiplied by first
  struct Stats {
    float mul;
    float m_safe[RT], alpha[RT];
  };
  auto mask_in_place = [&](Scores& sc, int base) {
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int key = base + 8 * (i >> 2) + 4 * h + (i & 3);
        const float x = sc.s[rt][i] * p.scale_log2e;
        sc.s[rt][i] = (key < row_lo[rt] || key > row_hi[rt]) ? kNegInf : x;
      }
  };
  auto lane_max = [&](const Scores& sc, float (&mx)[RT]) {
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
      float m = fmaxf(sc.s[rt][0], sc.s[rt][1]);
#pragma unroll
      for (int i = 2; i < 16; ++i) m = fmaxf(m, sc.s[rt][i]);
      mx[rt] = m;
    }
  };
  auto decide = [&](const float (&mx)[RT], Stats& st) {
    // Usual case: no lane of the wave saw a score more than kLazy above its row's running max.
    // Then no row's max moves (the other half of a row sits in this wave too), the state stays
    // as it is, and the cross-lane exchange, the selects and the exponential below are skipped:
    // one multiply, one compare and a scalar branch instead of a dozen instructions and an LDS
    // round trip.  The first tile (running max -inf) and fully masked halves take the long way.
    bool grew = false;
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) grew |= (mx[rt] * st.mul > m_run[rt] + kLazy);
    if (!__any(grew)) {
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) {
        st.m_safe[rt] = m_safe_run[rt];
        st.alpha[rt] = 1.0f;
      }
      return;
    }
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
      const float m = wave_max_xor(mx[rt] * st.mul, 32);
      const float m_old = m_run[rt];
      const float m_new = fmaxf(m_old, m);
      const float m_use = (m_new - m_old > kLazy) ? m_new : m_old;
      st.m_safe[rt] = (m_use == kNegInf) ? 0.f : m_use;
      m_safe_run[rt] = st.m_safe[rt];
      st.alpha[rt] = fast_exp2(m_old - st.m_safe[rt]);
      m_run[rt] = m_use;
      pin(st.m_safe[rt]);
      pin(st.alpha[rt]);
    }
  };
  // One pipeline step over half tiles i-1, i, i+1.  The matrix pipe computes the scores of
  // half i+1 (slices 0, 1) and adds P V of half i-1 (slices 2, 3); meanwhile the VALU turns
  // the scores of half i into P (slices 0..2) and, once the scores of half i+1 exist, takes
  // their row max and settles that half's softmax state (slices 2, 3), so the next step can
  // start exponentiating at once instead of waiting for a max -> exp dependency chain.
  // A scheduling barrier separates the slices: inside a slice the compiler interleaves MFMA,
  // LDS reads and VALU freely, across slices nothing moves, which bounds operand live ranges.
  // Each slice requests the LDS operands of the next one; the last slice requests the first
  // K operands of the next step (`kops`, carried between calls, also across the barrier: that
  // K tile was published a full iteration earlier).
  // `side(slice)` is a hook for work that rides along (the moves of the next tiles).
  auto fused_half = [&](Scores& cur, const Stats& st_cur, Scores& nxt, Stats& st_nxt, bool mask_nxt,
                        int nxt_base, const unsigned char* ks, const unsigned char* vs,
                        const unsigned char* ks_after, bf16x8_t (&kops)[4],
                        const bf16x8_t (&pb_prev)[RT][2], bf16x8_t (&pb_cur)[RT][2], auto&& side) {
    float psum[RT];
    // pin(): the value must exist at this point of the instruction stream.  Without it the
    // optimiser sinks the softmax arithmetic out of its slice, next to its first use in the
    // following step, and the MFMAs of this step run with the VALU idle.
    auto exp_slice = [&](int first) {  // elements first .. first+7
#pragma unroll
      for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int i = first; i < first + 8; ++i) {
          float e = fast_exp2(__builtin_fmaf(cur.s[rt][i], st_cur.mul, -st_cur.m_safe[rt]));
          pin(e);
          cur.s[rt][i] = e;
        }
    };
    auto pack_slice = [&](int u) {
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) {
        u32x4_t pk;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          uint32_t pw = pack_bf16x2(cur.s[rt][8 * u + 2 * j], cur.s[rt][8 * u + 2 * j + 1]);
          pin(pw);
          pk[j] = pw;
          // row sum of the rounded weights, the ones that multiply V
          psum[rt] = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, pw), kOnes, psum[rt], false);
        }
        pb_cur[rt][u] = as_bf16x8(pk);
      }
    };
    auto qk_slice = [&](int first, const bf16x8_t (&ops)[4]) {  // k-steps first .. first+3
#pragma unroll
      for (int e = 0; e < 4; ++e)
#pragma unroll
        for (int rt = 0; rt < RT; ++rt)
          nxt.s[rt] = mfma_32x32x16(ops[e], qreg[rt][first + e], nxt.s[rt]);
    };
    auto pv_slice = [&](int u, const bf16x8_t (&ops)[4]) {  // 16 keys, all four dim tiles
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) oacc[dt][rt] = mfma_32x32x16(ops[dt], pb_prev[rt][u], oacc[dt][rt]);
    };
    bf16x8_t ops_a[4], ops_b[4];
    // slice 0
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
      psum[rt] = 0.f;
#pragma unroll
      for (int i = 0; i < 16; ++i) nxt.s[rt][i] = 0.f;
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) ops_a[e] = k_operand(ks, 4 + e);
    qk_slice(0, kops);
    exp_slice(0);
    side(0);
    __builtin_amdgcn_sched_barrier(0);
    // slice 1
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) ops_b[dt] = v_operand(vs, 0, dt);
    qk_slice(4, ops_a);
    exp_slice(8);
    pack_slice(0);
    side(1);
    __builtin_amdgcn_sched_barrier(0);
    st_nxt.mul = p.scale_log2e;
    if (mask_nxt) {  // boundary half: scale and mask in place
      // the empty volatile statement keeps this a branch: turned into selects it would put
      // 64 extra VALU instructions into every half tile
      asm volatile("" ::: "memory");
      mask_in_place(nxt, nxt_base);
      st_nxt.mul = 1.0f;
    }
    // slice 2
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) ops_a[dt] = v_operand(vs, 1, dt);
    pv_slice(0, ops_b);
    pack_slice(1);
    float mx[RT];
    lane_max(nxt, mx);
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) pin(mx[rt]);
    side(2);
    __builtin_amdgcn_sched_barrier(0);
    // slice 3
#pragma unroll
    for (int e = 0; e < 4; ++e) kops[e] = k_operand(ks_after, e);
    pv_slice(1, ops_a);
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) l_run[rt] = l_run[rt] * st_cur.alpha[rt] + psum[rt];
    decide(mx, st_nxt);
    side(3);
    __builtin_amdgcn_sched_barrier(0);
  };

  // ---- main loop ---------------------------------------------------------------------
  // Iteration j reads K of tiles j (second half's scores) and j+1 (first half of the next
  // tile) and V of tiles j-1 and j, while K of tile j+2 and V of tile j+1 travel into the
  // third K and V stages.  Every move is unconditional (tiles past the end clamp to the last
  // key and are fully masked).  A wave waits for its own moves at the end of the iteration,
  // then the workgroup barrier publishes them: one barrier per tile.
  const bool general_scale = p.scale_log2e <= 0.f;  // fast path needs a positive scale
  auto needs_mask = [&](int base) {  // some row of this wave sees only part of keys base .. base+31
    return general_scale || (base < w_lo_max) || (base + 31 > w_hi_min);
  };
  if (n_tiles > 0) {
    slot_load(k_lo);
    offsets_from_slots();
    rotate_v_offsets();
#pragma unroll
    for (int n = 0; n < 2 * UPW; ++n) move(n, 0, kVBase);  // tile 0
    slot_load(k_lo + kBN);
    offsets_from_slots();
    rotate_v_offsets();  // V of tile 1 leaves in iteration 0
#pragma unroll
    for (int n = UPW; n < 2 * UPW; ++n) move(n, kKStage, 0);  // K of tile 1
    slot_load(k_lo + 2 * kBN);
    wait_all_vm();
    __syncthreads();
    // byte offsets of the stages: K of tiles j, j+1 and the one being filled; V of tiles
    // j-1, j and the one being filled (the first P is zero, so "tile -1" may alias tile 0)
    uint32_t k_cur = 0, k_next = kKStage, k_fill = 2 * kKStage;
    uint32_t v_prev = kVBase, v_cur = kVBase, v_fill = kVBase + kVStage, v_spare = kVBase + 2 * kVStage;
    if (idle) {
      // the same moves, waits and barriers as the computing waves, tile by tile
      for (int j = 0; j < n_tiles; ++j) {
        offsets_from_slots();
        slot_load(k_lo + (j + 3) * kBN);
#pragma unroll
        for (int n = 0; n < 2 * UPW; ++n) move(n, k_fill, v_fill);
        rotate_v_offsets();
        wait_all_vm();
        __syncthreads();
        const uint32_t k_freed = k_cur;
        k_cur = k_next;
        k_next = k_fill;
        k_fill = k_freed;
        const uint32_t v_freed = (j == 0) ? v_spare : v_prev;
        v_prev = v_cur;
        v_cur = v_fill;
        v_fill = v_freed;
      }
    } else {
      Scores sa, sb;
      Stats st_a, st_b;
      bf16x8_t pb_a[RT][2], pb_b[RT][2];
      qk_half(0, 0, sa);
      st_a.mul = p.scale_log2e;
      if (needs_mask(k_lo)) {
        mask_in_place(sa, k_lo);
        st_a.mul = 1.0f;
      }
      {
        float mx[RT];
        lane_max(sa, mx);
        decide(mx, st_a);
      }
      st_b.mul = 1.0f;
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) {
        st_b.alpha[rt] = 1.0f;
        st_b.m_safe[rt] = 0.f;
#pragma unroll
        for (int u = 0; u < 2; ++u) pb_b[rt][u] = as_bf16x8(u32x4_t{0u, 0u, 0u, 0u});
      }
      bf16x8_t kops[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) kops[e] = k_operand(smem + k_cur + k_lane + 512, e);
      for (int j = 0; j < n_tiles; ++j) {
        const int tb = k_lo + j * kBN;
        // the moves of this iteration (V of tile j+1, K of tile j+2) are issued one per slice
        // of the first half, between its MFMAs; the slot ids of tile j+3 are requested now and
        // used in the next iteration
        offsets_from_slots();
        slot_load(tb + 3 * kBN);
        // half (j,0): scores of (j,1) from K of tile j, P V of (j-1,1) from V of tile j-1
        rescale(st_b.alpha);
        fused_half(sa, st_a, sb, st_b, needs_mask(tb + 32), tb + 32, smem + k_cur + k_lane + 512,
                   smem + v_prev + v_lane + 512, smem + k_next + k_lane, kops, pb_b, pb_a,
                   [&](int sl) {
                     constexpr int PER = 2 * UPW / 4;
#pragma unroll
                     for (int n = sl * PER; n < (sl + 1) * PER; ++n) move(n, k_fill, v_fill);
                   });
        rotate_v_offsets();
        // half (j,1): scores of (j+1,0) from K of tile j+1, P V of (j,0) from V of tile j
        rescale(st_a.alpha);
        fused_half(sb, st_b, sa, st_a, needs_mask(tb + 64), tb + 64, smem + k_next + k_lane,
                   smem + v_cur + v_lane, smem + k_next + k_lane + 512, kops, pb_a, pb_b, [](int) {});
        wait_all_vm();
        __syncthreads();
        const uint32_t k_freed = k_cur;
        k_cur = k_next;
        k_next = k_fill;
        k_fill = k_freed;
        const uint32_t v_freed = (j == 0) ? v_spare : v_prev;
        v_prev = v_cur;
        v_cur = v_fill;
        v_fill = v_freed;
      }
      // the last half's P V is still owed
      rescale(st_b.alpha);
      pv_half(v_prev, 1, pb_b);
    }
    __syncthreads();  // the epilogue reuses the stages as its output staging area
  }

  // accumulator i of O^T tile dt is dim 32dt + 8(i/4) + 4h + i%4 of query row c32
  if (p.n_ksplit > 1) {
    // ---- key split: normalised fp32 partial and log-sum-exp (base 2) per row, from registers
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
      float l = l_run[rt];
      l += __shfl_xor(l, 32, kWave);
      const float inv = (l > 0.f) ? 1.0f / l : 0.f;
      const int row = row0 + (w * RT + rt) * 32 + c32;
      if (row < rows_total) {
        const int qi = row / p.group;
        const int hh = row - qi * p.group;
        const int64_t at = (int64_t)split * p.part_rows + (int64_t)(q_start + qi) * p.n_q + kvh * p.group + hh;
        if (h == 0) p.part_lse[at] = (l > 0.f) ? m_run[rt] + __log2f(l) : kNegInf;
        float* dst = p.part_o + at * D + 4 * h;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
          for (int a = 0; a < 4; ++a) {
            f32x4_t v = {oacc[dt][rt][4 * a] * inv, oacc[dt][rt][4 * a + 1] * inv,
                         oacc[dt][rt][4 * a + 2] * inv, oacc[dt][rt][4 * a + 3] * inv};
            *reinterpret_cast<f32x4_t*>(dst + 32 * dt + 8 * a) = v;
          }
      }
    }
    return;
  }
  // ---- epilogue: normalise, transpose through LDS, store whole rows ---------------------
  unsigned char* os = smem;
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    float l = l_run[rt];
    l += __shfl_xor(l, 32, kWave);
    const float inv = (l > 0.f) ? 1.0f / l : 0.f;
    const int lrow = (w * RT + rt) * 32 + c32;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int a = 0; a < 4; ++a) {
        u32x2_t wv;
        wv[0] = pack_bf16x2(oacc[dt][rt][4 * a] * inv, oacc[dt][rt][4 * a + 1] * inv);
        wv[1] = pack_bf16x2(oacc[dt][rt][4 * a + 2] * inv, oacc[dt][rt][4 * a + 3] * inv);
        *reinterpret_cast<u32x2_t*>(os + (lrow * OROW + 32 * dt + 8 * a + 4 * h) * 2) = wv;
      }
  }
  __syncthreads();
  constexpr int ROWS_PER_PASS = NW * 4;
  const int c = tid & 15;
#pragma unroll 4
  for (int pass = 0; pass < kRows / ROWS_PER_PASS; ++pass) {
    const int lrow = pass * ROWS_PER_PASS + (tid >> 4);
    const int row = row0 + lrow;
    if (row < rows_total) {
      const int qi = row / p.group;
      const int hh = row - qi * p.group;
      const u32x4_t v = *reinterpret_cast<const u32x4_t*>(os + (lrow * OROW + c * 8) * 2);
      st_global_b128(p.out + ((int64_t)(q_start + qi) * p.n_q + kvh * p.group + hh) * D + c * 8, v);
    }
  }
}


// =============================================================================================
// Ping-pong variant of the tile kernel (same tiling, same LDS layout, same data path).
//
// The two waves that share a SIMD (w and w + 4) never do the same kind of work at the same
// time.  Time is cut into slots separated by workgroup barriers; in every slot the waves of one
// group (w < 4, one per SIMD) run an M phase, nothing but MFMAs and their LDS operand reads:
//     O^T += V(j)^T P(j)^T,   S(j+1)^T = K(j+1) Q^T            (32 MFMAs, a whole 64-key tile)
// while the waves of the other group run a V phase, nothing but VALU and the tile moves:
//     P(j+1) = softmax step of S(j+1)  (row max, lazy rescale, exp2, bf16 pack, row sum)
// and then they swap.  The matrix pipe of a SIMD therefore always has exactly one wave feeding
// it, and that wave's softmax never competes with its own or its partner's MFMAs for issue
// slots in the same phase of the instruction stream.
//
//   slot      0       1       2       3       4      ...
//   w < 4   M(-1)   V(-1)   M(0)    V(0)    M(1)           M(-1): scores of tile 0 only
//   w >= 4   -      M(-1)   V(-1)   M(0)    V(0)
//
// Tiles: K(t) and V(t) live in stage t % 4 of four K and four V stages.  M phase j, whose wave
// has issue slots to spare between its MFMAs, also sends K(j+4) and V(j+2) on their way (each
// wave its two units of each) and, before the barrier that ends its slot, waits for what it sent
// in M phase j-1: a tile is in flight for two slots and has been published by a barrier before
// its first reader asks for operands.  A stage is refilled only after a barrier that every
// reader of its previous tile has passed with its reads done: K(j) is read by the score slices
// of M phase j-1, which precede that phase's barrier, and V(j-2) by M phase j-2, two phases back
// (an M phase passes its barrier before its last P V slices, so "one phase back" would not do).
// The slot ids of a tile travel through a small LDS ring of the wave's own (one dword
// LDS-direct load per tile, two M phases ahead; read back into registers at the barrier of the
// M phase before the one that uses them), which keeps every vector-memory operation of the loop
// out of the compiler's wait bookkeeping: the only vector-memory wait in the loop is the counted
// one before an M phase's barrier.  Order of issue inside an M phase: [ring fetch, 4 moves].
#ifndef MSGL_PP_PRIO_M
#define MSGL_PP_PRIO_M 3
#endif
#ifndef MSGL_PP_PRIO_V
#define MSGL_PP_PRIO_V 0
#endif
namespace pp {
constexpr int kStages = 4;
constexpr int kVBase = kStages * kKStage;
constexpr int kRingBase = kVBase + kStages * kVStage;
constexpr int kRingStage = 256;  // one dword per lane
constexpr int kRingStages = 4;
constexpr int kRingWave = kRingStages * kRingStage;
constexpr int kSmem = kRingBase + 8 * kRingWave;
// LDS operands of a slice of four MFMAs are requested this many slices ahead (two measured no
// faster than one and costs 16 more registers)
#ifndef MSGL_PP_AHEAD
#define MSGL_PP_AHEAD 1
#endif
constexpr int kAhead = MSGL_PP_AHEAD;
// An M phase passes the barrier that ends its slot this many slices before its last one: the
// partner wave needs a few hundred cycles from the barrier to its first MFMA, and the matrix
// pipe would idle for them.
#ifndef MSGL_PP_HANDOFF
#define MSGL_PP_HANDOFF 1
#endif
constexpr int kHandoff = MSGL_PP_HANDOFF;
static_assert(kHandoff >= 0 && kHandoff <= 2, "the sends of a phase must have left before its barrier");
constexpr int kOperandBuffers = kAhead + 1;
}  // namespace pp

template <bool WIDE>
__global__ __launch_bounds__(512) void prefill_pingpong_kernel(PrefillParams p) {
  constexpr int D = 128, NW = 8, UPW = kUnits / NW, KSTEPS = D / 16, DT = D / 32;
  constexpr int kRows = NW * 32;
  constexpr int OROW = D + 8;
  static_assert(kRows * OROW * 2 <= pp::kSmem, "output staging must fit the stages");
  __shared__ __attribute__((aligned(16))) unsigned char smem[pp::kSmem];
  using OffT = typename std::conditional<WIDE, uint64_t, uint32_t>::type;
  const ClockProbe clock_probe_(p.clock_probe);

  const int tid = threadIdx.x;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63;
  const int h = lane >> 5;
  const int c32 = lane & 31;

  // ---- gang ranges: the workgroup stays for the launch and takes the parts of the units that
  // fall into its gang's range, one after the other (see gang_plan) -----------------------------
  __shared__ GangLds gang_lds;
  __shared__ int gang_last;
  const bool ganged = p.gangs > 0;
  const int gang_xcd = (int)(blockIdx.x & 7);
  const int gang_id = ganged ? (int)(blockIdx.x >> 3) / p.n_qblk : 0;
  const int gang_member = ganged ? (int)(blockIdx.x >> 3) % p.n_qblk : 0;
  GangPlan plan{0, 0, 0, 0};
  if (ganged) plan = gang_plan<NW * 64>(p, gang_lds, gang_xcd, gang_id, gang_member, kRows, tid);
  for (int piece = plan.first_unit;; ++piece) {
  // ---- block -> (request, kv head, key split, q block): as in prefill_tile_kernel; with ragged
  // shares, block -> (unit = (request, share), kv head); with gang ranges, the next unit of the
  // range -------------------------------------------------------------------------------------
  int b, kvh, split = 0, qblk, n_shares = 1;
  bool to_partial = p.n_ksplit > 1;  // leave a partial for the merge kernel, not the result
  int64_t part_at = 0;               // partial row of the block's row 0 (ragged shares)
  int piece_a = 0, piece_b = 0x7fffff, unit_start = 0, unit_tiles = 0;  // gang ranges: tiles [a, b) of the unit
  bool piece_whole = true;
  if (ganged) {
    if (piece > plan.last_unit) break;
    // the stages double as the staging area of the previous part's output: read out by now
    if (piece > plan.first_unit) __syncthreads();
    unit_tiles = __builtin_amdgcn_readfirstlane(gang_lds.len[piece]);
    unit_start = __builtin_amdgcn_readfirstlane(gang_lds.start[piece]);
    piece_a = max(plan.lo - unit_start, 0);
    piece_b = min(plan.hi - unit_start, unit_tiles);
    if (piece_b <= piece_a) continue;
    piece_whole = piece_a == 0 && piece_b == unit_tiles;
    const int unit = piece * 8 + gang_xcd;
    b = __builtin_amdgcn_readfirstlane(gang_lds.order[unit / p.n_kv]);
    kvh = unit % p.n_kv;
    qblk = gang_member;
    to_partial = false;
  } else if (piece > 0) {
    break;
  } else if (p.ragged_tiles > 0) {
    kvh = (int)(blockIdx.x % (unsigned)p.n_kv);
    const int u = (int)(blockIdx.x / (unsigned)p.n_kv);
    const RaggedUnit ru = ragged_unit<NW * 64>(p, u, tid);
    if (!ru.ok) return;
    b = ru.request;
    split = ru.share;
    qblk = 0;
    n_shares = ru.count;
    to_partial = ru.count > 1;
    part_at = ((int64_t)u * p.n_kv + kvh) * p.ragged_rows;
    if (ru.share == 0 && kvh == 0 && tid == 0 && p.req_units != nullptr) {
      p.req_units[2 * b] = ru.first;  // tells the merge kernel where the request's partials are
      p.req_units[2 * b + 1] = ru.count;
    }
  } else {
    const BlockWork work = prefill_block_work(p);
    if (!work.ok) return;
    const int pair = work.unit / p.n_ksplit;  // unit = (request, kv head, key split)
    split = work.unit - pair * p.n_ksplit;
    qblk = work.qblk;
    const int want_rank = pair / p.n_kv;
    kvh = pair - want_rank * p.n_kv;
    b = request_of_rank<NW * 64>(p.kv_indptr, p.batch, want_rank, tid);
  }

  // (gang ranges keep every request's geometry in LDS: a part starts without a memory round trip)
  auto uniform = [](int x) { return __builtin_amdgcn_readfirstlane(x); };  // the same in every lane: a scalar
  const int q_start = ganged ? uniform(gang_lds.q_start[b]) : p.qo_indptr[b];
  const int q_len = ganged ? uniform(gang_lds.q_len[b]) : min(p.qo_indptr[b + 1] - q_start, p.max_len_extend);
  const int kv_start = ganged ? uniform(gang_lds.kv_start[b]) : p.kv_indptr[b];
  const int kn = ganged ? uniform(gang_lds.kv_len[b]) : max(p.kv_indptr[b + 1] - kv_start, 0);
  const int prefix = ganged ? uniform(gang_lds.prefix[b]) : p.prefix_lens[b];
  const int rows_total = q_len * p.group;
  const int row0 = qblk * kRows;
  if (row0 >= rows_total) {
    if (ganged) continue;  // this request has no such query block
    return;
  }

  const bool idle = __builtin_amdgcn_readfirstlane(row0 + w * 32 >= rows_total ? 1 : 0) != 0;
  const int qi_lo = row0 / p.group;
  const int qi_hi = min(rows_total - 1, row0 + kRows - 1) / p.group;
  int k_hi = p.is_cross ? kn : min(kn, prefix + qi_hi + 1);
  int k_lo = (p.window > 0) ? max(0, prefix + qi_lo - p.window + 1) : 0;
  k_lo &= ~(kBN - 1);
  if (k_hi < k_lo) k_hi = k_lo;
  if (ganged) {  // tiles [piece_a, piece_b) of the unit, as far as this query block sees them
    k_lo = min(k_lo + piece_a * kBN, k_hi);
    k_hi = min(k_hi, piece_b * kBN);
    if (k_hi < k_lo) k_hi = k_lo;
  } else if (p.ragged_tiles > 0) {  // the request's shares are equal: none longer than ragged_tiles
    const int all_tiles = (k_hi - k_lo + kBN - 1) / kBN;
    const int share = (all_tiles + n_shares - 1) / n_shares * kBN;
    k_lo = min(k_lo + split * share, k_hi);
    k_hi = min(k_hi, k_lo + share);
  } else if (p.n_ksplit > 1) {
    const int all_tiles = (k_hi - k_lo + kBN - 1) / kBN;
    const int share = (all_tiles + p.n_ksplit - 1) / p.n_ksplit * kBN;
    k_lo = min(k_lo + split * share, k_hi);
    k_hi = min(k_hi, k_lo + share);
  }
  const int n_tiles = (k_hi - k_lo + kBN - 1) / kBN;

  // ---- this lane's row: Q operand, visibility bounds ---------------------------------------
  // (the Q rows themselves are requested in the prologue, after the first tiles' slot ids: the
  // ids gate the first tile moves, and a wait for them would otherwise wait for the Q rows too)
  bf16x8_t qreg[KSTEPS];
  bool q_valid;
  int64_t q_off;
  int row_lo, row_hi;
  int w_lo_max = -0x7fffffff, w_hi_min = 0x7fffffff;
  {
    const int row = row0 + w * 32 + c32;
    const bool valid = row < rows_total;
    const int qi = valid ? row / p.group : 0;
    const int hh = valid ? row - qi * p.group : 0;
    q_valid = valid;
    q_off = ((int64_t)(q_start + qi) * p.n_q + kvh * p.group + hh) * D;
    const int qpos = prefix + qi;
    int lo = (p.window > 0) ? qpos - p.window + 1 : 0;
    int hi = min(p.is_cross ? kn - 1 : min(qpos, kn - 1), k_hi - 1);
    if (valid) {
      w_lo_max = lo;
      w_hi_min = hi;
    } else {
      lo = 1;
      hi = 0;
    }
    row_lo = lo;
    row_hi = hi;
  }
#pragma unroll
  for (int off = 1; off < kWave; off <<= 1) {
    w_lo_max = max(w_lo_max, __shfl_xor(w_lo_max, off, kWave));
    w_hi_min = min(w_hi_min, __shfl_xor(w_hi_min, off, kWave));
  }
  w_lo_max = __builtin_amdgcn_readfirstlane(w_lo_max);
  w_hi_min = __builtin_amdgcn_readfirstlane(w_hi_min);

  f32x16_t oacc[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int i = 0; i < 16; ++i) oacc[dt][i] = 0.f;
  float m_run = kNegInf, l_run = 0.f, m_safe_run = 0.f;

  // ---- moving tiles -------------------------------------------------------------------------
  const uint32_t lds0 = (uint32_t)(uintptr_t)MSGL_LDS_PTR(unsigned char, smem);
  const int32_t* idx_base = p.kv_indices + kv_start;
  const unsigned char* k_src = reinterpret_cast<const unsigned char*>(p.k_cache + (int64_t)kvh * D);
  const unsigned char* v_src = reinterpret_cast<const unsigned char*>(p.v_cache + (int64_t)kvh * D);
  const uint32_t k_row_bytes = (uint32_t)p.k_stride0 * 2u;
  const uint32_t v_row_bytes = (uint32_t)p.v_stride0 * 2u;
  const uint32_t chunk_off = (uint32_t)(lane & 15) * 16u;
  const int unit_key = w * UPW + 16 * (lane >> 4);  // + i for unit i of this wave
  auto row_offset = [&](uint32_t slot_id, uint32_t row_bytes) -> OffT {
    if constexpr (WIDE) return (uint64_t)slot_id * row_bytes + chunk_off;
    else return __umul24(slot_id, row_bytes) + chunk_off;  // both below 2^24 here
  };
  // ring entry e of a wave = slot id of key (w UPW + e % UPW + 16 (e / UPW)) of the tile,
  // e = 0 .. 4 UPW - 1; lanes past that repeat the entries
  const uint32_t ring0 = (uint32_t)pp::kRingBase + (uint32_t)w * pp::kRingWave;
  const int ring_key = w * UPW + (lane % UPW) + 16 * ((lane / UPW) & 3);
  auto ring_fetch = [&](int t) {  // tile t of this block
    const uint32_t off = (uint32_t)min(k_lo + t * kBN + ring_key, kn - 1) * 4u;
    lds_direct_b32(lds0 + ring0 + (uint32_t)(t & (pp::kRingStages - 1)) * pp::kRingStage, idx_base, off);
  };
  auto ring_read = [&](int t, uint32_t (&ids)[UPW]) {
    // read through an LDS pointer: a volatile read through a generic one would be a flat load,
    // which waits for every vector-memory operation in flight
    const volatile __attribute__((address_space(3))) uint32_t* r = MSGL_LDS_PTR(
        const volatile uint32_t, smem + ring0 + (t & (pp::kRingStages - 1)) * pp::kRingStage + (lane >> 4) * (4 * UPW));
#pragma unroll
    for (int i = 0; i < UPW; ++i) ids[i] = min(r[i], p.max_slot);
  };
  uint32_t ids[UPW];  // slot ids of the tile whose K leaves in the next M phase
  OffT v_off[UPW];       // V row offsets of the tile whose V leaves in the next M phase
  OffT v_off_then[UPW];  // ... and of the tile whose V leaves in the one after
  auto k_stage_of = [](int t) { return (uint32_t)(t & 3) * kKStage; };
  auto v_stage_of = [](int t) { return (uint32_t)pp::kVBase + (uint32_t)(t & 3) * kVStage; };
  // The vector-memory part of M phase j in three pieces that ride along with its first slices:
  // ids of tile j+6 requested; V(j+2) sent; K(j+4) sent and the V offsets of tile j+4 kept.
  auto send_tiles = [&](int j, int piece) {
    if (piece == 0) {
      ring_fetch(j + 6);
    } else if (piece == 1) {
#pragma unroll
      for (int i = 0; i < UPW; ++i)
        lds_direct_b128(lds0 + v_stage_of(j + 2) + (uint32_t)(w * UPW + i) * kVUnit, v_src, v_off[i]);
    } else {
#pragma unroll
      for (int i = 0; i < UPW; ++i)
        lds_direct_b128(lds0 + k_stage_of(j + 4) + (uint32_t)(w * UPW + i) * kKUnit, k_src,
                        row_offset(ids[i], k_row_bytes));
#pragma unroll
      for (int i = 0; i < UPW; ++i) {
        v_off[i] = v_off_then[i];
        v_off_then[i] = row_offset(ids[i], v_row_bytes);
      }
    }
  };
  // end of M phase j: everything older than this phase's own ring fetch and moves has landed,
  // among it the ring entries of tile j+5, which the next M phase turns into addresses
  auto end_of_sends = [&](int j) {
    wait_vm_at_most<2 * UPW + 1>();
    ring_read(j + 5, ids);
  };
  auto slot_barrier = [&]() {
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
  };

  // per-lane LDS read offsets inside a stage (see prefill_tile_kernel)
  const uint32_t k_lane = (uint32_t)(c32 & 15) * kKUnit + (uint32_t)(c32 >> 4) * 256u + (uint32_t)h * 16u;
  const uint32_t v_lane = (uint32_t)(4 * h + ((lane & 15) >> 2)) * kVUnit +
                          (uint32_t)((lane >> 4) & 1) * 32u + (uint32_t)(lane & 3) * 8u;

  // S^T of one tile: s[kt][i] is key 32 kt + 8 (i / 4) + 4 h + i % 4, row c32
  f32x16_t s[2];
  bf16x8_t pb[2][2];  // P^T operands: [half][16 keys]
  auto k_ops = [&](const unsigned char* ks, int kt, int first, bf16x8_t (&ops)[4]) {
#pragma unroll
    for (int e = 0; e < 4; ++e)
      ops[e] = as_bf16x8(*reinterpret_cast<const u32x4_t*>(ks + kt * 512 + (first + e) * 32));
  };
  auto v_ops = [&](const unsigned char* vs, int kt, int u, bf16x8_t (&ops)[4]) {
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      const u32x2_t lo = lds_read_tr16(vs + kt * 512 + u * 256 + dt * 64);
      const u32x2_t hi = lds_read_tr16(vs + kt * 512 + u * 256 + dt * 64 + 8 * kVUnit);
      ops[dt] = as_bf16x8(u32x4_t{lo[0], lo[1], hi[0], hi[1]});
    }
  };
  auto pv4 = [&](const bf16x8_t& pw, const bf16x8_t (&ops)[4]) {
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) oacc[dt] = mfma_32x32x16(ops[dt], pw, oacc[dt]);
  };
  auto qk4 = [&](int kt, int first, const bf16x8_t (&ops)[4]) {
#pragma unroll
    for (int e = 0; e < 4; ++e) s[kt] = mfma_32x32x16(ops[e], qreg[first + e], s[kt]);
  };
  auto zero_scores = [&]() {
#pragma unroll
    for (int kt = 0; kt < 2; ++kt)
#pragma unroll
      for (int i = 0; i < 16; ++i) s[kt][i] = 0.f;
  };
  // Lane maximum of half kt of the scores, as two independent chains (a single chain would pay
  // the full VALU latency per link: the partner wave issues no VALU work to fill the gaps).
  auto half_max = [&](int kt) {
    const f32x16_t& x = s[kt];
    float m2[2];
#pragma unroll
    for (int c = 0; c < 2; ++c) {
      const int o = 8 * c;
      float t = fmaxf(fmaxf(x[o], x[o + 1]), x[o + 2]);
      t = fmaxf(fmaxf(t, x[o + 3]), x[o + 4]);
      t = fmaxf(fmaxf(t, x[o + 5]), x[o + 6]);
      m2[c] = fmaxf(t, x[o + 7]);
    }
    return fmaxf(m2[0], m2[1]);
  };
  // M phase j: first the scores of tile j+1, then P V of tile j.  Eight slices of four MFMAs; the
  // operands of a slice are requested kAhead slices ahead into one of kAhead + 1 operand
  // buffers, those of the first slice(s) before the barrier (in the first and the last phase: at
  // its start).  The tile sends ride along with the first three slices; the barrier that ends
  // the phase's slot comes kHandoff slices before the end.  Nothing else rides along: the wave's
  // issue slots between MFMAs are taken by the LDS requests and their waits (measured: with the
  // row maxima computed here instead of in the V phase the kernel is 2 % slower).
  auto m_phase = [&](int j, bf16x8_t (&o)[pp::kOperandBuffers][4], auto with_pv, auto with_qk) {
    constexpr bool PV = decltype(with_pv)::value, QK = decltype(with_qk)::value;
    constexpr int NS = 4 * ((PV ? 1 : 0) + (QK ? 1 : 0));  // slices of four MFMAs
    __builtin_amdgcn_s_setprio(MSGL_PP_PRIO_M);
    const unsigned char* ks = smem + k_stage_of(j + 1) + k_lane;
    const unsigned char* vs = smem + v_stage_of(j) + v_lane;
    // Slice i is a score slice (half t / 2, k-steps 4 (t % 2) ..) or a P V slice (half t / 2, keys
    // 16 (t % 2) ..), t = i % 4; a full phase runs its four score slices first.  (Alternating the
    // two kinds, which spreads the transposing V reads over the phase, measured 2-5 % slower.)
    auto request = [&](auto ic) {
      constexpr int i = decltype(ic)::value;
      if constexpr (i < NS) {
        constexpr bool is_qk = QK && (!PV || i < 4);
        constexpr int t = i % 4;
        if constexpr (is_qk) k_ops(ks, t >> 1, (t & 1) * 4, o[i % pp::kOperandBuffers]);
        else v_ops(vs, t >> 1, t & 1, o[i % pp::kOperandBuffers]);
      }
    };
    auto slice = [&](auto ic) {
      constexpr int i = decltype(ic)::value;
      constexpr bool is_qk = QK && (!PV || i < 4);
      constexpr int t = i % 4;
      if constexpr (QK && pp::kHandoff > 0 && i == NS - pp::kHandoff) {
        end_of_sends(j);
        slot_barrier();
      }
      request(std::integral_constant<int, i + pp::kAhead>{});
      if constexpr (is_qk) qk4(t >> 1, (t & 1) * 4, o[i % pp::kOperandBuffers]);
      else pv4(pb[t >> 1][t & 1], o[i % pp::kOperandBuffers]);
      if constexpr (QK) {  // the sends: all of them before the barrier
        if constexpr (NS == 8) {
          if constexpr (i < 3) send_tiles(j, i);
        } else {
          if constexpr (i == 0) { send_tiles(j, 0); send_tiles(j, 1); }
          if constexpr (i == 1) send_tiles(j, 2);
        }
      }
      // the LDS requests first, then the MFMAs and whatever rides along
      if constexpr (i + pp::kAhead < NS) {
        constexpr int i2 = i + pp::kAhead;
        constexpr bool next_qk = QK && (!PV || i2 < 4);
        if constexpr (next_qk) __builtin_amdgcn_sched_group_barrier(0x100, 4, 0);
        else __builtin_amdgcn_sched_group_barrier(0x100, 8, 0);
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
    };
    // Slice 0's operands were requested before the barrier in a full phase (the V tile may only
    // just have been published, so nothing of it is asked for ahead of the barrier).
    if constexpr (!(QK && PV)) request(std::integral_constant<int, 0>{});
    if constexpr (pp::kAhead > 1) request(std::integral_constant<int, 1>{});
    if constexpr (QK) zero_scores();
    slice(std::integral_constant<int, 0>{});
    slice(std::integral_constant<int, 1>{});
    slice(std::integral_constant<int, 2>{});
    slice(std::integral_constant<int, 3>{});
    if constexpr (NS == 8) {
      slice(std::integral_constant<int, 4>{});
      slice(std::integral_constant<int, 5>{});
      slice(std::integral_constant<int, 6>{});
      slice(std::integral_constant<int, 7>{});
    }
    if constexpr (QK && pp::kHandoff == 0) {
      end_of_sends(j);
      slot_barrier();
    }
    __builtin_amdgcn_s_setprio(MSGL_PP_PRIO_V);
  };
  using Yes = std::true_type;
  using No = std::false_type;

  const bool general_scale = p.scale_log2e <= 0.f;  // the fast path needs a positive scale
  // P of one tile from its scores: exp2(s * mul - m_safe), cut to bf16 (the upper halves of two
  // fp32 values side by side, one v_perm_b32: truncation; the row sum below is taken from the
  // same cut values, so the half step they all lose on average cancels in O / l, and what is
  // left is an error as wide as that of rounding to nearest).  Returns the lane's sum of them.
  auto exp_pack = [&](float mul, float m_safe) {
    float psum[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int kt = 0; kt < 2; ++kt)
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        u32x4_t pk;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const float e0 = fast_exp2(__builtin_fmaf(s[kt][8 * u + 2 * e], mul, -m_safe));
          const float e1 = fast_exp2(__builtin_fmaf(s[kt][8 * u + 2 * e + 1], mul, -m_safe));
          const uint32_t pw = pack_hi16(__builtin_bit_cast(uint32_t, e0), __builtin_bit_cast(uint32_t, e1));
          pk[e] = pw;
          psum[e] = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, pw), kOnes, psum[e], false);
        }
        pb[kt][u] = as_bf16x8(pk);
      }
    return (psum[0] + psum[1]) + (psum[2] + psum[3]);
  };
  // V phase j: P(j+1) from S(j+1), then the first operands of M phase j+1
  auto v_phase = [&](int j, bf16x8_t (&o)[pp::kOperandBuffers][4]) {
    // First of all the operands of the first slice of M phase j+1 (its scores', if it computes
    // any) are requested: they arrive while the VALU works, and that phase's first MFMA finds
    // them there.  (The last phase, P V only, asks for its operands itself: the V tile it reads
    // may only have been published by the barrier that precedes it.)
    if (j + 2 < n_tiles) k_ops(smem + k_stage_of(j + 2) + k_lane, 0, 0, o[0]);
    __builtin_amdgcn_sched_barrier(0);
    const int base = k_lo + (j + 1) * kBN;
    const bool boundary = general_scale || base < w_lo_max || base + kBN - 1 > w_hi_min;
    {
      float mul = p.scale_log2e;
      if (boundary) {
        // boundary tile: scale and mask in place.  The empty volatile statement keeps this a
        // branch: as selects it would put 100 more VALU instructions into every tile.
        asm volatile("" ::: "memory");
#pragma unroll
        for (int kt = 0; kt < 2; ++kt)
#pragma unroll
          for (int i = 0; i < 16; ++i) {
            const int key = base + 32 * kt + 8 * (i >> 2) + 4 * h + (i & 3);
            const float x = s[kt][i] * p.scale_log2e;
            s[kt][i] = (key < row_lo || key > row_hi) ? kNegInf : x;
          }
        mul = 1.0f;
      }
      const float mx = fmaxf(half_max(0), half_max(1));
      float m_safe = m_safe_run, alpha = 1.0f;
      // Has some lane seen a score more than kLazy above its row's reference?  If not, no row's
      // reference moves (both halves of a row sit in this wave).  Otherwise the cross-lane
      // exchange, the new state and, where a reference did move, the rescaling of O.
      if (__any(mx * mul > m_run + kLazy)) {
        const float m = wave_max_xor(mx * mul, 32);
        const float m_old = m_run;
        const float m_new = fmaxf(m_old, m);
        const float m_use = (m_new - m_old > kLazy) ? m_new : m_old;
        m_safe = (m_use == kNegInf) ? 0.f : m_use;
        m_safe_run = m_safe;
        alpha = fast_exp2(m_old - m_safe);
        m_run = m_use;
        if (__any(alpha != 1.0f)) {
#pragma unroll
          for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int i = 0; i < 16; ++i) oacc[dt][i] *= alpha;
        }
      }
      l_run = l_run * alpha + exp_pack(mul, m_safe);
    }
  };

  if (n_tiles > 0) {
    // ---- prologue: K(0..2) and V(0) leave and are waited for; the ring holds tiles 3, 4 ------
    {
      uint32_t first[3][UPW];
#pragma unroll
      for (int t = 0; t < 3; ++t)
#pragma unroll
        for (int i = 0; i < UPW; ++i)
          first[t][i] = min((uint32_t)idx_base[min(k_lo + t * kBN + unit_key + i, kn - 1)], p.max_slot);
#pragma unroll
      for (int ks = 0; ks < KSTEPS; ++ks) {
        u32x4_t raw = {0u, 0u, 0u, 0u};
        if (q_valid) raw = ld_global_b128(p.q + q_off + ks * 16 + h * 8);
        qreg[ks] = as_bf16x8(raw);
      }
      ring_fetch(3);
      ring_fetch(4);
#pragma unroll
      for (int t = 0; t < 3; ++t) {
#pragma unroll
        for (int i = 0; i < UPW; ++i) {
          const OffT vo = row_offset(first[t][i], v_row_bytes);
          lds_direct_b128(lds0 + k_stage_of(t) + (uint32_t)(w * UPW + i) * kKUnit, k_src,
                          row_offset(first[t][i], k_row_bytes));
          if (t == 0) lds_direct_b128(lds0 + v_stage_of(t) + (uint32_t)(w * UPW + i) * kVUnit, v_src, vo);
          if (t == 1) v_off[i] = vo;       // leaves in M phase -1
          if (t == 2) v_off_then[i] = vo;  // leaves in M phase 0
        }
      }
    }
    wait_all_vm();
    ring_read(3, ids);
    __syncthreads();
    const bool second = w >= 4;  // the group that runs one slot behind
    if (idle) {
      // the moves, waits and barriers of a computing wave of the same group, nothing else
      if (second) slot_barrier();
      for (int j = -1; j < n_tiles - 1; ++j) {
#pragma unroll
        for (int piece = 0; piece < 3; ++piece) send_tiles(j, piece);
        end_of_sends(j);
        slot_barrier();
        slot_barrier();
      }
      wait_all_vm();
      slot_barrier();
      if (!second) slot_barrier();
    } else {
      bf16x8_t oa[pp::kOperandBuffers][4];
      if (second) slot_barrier();
      m_phase(-1, oa, No{}, Yes{});  // with its barrier
      v_phase(-1, oa);
      slot_barrier();
      for (int j = 0; j < n_tiles - 1; ++j) {
        m_phase(j, oa, Yes{}, Yes{});  // with its barrier
        v_phase(j, oa);
        slot_barrier();
      }
      m_phase(n_tiles - 1, oa, Yes{}, No{});
      wait_all_vm();
      slot_barrier();
      if (!second) slot_barrier();
    }
    // every wave has passed its last read of the stages and every move has landed: the
    // epilogue reuses the stages as its output staging area
  }

  // ---- gang ranges: a part of a unit.  Its unnormalised rows, row references and row sums go to
  // the part's slot (lane-major: the only reader has this kernel's register layout), the workgroup
  // counts itself, and the part that counts last adds the others to its registers and goes on to
  // write the result.  Slots and counts are read and written at agent scope (parts of a unit
  // may sit on different XCDs as far as the program is concerned; nothing here relies on the
  // order in which the parts finish, and nobody waits for anybody).
  if (ganged && !piece_whole) {
    auto slot_of = [&](int g) {
      const int64_t at = (((int64_t)gang_xcd * p.gangs + g) * 2 + gang_slot_of(gang_lds, g, unit_start)) * p.n_qblk + gang_member;
      return reinterpret_cast<unsigned long long*>(p.gang_slots) + at * (int64_t)(kGangSlotBytes / 8);
    };
    auto pair_bits = [](float x, float y) {
      return (unsigned long long)__builtin_bit_cast(uint32_t, x) | ((unsigned long long)__builtin_bit_cast(uint32_t, y) << 32);
    };
    {
      unsigned long long* mine = slot_of(gang_id);
      unsigned long long* o64 = mine + (int64_t)w * 32 * kWave + lane;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int i = 0; i < 16; i += 2)
          __hip_atomic_store(o64 + (dt * 8 + i / 2) * kWave, pair_bits(oacc[dt][i], oacc[dt][i + 1]), __ATOMIC_RELAXED,
                             __HIP_MEMORY_SCOPE_AGENT);
      __hip_atomic_store(mine + 8 * 32 * kWave + w * kWave + lane, pair_bits(m_run, l_run), __ATOMIC_RELAXED,
                         __HIP_MEMORY_SCOPE_AGENT);
    }
    // count word = launch number << 16 | parts done; a word from another launch counts as zero.
    // It is read while the slot's stores drain (the update below then usually succeeds at once).
    unsigned long long* cnt = p.gang_counts + ((int64_t)(piece * 8 + gang_xcd) * p.n_qblk + gang_member);
    unsigned long long seen = 0;
    if (tid == 0) seen = __hip_atomic_load(cnt, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    wait_all_vm();  // the slot is written before the workgroup counts itself
    __syncthreads();
    if (tid == 0) {
      int n_parts = 0;
      for (int g = 0; g < p.gangs; ++g)
        n_parts += (gang_lds.cuts[g] < unit_start + unit_tiles && gang_lds.cuts[g + 1] > unit_start &&
                    gang_lds.cuts[g + 1] > gang_lds.cuts[g]) ? 1 : 0;
      unsigned long long want;
      do {
        want = ((seen >> 16) == p.gang_nonce ? seen : (p.gang_nonce << 16)) + 1;
      } while (!__hip_atomic_compare_exchange_strong(cnt, &seen, want, __ATOMIC_RELAXED, __ATOMIC_RELAXED,
                                                     __HIP_MEMORY_SCOPE_AGENT));
      const bool last = (int)(want & 0xffff) == n_parts;
      // the last part leaves the word as a launch that never happened (a replayed launch
      // carries the same number)
      if (last) __hip_atomic_store(cnt, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      gang_last = last ? 1 : 0;
    }
    __syncthreads();
    if (gang_last == 0) continue;
    for (int g = 0; g < p.gangs; ++g) {
      if (g == gang_id || !(gang_lds.cuts[g] < unit_start + unit_tiles && gang_lds.cuts[g + 1] > unit_start &&
                            gang_lds.cuts[g + 1] > gang_lds.cuts[g]))
        continue;
      const unsigned long long* theirs = slot_of(g);
      const unsigned long long* o64 = theirs + (int64_t)w * 32 * kWave + lane;
      unsigned long long got[32];
#pragma unroll
      for (int j = 0; j < 32; ++j) got[j] = __hip_atomic_load(o64 + j * kWave, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      const unsigned long long ml = __hip_atomic_load(theirs + 8 * 32 * kWave + w * kWave + lane, __ATOMIC_RELAXED,
                                                      __HIP_MEMORY_SCOPE_AGENT);
      const float m_other = __builtin_bit_cast(float, (uint32_t)ml);
      const float l_other = __builtin_bit_cast(float, (uint32_t)(ml >> 32));
      const float m_new = fmaxf(m_run, m_other);
      const float m_ref = (m_new == kNegInf) ? 0.f : m_new;
      const float a_mine = fast_exp2(m_run - m_ref), a_other = fast_exp2(m_other - m_ref);
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int i = 0; i < 16; i += 2) {
          const unsigned long long v = got[dt * 8 + i / 2];
          oacc[dt][i] = oacc[dt][i] * a_mine + a_other * __builtin_bit_cast(float, (uint32_t)v);
          oacc[dt][i + 1] = oacc[dt][i + 1] * a_mine + a_other * __builtin_bit_cast(float, (uint32_t)(v >> 32));
        }
      l_run = l_run * a_mine + l_other * a_other;
      m_run = m_new;
    }
  }

  // accumulator i of O^T tile dt is dim 32dt + 8(i/4) + 4h + i%4 of query row c32
  float l = l_run;
  l += __shfl_xor(l, 32, kWave);
  const float inv = (l > 0.f) ? 1.0f / l : 0.f;
  if (to_partial) {
    const int row = row0 + w * 32 + c32;
    if (row < rows_total) {
      const int qi = row / p.group;
      const int hh = row - qi * p.group;
      const int64_t at = p.ragged_tiles > 0 ? part_at + row
                                            : (int64_t)split * p.part_rows + (int64_t)(q_start + qi) * p.n_q + kvh * p.group + hh;
      if (h == 0) p.part_lse[at] = (l > 0.f) ? m_run + __log2f(l) : kNegInf;
      float* dst = p.part_o + at * D + 4 * h;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int a = 0; a < 4; ++a) {
          f32x4_t v = {oacc[dt][4 * a] * inv, oacc[dt][4 * a + 1] * inv, oacc[dt][4 * a + 2] * inv,
                       oacc[dt][4 * a + 3] * inv};
          *reinterpret_cast<f32x4_t*>(dst + 32 * dt + 8 * a) = v;
        }
    }
    return;
  }
  unsigned char* os = smem;
  {
    const int lrow = w * 32 + c32;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int a = 0; a < 4; ++a) {
        u32x2_t wv;
        wv[0] = pack_bf16x2(oacc[dt][4 * a] * inv, oacc[dt][4 * a + 1] * inv);
        wv[1] = pack_bf16x2(oacc[dt][4 * a + 2] * inv, oacc[dt][4 * a + 3] * inv);
        *reinterpret_cast<u32x2_t*>(os + (lrow * OROW + 32 * dt + 8 * a + 4 * h) * 2) = wv;
      }
  }
  __syncthreads();
  constexpr int ROWS_PER_PASS = NW * 4;
  const int c = tid & 15;
#pragma unroll 4
  for (int pass = 0; pass < kRows / ROWS_PER_PASS; ++pass) {
    const int lrow = pass * ROWS_PER_PASS + (tid >> 4);
    const int row = row0 + lrow;
    if (row < rows_total) {
      const int qi = row / p.group;
      const int hh = row - qi * p.group;
      const u32x4_t v = *reinterpret_cast<const u32x4_t*>(os + (lrow * OROW + c * 8) * 2);
      st_global_b128(p.out + ((int64_t)(q_start + qi) * p.n_q + kvh * p.group + hh) * D + c * 8, v);
    }
  }
  }  // the next part of the gang's range (a launch without gang ranges leaves here)
}


// ---- merge of a key-split launch: one 32-lane group per (token, q head) row -----------------
template <int D>
__global__ __launch_bounds__(256) void prefill_merge_kernel(const float* __restrict__ part_o,
                                                            const float* __restrict__ part_lse,
                                                            const int32_t* __restrict__ qo_indptr,
                                                            uint16_t* __restrict__ out, int64_t part_rows,
                                                            int n_q, int n_ksplit, int max_len_extend) {
  constexpr int V = D / 32;  // dims per lane
  const int b = blockIdx.y;
  const int q_start = qo_indptr[b];
  const int q_len = min(qo_indptr[b + 1] - q_start, max_len_extend);
  const int64_t r = (int64_t)blockIdx.x * 8 + (threadIdx.x >> 5);  // row of the request, token-major
  if (r >= (int64_t)q_len * n_q) return;
  const int64_t row = (int64_t)q_start * n_q + r;
  const int c = threadIdx.x & 31;
  float top = kNegInf;
  for (int s = 0; s < n_ksplit; ++s) top = fmaxf(top, part_lse[s * part_rows + row]);
  float acc[V];
#pragma unroll
  for (int i = 0; i < V; ++i) acc[i] = 0.f;
  float total = 0.f;
  for (int s = 0; s < n_ksplit; ++s) {
    const float lse = part_lse[s * part_rows + row];
    if (lse == kNegInf) continue;  // that share saw no key of this row
    const float wgt = exp2f(lse - top);
    total += wgt;
    const float* src = part_o + (s * part_rows + row) * D + c * V;
#pragma unroll
    for (int i = 0; i < V; i += 4) {
      const f32x4_t x = *reinterpret_cast<const f32x4_t*>(src + i);
#pragma unroll
      for (int e = 0; e < 4; ++e) acc[i + e] += wgt * x[e];
    }
  }
  const float inv = (total > 0.f) ? 1.0f / total : 0.f;
  uint16_t* dst = out + row * D + c * V;
#pragma unroll
  for (int i = 0; i < V; i += 4) {
    u32x2_t wv;
    wv[0] = pack_bf16x2(acc[i] * inv, acc[i + 1] * inv);
    wv[1] = pack_bf16x2(acc[i + 2] * inv, acc[i + 3] * inv);
    *reinterpret_cast<u32x2_t*>(dst + i) = wv;
  }
}

// The same for ragged shares: request b's partials are units req_units[2 b] .. + req_units[2 b + 1],
// each [kv head][row of the block]; a request with one share was written by the attention kernel.
template <int D>
__global__ __launch_bounds__(256) void prefill_ragged_merge_kernel(PrefillParams p) {
  constexpr int V = D / 32;  // dims per lane
  const int b = blockIdx.y;
  const int q_start = p.qo_indptr[b];
  const int q_len = min(p.qo_indptr[b + 1] - q_start, p.max_len_extend);
  const int64_t r = (int64_t)blockIdx.x * 8 + (threadIdx.x >> 5);  // row of the request, token-major
  if (r >= (int64_t)q_len * p.n_q) return;
  const int first = p.req_units[2 * b];
  const int count = p.req_units[2 * b + 1];
  if (count <= 1) return;
  const int qi = (int)(r / p.n_q);
  const int hq = (int)(r - (int64_t)qi * p.n_q);
  const int kvh = hq / p.group;
  const int local = qi * p.group + (hq - kvh * p.group);
  const int64_t step = (int64_t)p.n_kv * p.ragged_rows;  // partial rows from one unit to the next
  const int64_t at0 = ((int64_t)first * p.n_kv + kvh) * p.ragged_rows + local;
  const int c = threadIdx.x & 31;
  float top = kNegInf;
  for (int s = 0; s < count; ++s) top = fmaxf(top, p.part_lse[at0 + s * step]);
  float acc[V];
#pragma unroll
  for (int i = 0; i < V; ++i) acc[i] = 0.f;
  float total = 0.f;
  for (int s = 0; s < count; ++s) {
    const float lse = p.part_lse[at0 + s * step];
    if (lse == kNegInf) continue;  // that share saw no key of this row
    const float wgt = exp2f(lse - top);
    total += wgt;
    const float* src = p.part_o + (at0 + s * step) * D + c * V;
#pragma unroll
    for (int i = 0; i < V; i += 4) {
      const f32x4_t x = *reinterpret_cast<const f32x4_t*>(src + i);
#pragma unroll
      for (int e = 0; e < 4; ++e) acc[i + e] += wgt * x[e];
    }
  }
  const float inv = (total > 0.f) ? 1.0f / total : 0.f;
  uint16_t* dst = p.out + ((int64_t)q_start * p.n_q + r) * D + c * V;
#pragma unroll
  for (int i = 0; i < V; i += 4) {
    u32x2_t wv;
    wv[0] = pack_bf16x2(acc[i] * inv, acc[i + 1] * inv);
    wv[1] = pack_bf16x2(acc[i + 2] * inv, acc[i + 3] * inv);
    *reinterpret_cast<u32x2_t*>(dst + i) = wv;
  }
}

}  // namespace

int launch_prefill_merge(const PrefillParams& p, int head_dim, hipStream_t stream) {
  const int64_t rows = (int64_t)p.max_len_extend * p.n_q;
  const dim3 grid((unsigned)((rows + 7) / 8), (unsigned)p.batch);
  if (p.ragged_tiles > 0) {
    if (p.req_units == nullptr) return MSGL_OK;  // no request can have a second share
    if (head_dim == 256) hipLaunchKernelGGL((prefill_ragged_merge_kernel<256>), grid, dim3(256), 0, stream, p);
    else hipLaunchKernelGGL((prefill_ragged_merge_kernel<128>), grid, dim3(256), 0, stream, p);
    return check_launch();
  }
  if (head_dim == 256)
    hipLaunchKernelGGL((prefill_merge_kernel<256>), grid, dim3(256), 0, stream, p.part_o, p.part_lse,
                       p.qo_indptr, p.out, p.part_rows, p.n_q, p.n_ksplit, p.max_len_extend);
  else
    hipLaunchKernelGGL((prefill_merge_kernel<128>), grid, dim3(256), 0, stream, p.part_o, p.part_lse,
                       p.qo_indptr, p.out, p.part_rows, p.n_q, p.n_ksplit, p.max_len_extend);
  return check_launch();
}

// benchmarking switch, one value per host thread (see msgl_set_tuning): 0 the ping-pong kernel,
// anything else the fused kernel it replaced (8 waves x 32 rows), kept as its comparison partner
static thread_local int t_tile_variant = 0;
int tile_variant() { return t_tile_variant; }
void set_tile_variant(int v) { t_tile_variant = v; }

int launch_prefill_tile(const PrefillArgs& a, hipStream_t stream) {
  if (a.head_dim != 128) return MSGL_ERR_HEAD_DIM;
  PrefillParams p;
  int64_t n_blocks = 0;
  bool wide = false;
  PrefillArgs args = a;
  if (tile_variant() != 0) {  // the fused kernel knows uniform key splits only
    args.ragged_tiles = 0;
    args.gangs = 0;
  }
  const int rc = make_prefill_params(args, p, n_blocks, wide);
  if (rc != MSGL_OK || n_blocks == 0) return rc;
  const dim3 grid((unsigned)n_blocks);
  if (tile_variant() != 0) {
    if (wide) hipLaunchKernelGGL((prefill_tile_kernel<128, 1, 8, true>), grid, dim3(512), 0, stream, p);
    else hipLaunchKernelGGL((prefill_tile_kernel<128, 1, 8, false>), grid, dim3(512), 0, stream, p);
  } else {
    if (wide) hipLaunchKernelGGL((prefill_pingpong_kernel<true>), grid, dim3(512), 0, stream, p);
    else hipLaunchKernelGGL((prefill_pingpong_kernel<false>), grid, dim3(512), 0, stream, p);
  }
  const int launched = check_launch();
  if (launched != MSGL_OK || (p.n_ksplit == 1 && p.ragged_tiles == 0)) return launched;
  return launch_prefill_merge(p, 128, stream);
}

}  // namespace msgl
