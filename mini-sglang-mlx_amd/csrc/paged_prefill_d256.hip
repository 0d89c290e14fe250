// MFMA tile kernel for paged prefill / chunked extend attention at head_dim 256 on gfx950.
// Replaces paged_prefill_attention<bfloat16, 256, 256>
// (mini-sglang-mlx-kernel/csrc/paged_prefill_attention.metal:382-640, instantiated at :647).
//
// Same products and data path as the head_dim 128 kernel (S^T = K Q^T and O^T += V^T P^T on
// mfma 32x32x16 with rows on N, K and V rows moved HBM -> LDS by global_load_lds, V^T operands
// from row-major V through ds_read_b64_tr_b16), re-cut for 512-byte rows:
//   workgroup  = 4 waves (one per SIMD, up to 512 registers each: the 32 x 256 fp32 output
//                tile of a wave is 128 of them, its Q operand 64), 128 rows of one
//                (request, kv head), row = q_idx * group + head.
//   stage      = 32 keys.  One LDS-direct load moves two whole rows (lanes 0..31 one key,
//                lanes 32..63 the key 16 further on); unit u of a stage holds keys u and u + 16,
//                units sit 1040 B (K) or 1088 B (V) apart so the 16 lanes of an LDS read phase
//                fall into different banks.
//   pipeline   = one step per 32 keys: the matrix pipe computes the scores of half i+1 and adds
//                P V of half i-1 (32 MFMAs) while the VALU turns the scores of half i into P.
//                K of half i+4 and V of half i+2 leave during step i; a wave waits at the end of
//                step i for the moves it issued in step i-1 (vmcnt counts the newer ones), then
//                the workgroup barrier publishes them: a move has between one and two steps to
//                land, and every stage is published a step before its first operand is
//                requested (the last slice of a step requests the first operands of the next).
//                Four K stages and four V stages of LDS.
//   slot ids   = fetched a step ahead by loads issued before the step's moves and hidden from
//                the compiler's wait bookkeeping, so that the counted wait at the end of the
//                step (all but the 8 newest operations) covers them and nothing else waits.
//
// Algorithmic flops: 4 * D per visible (query, key) pair and q head (QK^T + PV).
#include <type_traits>

#include "msgl_device.h"
#include "msgl_internal.h"
#include "prefill_params.h"
#include "prefill_tile_common.h"

namespace msgl {
namespace {

constexpr int kD = 256;
constexpr int kHalf = 32;                     // keys per stage and per pipeline step
constexpr int kNW = 4;                        // waves per workgroup
constexpr int kUnits = 16;                    // LDS-direct loads per stage (two 512-byte rows each)
constexpr int kUPW = kUnits / kNW;            // units each wave moves per stage
constexpr int kKUnit = 1024 + 16;             // bytes between K units
constexpr int kVUnit = 1024 + 64;             // bytes between V units
constexpr int kKStage = kUnits * kKUnit;      // 16640
constexpr int kVStage = kUnits * kVUnit;      // 17408
constexpr int kKStages = 4, kVStages = 4;
constexpr int kVBase = kKStages * kKStage;
constexpr int kStageTotal = kVBase + kVStages * kVStage;  // 136192
constexpr int kKSteps = kD / 16;              // k-steps of QK^T
constexpr int kDT = kD / 32;                  // 32-dim tiles of O^T
constexpr int kMovesPerStep = 2 * kUPW;       // V units then K units, per wave

template <bool WIDE>
__global__ __launch_bounds__(kNW * 64) void prefill_tile256_kernel(PrefillParams p) {
  constexpr int kRows = kPrefillBlockRows256;
  static_assert(kRows == kNW * 32, "one 32-row tile per wave");
  constexpr int OROW = kD + 8;
  constexpr int O_BYTES = kRows * OROW * 2;
  constexpr int SMEM_BYTES = kStageTotal > O_BYTES ? kStageTotal : O_BYTES;
  __shared__ __attribute__((aligned(16))) unsigned char smem[SMEM_BYTES];
  using OffT = typename std::conditional<WIDE, uint64_t, uint32_t>::type;
  const ClockProbe clock_probe_(p.clock_probe);

  const int tid = threadIdx.x;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63;
  const int h = lane >> 5;
  const int c32 = lane & 31;

  // ---- block -> (request, kv head, key split, q block): consecutive block ids go to different
  // XCDs, the q blocks of one (request, kv head, key split) read the same keys, share an XCD and
  // run heaviest first, requests in order of decreasing kv length (each block ranks the requests
  // itself from kv_indptr)
  // With ragged shares: block -> (unit = (request, share), kv head), see prefill_ragged_tiles().
  int b, kvh, split, qblk, n_shares = 1;
  bool to_partial = p.n_ksplit > 1;  // leave a partial for the merge kernel, not the result
  int64_t part_at = 0;               // partial row of the block's row 0 (ragged shares)
  if (p.ragged_tiles > 0) {
    kvh = (int)(blockIdx.x % (unsigned)p.n_kv);
    const int u = (int)(blockIdx.x / (unsigned)p.n_kv);
    const RaggedUnit ru = ragged_unit<kNW * 64>(p, u, tid);
    if (!ru.ok) return;
    b = __builtin_amdgcn_readfirstlane(ru.request);
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
    b = __builtin_amdgcn_readfirstlane(request_of_rank<kNW * 64>(p.kv_indptr, p.batch, want_rank, tid));
  }

  const int q_start = __builtin_amdgcn_readfirstlane(p.qo_indptr[b]);
  const int q_len = min(__builtin_amdgcn_readfirstlane(p.qo_indptr[b + 1]) - q_start, p.max_len_extend);
  const int kv_start = __builtin_amdgcn_readfirstlane(p.kv_indptr[b]);
  const int kn = max(__builtin_amdgcn_readfirstlane(p.kv_indptr[b + 1]) - kv_start, 0);
  const int prefix = __builtin_amdgcn_readfirstlane(p.prefix_lens[b]);
  const int rows_total = q_len * p.group;
  const int row0 = qblk * kRows;
  if (row0 >= rows_total) return;

  const int qi_lo = row0 / p.group;
  const int qi_hi = min(rows_total - 1, row0 + kRows - 1) / p.group;
  int k_hi = p.is_cross ? kn : min(kn, prefix + qi_hi + 1);
  int k_lo = (p.window > 0) ? max(0, prefix + qi_lo - p.window + 1) : 0;
  k_lo &= ~(kHalf - 1);
  if (k_hi < k_lo) k_hi = k_lo;
  // key split `split` of n_ksplit: a whole number of step pairs (64 keys) each, the last takes
  // the ragged end; shares past the end are empty (they still leave a "nothing seen" partial)
  if (p.ragged_tiles > 0 || p.n_ksplit > 1) {
    const int shares = p.ragged_tiles > 0 ? n_shares : p.n_ksplit;  // ragged: the request's own count
    const int all_pairs = (k_hi - k_lo + 2 * kHalf - 1) / (2 * kHalf);
    const int share = (all_pairs + shares - 1) / shares * 2 * kHalf;
    k_lo = min(k_lo + split * share, k_hi);
    k_hi = min(k_hi, k_lo + share);
  }
  // steps come in pairs (the loop body handles two, swapping register sets); a half past the
  // end reads clamped keys and is fully masked
  const int n_steps = ((k_hi - k_lo + kHalf - 1) / kHalf + 1) & ~1;

  // ---- this lane's row: Q operand, visibility bounds ------------------------------------
  bf16x8_t qreg[kKSteps];
  int row_lo, row_hi;
  int w_lo_max, w_hi_min;
  {
    const int row = row0 + w * 32 + c32;
    const bool valid = row < rows_total;
    const int qi = valid ? row / p.group : 0;
    const int hh = valid ? row - qi * p.group : 0;
    const int64_t off = ((int64_t)(q_start + qi) * p.n_q + kvh * p.group + hh) * kD;
#pragma unroll
    for (int ks = 0; ks < kKSteps; ++ks) {
      u32x4_t raw = {0u, 0u, 0u, 0u};
      if (valid) raw = ld_global_b128(p.q + off + ks * 16 + h * 8);
      qreg[ks] = as_bf16x8(raw);
    }
    const int qpos = prefix + qi;
    row_lo = (p.window > 0) ? qpos - p.window + 1 : 0;
    // k_hi - 1 only binds under a key split: the pipeline settles one half past its share
    row_hi = min(p.is_cross ? kn - 1 : min(qpos, kn - 1), k_hi - 1);
    w_lo_max = valid ? row_lo : -0x7fffffff;
    w_hi_min = valid ? row_hi : 0x7fffffff;
    if (!valid) {
      row_lo = 1;
      row_hi = 0;
    }
  }
#pragma unroll
  for (int off = 1; off < kWave; off <<= 1) {
    w_lo_max = max(w_lo_max, __shfl_xor(w_lo_max, off, kWave));
    w_hi_min = min(w_hi_min, __shfl_xor(w_hi_min, off, kWave));
  }
  w_lo_max = __builtin_amdgcn_readfirstlane(w_lo_max);
  w_hi_min = __builtin_amdgcn_readfirstlane(w_hi_min);

  f32x16_t oacc[kDT];
#pragma unroll
  for (int dt = 0; dt < kDT; ++dt)
#pragma unroll
    for (int i = 0; i < 16; ++i) oacc[dt][i] = 0.f;
  float m_run = kNegInf, l_run = 0.f;

  // ---- moving a stage: wave w owns units 4w .. 4w+3; in a unit, lane l fetches 16-byte chunk
  // l % 32 of key (unit + 16 (l / 32)) ----------------------------------------------------
  const uint32_t lds0 = (uint32_t)(uintptr_t)MSGL_LDS_PTR(unsigned char, smem);
  const unsigned char* k_src = reinterpret_cast<const unsigned char*>(p.k_cache + (int64_t)kvh * kD);
  const unsigned char* v_src = reinterpret_cast<const unsigned char*>(p.v_cache + (int64_t)kvh * kD);
  const uint32_t k_row_bytes = (uint32_t)p.k_stride0 * 2u;
  const uint32_t v_row_bytes = (uint32_t)p.v_stride0 * 2u;
  const uint32_t chunk_off = (uint32_t)(lane & 31) * 16u;
  // Slot ids of a half: lane l wants the ids of keys 4w .. 4w+3 (+16 for the upper half of the
  // wave).  They are fetched by vector loads the compiler does not see (it would answer the
  // first use of their result with a wait for every load in flight, the moves included); the
  // caller's next counted wait, which names the result registers, makes them valid.  One 16-byte
  // load when the half lies inside the request, element-wise clamped loads on its last,
  // partial half.
  const int32_t* idx_ptr = p.kv_indices + kv_start;
  const int lane_key = w * kUPW + 16 * (lane >> 5);
  auto slot_load = [&](int base, u32x4_t& sl) {
    const int first = base + lane_key;
    if (base + (kNW - 1) * kUPW + 16 + kUPW <= kn) {  // uniform: the whole half is in range
      const uint32_t off = (uint32_t)first * 4u;
      asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(sl) : "v"(off), "s"(idx_ptr) : "memory");
    } else {
      uint32_t e[kUPW];
#pragma unroll
      for (int i = 0; i < kUPW; ++i) {
        const uint32_t off = (uint32_t)min(first + i, kn - 1) * 4u;
        asm volatile("global_load_dword %0, %1, %2" : "=v"(e[i]) : "v"(off), "s"(idx_ptr) : "memory");
      }
      sl = u32x4_t{e[0], e[1], e[2], e[3]};
    }
  };
  // s_waitcnt vmcnt(N) that also stands for "these slot ids have arrived": nothing that reads
  // them can be scheduled above it
  auto wait_vm_and_slots = [&](auto n, u32x4_t& sl) {
    constexpr int N = decltype(n)::value;
    static_assert(N >= 0 && N < 16, "low bits of vmcnt only");
    asm volatile("s_waitcnt vmcnt(%1)" : "+v"(sl) : "n"(N) : "memory");
  };
  // slot ids are clamped to the pool before they become addresses: an id that is out of range
  // (or stale) then reads a wrong row instead of faulting
  auto lane_offset = [&](uint32_t slot, uint32_t row_bytes) -> OffT {
    slot = min(slot, p.max_slot);
    if constexpr (WIDE) return (uint64_t)slot * row_bytes + chunk_off;
    else return __umul24(slot, row_bytes) + chunk_off;  // both factors below 2^24 here
  };
  // K offsets of the half whose K leaves in this step; V offsets of the halves whose V leaves in
  // this step (`v_off[par]`, computed two steps ago from the same slot ids as that half's K)
  OffT k_off[kUPW], v_off[2][kUPW];
  // move number n of a step: the V units first, then the K units
  auto move = [&](int n, uint32_t k_stage, uint32_t v_stage, const OffT (&voff)[kUPW]) {
    if (n < kUPW)
      lds_direct_b128(lds0 + v_stage + (uint32_t)(w * kUPW + n) * kVUnit, v_src, voff[n]);
    else
      lds_direct_b128(lds0 + k_stage + (uint32_t)(w * kUPW + n - kUPW) * kKUnit, k_src, k_off[n - kUPW]);
  };

  // per-lane LDS read offsets inside a stage
  //   K operand of MFMA row c32 (key c32 of the half): unit c32 % 16, row c32 / 16
  const uint32_t k_lane = (uint32_t)(c32 & 15) * kKUnit + (uint32_t)(c32 >> 4) * 512u + (uint32_t)h * 16u;
  //   V^T operand: group g = lane/16 reads dims 16 (g%2) .. +15 of keys 4h .. 4h+3 (+8)
  const uint32_t v_lane = (uint32_t)(4 * h + ((lane & 15) >> 2)) * kVUnit +
                          (uint32_t)((lane >> 4) & 1) * 32u + (uint32_t)(lane & 3) * 8u;

  // ---- the pieces of one step -------------------------------------------------------------
  // S^T[key][row]: key = base + 8(i/4) + 4h + i%4, row = c32
  auto k_operand = [&](const unsigned char* ks, int kstep) {
    return as_bf16x8(*reinterpret_cast<const u32x4_t*>(ks + kstep * 32));
  };
  // keys {16u + 4h + e} and {16u + 8 + 4h + e}, e = 0..3, of the half: the S^T rows that the
  // lane's accumulators 8u .. 8u+7 hold
  auto v_operand = [&](const unsigned char* vs, int u, int dt) {
    const u32x2_t lo = lds_read_tr16(vs + u * 512 + dt * 64);
    const u32x2_t hi = lds_read_tr16(vs + u * 512 + dt * 64 + 8 * kVUnit);
    return as_bf16x8(u32x4_t{lo[0], lo[1], hi[0], hi[1]});
  };
  auto mask_in_place = [&](f32x16_t& s, int base) {
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int key = base + 8 * (i >> 2) + 4 * h + (i & 3);
      const float x = s[i] * p.scale_log2e;
      s[i] = (key < row_lo || key > row_hi) ? kNegInf : x;
    }
  };
  const f32x16_t zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  float alpha_prev = 1.0f;  // what O must be multiplied by before the next P V is added
  // O *= alpha.  The output tile lives in accumulation registers, which the VALU cannot
  // address; written as plain C++ the allocator copies all 128 of them into VGPRs at the top of
  // every step, whether or not this rare path runs.  Spelled out, the copies stay in here.
  auto rescale_output = [&](float alpha) {
    // the hazard checker does not look inside the statements below: give the last MFMAs time to
    // retire their results before they are read, and the writes time to land before the next MFMA
    asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
#pragma unroll
    for (int dt = 0; dt < kDT; ++dt)
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        float x = oacc[dt][i], t;
        asm volatile("v_accvgpr_read_b32 %1, %0\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 %0, %1"
                     : "+a"(x), "=&v"(t)
                     : "v"(alpha));
        oacc[dt][i] = x;
      }
    asm volatile("s_nop 7" ::: "memory");
  };
  // Softmax state of one half, decided as soon as its scores exist:
  //   mul     factor still to be applied to the scores: the softmax scale on interior halves
  //           (max commutes with a positive scale), 1 on boundary halves, which are scaled and
  //           masked in place
  //   m_safe  the (lazy) running row max the exponentials are taken against
  //   alpha   exp2(previous max - m_safe): what O and l must be multiplied by first
  struct Stats {
    float mul, m_safe, alpha;
  };
  auto settle = [&](f32x16_t& s, bool mask, int base, Stats& st) {
    st.mul = p.scale_log2e;
    if (mask) {  // boundary half
      asm volatile("" ::: "memory");  // keeps this a branch instead of 64 selects in every step
      mask_in_place(s, base);
      st.mul = 1.0f;
    }
    float mx = fmaxf(s[0], s[1]);
#pragma unroll
    for (int i = 2; i < 16; ++i) mx = fmaxf(mx, s[i]);
    const float m = wave_max_xor(mx * st.mul, 32);
    const float m_old = m_run;
    const float m_new = fmaxf(m_old, m);
    const float m_use = (m_new - m_old > kLazy) ? m_new : m_old;
    st.m_safe = (m_use == kNegInf) ? 0.f : m_use;
    st.alpha = fast_exp2(m_old - st.m_safe);
    m_run = m_use;
  };
  // One step over halves i-1, i, i+1.  The 32 MFMAs (16 chained ones for the scores of half
  // i+1, 16 independent ones adding P V of half i-1) depend on nothing the VALU does in this
  // step; they are spread over four slices, 4 + 4 each, so that the score chain always has an
  // independent neighbour, and each slice requests the LDS operands of the next (the last one
  // those of the next step's first slice: `kq[0]`, `vq[0]` are carried between calls).  The
  // VALU turns the scores of half i into bf16 P and the row sum (slices 0..2); in the last
  // slice the score chain of half i+1 ends first and its softmax state is settled behind the
  // four P V MFMAs that remain, so the next step starts exponentiating at once.  Scheduling
  // barriers separate the slices: inside one the compiler interleaves freely, across them
  // nothing moves.
  auto step = [&](f32x16_t& cur, const Stats& st_cur, f32x16_t& nxt, Stats& st_nxt, bool mask_nxt,
                  int nxt_base, const unsigned char* ks,
                  const unsigned char* vs, const unsigned char* ks_after, const unsigned char* vs_after,
                  bf16x8_t (&kq)[2][4], bf16x8_t (&vq)[2][4], const bf16x8_t (&pb_prev)[2],
                  bf16x8_t (&pb_cur)[2], uint32_t k_fill, uint32_t v_fill, const OffT (&voff)[kUPW]) {
    if (__any(alpha_prev != 1.0f)) {  // rare: some row's lazy max moved in the previous step
      rescale_output(alpha_prev);
    }
    float psum = 0.f;
    auto exp_slice = [&](int first) {  // elements first .. first+7
#pragma unroll
      for (int i = first; i < first + 8; ++i) {
        float e = fast_exp2(__builtin_fmaf(cur[i], st_cur.mul, -st_cur.m_safe));
        pin(e);  // keeps the arithmetic in its slice
        cur[i] = e;
      }
    };
    auto pack_slice = [&](int u) {
      u32x4_t pk;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        uint32_t pw = pack_bf16x2(cur[8 * u + 2 * j], cur[8 * u + 2 * j + 1]);
        pin(pw);
        pk[j] = pw;
        // row sum of the rounded weights, the ones that multiply V
        psum = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, pw), kOnes, psum, false);
      }
      pb_cur[u] = as_bf16x8(pk);
    };
    auto qk_mfmas = [&](int s) {  // k-steps 4s .. 4s+3 of the scores
#pragma unroll
      for (int e = 0; e < 4; ++e)
        nxt = mfma_32x32x16(kq[s & 1][e], qreg[4 * s + e], (s == 0 && e == 0) ? zero16 : nxt);
    };
    auto pv_mfmas = [&](int s) {  // keys 16 (s/2) .. +15, dim tiles 4 (s%2) .. +3
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int dt = 4 * (s & 1) + e;
        oacc[dt] = mfma_32x32x16(vq[s & 1][e], pb_prev[s >> 1], oacc[dt]);
      }
    };
    auto request_slice = [&](int s) {  // LDS operands of slice s (s == 4: slice 0 of the next step)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        kq[s & 1][e] = (s < 4) ? k_operand(ks, 4 * s + e) : k_operand(ks_after, e);
        vq[s & 1][e] = (s < 4) ? v_operand(vs, s >> 1, 4 * (s & 1) + e) : v_operand(vs_after, 0, e);
      }
    };
    auto moves = [&](int s) {
#pragma unroll
      for (int n = s * 2; n < s * 2 + 2; ++n) move(n, k_fill, v_fill, voff);
    };
    // Order inside a slice: its 12 LDS requests first, then each of the 8 MFMAs followed by a
    // share of the slice's VALU work (left alone, the scheduler issues the requests last, and
    // the next slice starts by waiting for them).
    auto slice_order = [](auto valu_per_mfma) {
      __builtin_amdgcn_sched_group_barrier(0x100, 12, 0);  // LDS reads
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                    // MFMA
        __builtin_amdgcn_sched_group_barrier(0x002, decltype(valu_per_mfma)::value, 0);  // VALU
      }
    };
    // slice 0
    request_slice(1);
    qk_mfmas(0);
    pv_mfmas(0);
    exp_slice(0);
    moves(0);
    slice_order(std::integral_constant<int, 4>{});
    __builtin_amdgcn_sched_barrier(0);
    // slice 1
    request_slice(2);
    qk_mfmas(1);
    pv_mfmas(1);
    exp_slice(8);
    pack_slice(0);
    moves(1);
    slice_order(std::integral_constant<int, 5>{});
    __builtin_amdgcn_sched_barrier(0);
    // slice 2
    request_slice(3);
    qk_mfmas(2);
    pv_mfmas(2);
    pack_slice(1);
    moves(2);
    slice_order(std::integral_constant<int, 2>{});
    __builtin_amdgcn_sched_barrier(0);
    // slice 3: the end of the score chain first ...
    request_slice(4);
    qk_mfmas(3);
    moves(3);
    __builtin_amdgcn_sched_barrier(0);
    // ... then the state of half i+1 behind the last P V MFMAs
    pv_mfmas(3);
    settle(nxt, mask_nxt, nxt_base, st_nxt);
    l_run = l_run * st_cur.alpha + psum;
    alpha_prev = st_cur.alpha;
    __builtin_amdgcn_sched_barrier(0);
  };

  const bool general_scale = p.scale_log2e <= 0.f;  // the fast path needs a positive scale
  auto needs_mask = [&](int base) {  // some row of this wave sees only part of keys base .. base+31
    return general_scale || (base < w_lo_max) || (base + 31 > w_hi_min);
  };
  if (n_steps > 0) {
    // ---- prologue: K of halves 0..3 and V of halves 0, 1 leave; all but K of half 3 are waited
    // for.  K of half x lives in K stage x % 4, V of half x in V stage x % 4.
    u32x4_t sl, first_slots[4];
#pragma unroll
    for (int x = 0; x < 4; ++x) slot_load(k_lo + x * kHalf, first_slots[x]);
    slot_load(k_lo + 4 * kHalf, sl);  // for the K move of step 0
    // one round trip for all five (the Q rows requested above arrive with them)
    asm volatile("s_waitcnt vmcnt(0)"
                 : "+v"(first_slots[0]), "+v"(first_slots[1]), "+v"(first_slots[2]), "+v"(first_slots[3]),
                   "+v"(sl)
                 :
                 : "memory");
#pragma unroll
    for (int x = 0; x < 4; ++x) {
#pragma unroll
      for (int i = 0; i < kUPW; ++i) {
        k_off[i] = lane_offset(first_slots[x][i], k_row_bytes);
        v_off[x & 1][i] = lane_offset(first_slots[x][i], v_row_bytes);
      }
#pragma unroll
      for (int n = (x < 2 ? 0 : kUPW); n < kMovesPerStep; ++n)
        move(n, x * kKStage, kVBase + x * kVStage, v_off[x & 1]);
      // the V offsets of halves 2 and 3 stay in v_off[0], v_off[1] for the moves of steps 0 and 1
    }
    // everything but K of half 3 has to have landed
    wait_vm_at_most<kUPW>();
    __syncthreads();

    f32x16_t sa = zero16, sb;
    bf16x8_t pb_a[2], pb_b[2];
    {  // scores of half 0
      const unsigned char* ks = smem + k_lane;
#pragma unroll
      for (int kstep = 0; kstep < kKSteps; ++kstep) sa = mfma_32x32x16(k_operand(ks, kstep), qreg[kstep], sa);
    }
    // Step 0 refills K stage 0 (every later step refills a stage whose readers passed the barrier
    // at the end of the step before): no wave may start those moves while another still reads
    // half 0 from it.
    __syncthreads();
    Stats st_a, st_b;
    settle(sa, needs_mask(k_lo), k_lo, st_a);
#pragma unroll
    for (int u = 0; u < 2; ++u) pb_b[u] = as_bf16x8(u32x4_t{0u, 0u, 0u, 0u});
    // Step i reads K of half i+1, requests the first operands of half i+2 and fills the stage
    // of half i with half i+4; it reads V of half i-1 (the P of "half -1" is zero, so step 0
    // may read V of half 0), requests the first operands of half i and fills the stage of
    // half i-2 with half i+2.
    bf16x8_t kq[2][4], vq[2][4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      kq[0][e] = k_operand(smem + kKStage + k_lane, e);
      vq[0][e] = v_operand(smem + kVBase + v_lane, 0, e);
    }
    auto k_stage = [&](int x) { return (uint32_t)(x & 3) * (uint32_t)kKStage; };
    auto v_stage = [&](int x) { return (uint32_t)kVBase + (uint32_t)(x & 3) * (uint32_t)kVStage; };
    auto one_step = [&](int i, f32x16_t& cur, const Stats& st_cur, f32x16_t& nxt, Stats& st_nxt,
                        const bf16x8_t (&pb_prev)[2], bf16x8_t (&pb_cur)[2], OffT (&voff)[kUPW]) {
      const int tb = k_lo + i * kHalf;
      // offsets of K of half i+4 from the slot ids requested one step ago; the same ids give the
      // V offsets that half will need two steps from now
#pragma unroll
      for (int n = 0; n < kUPW; ++n) k_off[n] = lane_offset(sl[n], k_row_bytes);
      OffT v_new[kUPW];
#pragma unroll
      for (int n = 0; n < kUPW; ++n) v_new[n] = lane_offset(sl[n], v_row_bytes);
      slot_load(tb + 5 * kHalf, sl);  // issued before this step's moves: older than all of them
      step(cur, st_cur, nxt, st_nxt, needs_mask(tb + kHalf), tb + kHalf, smem + k_stage(i + 1) + k_lane,
           smem + v_stage(i == 0 ? 0 : i - 1) + v_lane, smem + k_stage(i + 2) + k_lane,
           smem + v_stage(i) + v_lane, kq, vq, pb_prev, pb_cur, k_stage(i), v_stage(i + 2), voff);
#pragma unroll
      for (int n = 0; n < kUPW; ++n) voff[n] = v_new[n];
      wait_vm_and_slots(std::integral_constant<int, kMovesPerStep>{}, sl);
      __syncthreads();
    };
    for (int i = 0; i < n_steps; i += 2) {
      one_step(i, sa, st_a, sb, st_b, pb_b, pb_a, v_off[0]);
      one_step(i + 1, sb, st_b, sa, st_a, pb_a, pb_b, v_off[1]);
    }
    // the last half's P V is still owed
    if (__any(alpha_prev != 1.0f)) rescale_output(alpha_prev);
    {
      const unsigned char* vs = smem + v_stage(n_steps - 1) + v_lane;
#pragma unroll
      for (int u = 0; u < 2; ++u)
#pragma unroll
        for (int dt = 0; dt < kDT; ++dt) oacc[dt] = mfma_32x32x16(v_operand(vs, u, dt), pb_b[u], oacc[dt]);
    }
    wait_all_vm();     // moves still in flight target the stages the epilogue is about to reuse
    __syncthreads();
  }

  // accumulator i of O^T tile dt is dim 32dt + 8(i/4) + 4h + i%4 of query row c32
  if (to_partial) {
    // ---- key split: normalised fp32 partial and log-sum-exp (base 2) per row, from registers
    float l = l_run;
    l += __shfl_xor(l, 32, kWave);
    const float inv = (l > 0.f) ? 1.0f / l : 0.f;
    const int row = row0 + w * 32 + c32;
    if (row < rows_total) {
      const int qi = row / p.group;
      const int hh = row - qi * p.group;
      const int64_t at = p.ragged_tiles > 0 ? part_at + row
                                            : (int64_t)split * p.part_rows + (int64_t)(q_start + qi) * p.n_q + kvh * p.group + hh;
      if (h == 0) p.part_lse[at] = (l > 0.f) ? m_run + __log2f(l) : kNegInf;
      float* dst = p.part_o + at * kD + 4 * h;
#pragma unroll
      for (int dt = 0; dt < kDT; ++dt)
#pragma unroll
        for (int a = 0; a < 4; ++a) {
          f32x4_t v = {oacc[dt][4 * a] * inv, oacc[dt][4 * a + 1] * inv, oacc[dt][4 * a + 2] * inv,
                       oacc[dt][4 * a + 3] * inv};
          *reinterpret_cast<f32x4_t*>(dst + 32 * dt + 8 * a) = v;
        }
    }
    return;
  }
  // ---- epilogue: normalise, transpose through LDS, store whole rows ---------------------
  unsigned char* os = smem;
  {
    float l = l_run;
    l += __shfl_xor(l, 32, kWave);
    const float inv = (l > 0.f) ? 1.0f / l : 0.f;
    const int lrow = w * 32 + c32;
#pragma unroll
    for (int dt = 0; dt < kDT; ++dt)
#pragma unroll
      for (int a = 0; a < 4; ++a) {
        u32x2_t wv;
        wv[0] = pack_bf16x2(oacc[dt][4 * a] * inv, oacc[dt][4 * a + 1] * inv);
        wv[1] = pack_bf16x2(oacc[dt][4 * a + 2] * inv, oacc[dt][4 * a + 3] * inv);
        *reinterpret_cast<u32x2_t*>(os + (lrow * OROW + 32 * dt + 8 * a + 4 * h) * 2) = wv;
      }
  }
  __syncthreads();
  constexpr int ROWS_PER_PASS = kNW * 64 / 32;  // 32 lanes store one 512-byte row
  const int c = tid & 31;
#pragma unroll 4
  for (int pass = 0; pass < kRows / ROWS_PER_PASS; ++pass) {
    const int lrow = pass * ROWS_PER_PASS + (tid >> 5);
    const int row = row0 + lrow;
    if (row < rows_total) {
      const int qi = row / p.group;
      const int hh = row - qi * p.group;
      const u32x4_t v = *reinterpret_cast<const u32x4_t*>(os + (lrow * OROW + c * 8) * 2);
      st_global_b128(p.out + ((int64_t)(q_start + qi) * p.n_q + kvh * p.group + hh) * kD + c * 8, v);
    }
  }
}

}  // namespace

int launch_prefill_tile256(const PrefillArgs& a, hipStream_t stream) {
  if (a.head_dim != kD) return MSGL_ERR_HEAD_DIM;
  PrefillParams p;
  int64_t n_blocks = 0;
  bool wide = false;
  const int rc = make_prefill_params(a, p, n_blocks, wide, kPrefillBlockRows256);
  if (rc != MSGL_OK || n_blocks == 0) return rc;
  const dim3 grid((unsigned)n_blocks);
  if (wide) hipLaunchKernelGGL((prefill_tile256_kernel<true>), grid, dim3(kNW * 64), 0, stream, p);
  else hipLaunchKernelGGL((prefill_tile256_kernel<false>), grid, dim3(kNW * 64), 0, stream, p);
  const int launched = check_launch();
  if (launched != MSGL_OK || (p.n_ksplit == 1 && p.ragged_tiles == 0)) return launched;
  return launch_prefill_merge(p, kD, stream);
}

}  // namespace msgl
