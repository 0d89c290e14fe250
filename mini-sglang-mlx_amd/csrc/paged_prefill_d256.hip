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
//                K of half i+4 and V of half i+1 leave during step i; a wave waits at the end of
//                step i for the moves it issued in step i-1 (vmcnt counts the newer ones), then
//                the workgroup barrier publishes them: a move has between one and two steps to
//                land.  Four K stages and three V stages of LDS.
//   slot ids   = read through the scalar cache (uniform addresses in the constant address
//                space), so that the only vector-memory operations of a step are its 8 moves
//                and the counted wait means what it says.
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
constexpr int kKStages = 4, kVStages = 3;
constexpr int kVBase = kKStages * kKStage;
constexpr int kStageTotal = kVBase + kVStages * kVStage;  // 118784
constexpr int kKSteps = kD / 16;              // k-steps of QK^T
constexpr int kDT = kD / 32;                  // 32-dim tiles of O^T
constexpr int kMovesPerStep = 2 * kUPW;       // V units then K units, per wave

typedef const __attribute__((address_space(4))) int32_t* ConstI32Ptr;

template <bool WIDE>
__global__ __launch_bounds__(kNW * 64) void prefill_tile256_kernel(PrefillParams p) {
  constexpr int kRows = kPrefillBlockRows256;
  static_assert(kRows == kNW * 32, "one 32-row tile per wave");
  constexpr int OROW = kD + 8;
  constexpr int O_BYTES = kRows * OROW * 2;
  constexpr int SMEM_BYTES = kStageTotal > O_BYTES ? kStageTotal : O_BYTES;
  __shared__ __attribute__((aligned(16))) unsigned char smem[SMEM_BYTES];
  using OffT = typename std::conditional<WIDE, uint64_t, uint32_t>::type;

  const int tid = threadIdx.x;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63;
  const int h = lane >> 5;
  const int c32 = lane & 31;

  // ---- block -> (request, kv head, q block): consecutive block ids go to different XCDs, the
  // q blocks of one (request, kv head) share an XCD and run heaviest first, requests in order
  // of decreasing kv length (each block ranks the requests itself from kv_indptr)
  const int xcd = blockIdx.x & 7;
  const int seq = blockIdx.x >> 3;
  const int pair = (seq / p.n_qblk) * 8 + xcd;
  if (pair >= p.n_pairs) return;
  const int qblk = p.n_qblk - 1 - (seq % p.n_qblk);
  const int want_rank = pair / p.n_kv;
  const int kvh = pair - want_rank * p.n_kv;
  __shared__ int ranked_request;
  for (int i = tid; i < p.batch; i += kNW * 64) {
    const int len_i = p.kv_indptr[i + 1] - p.kv_indptr[i];
    int rank = 0;
    for (int j = 0; j < p.batch; ++j) {
      const int len_j = p.kv_indptr[j + 1] - p.kv_indptr[j];
      rank += (len_j > len_i) || (len_j == len_i && j < i);
    }
    if (rank == want_rank) ranked_request = i;
  }
  __syncthreads();
  const int b = __builtin_amdgcn_readfirstlane(ranked_request);

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
    row_hi = p.is_cross ? kn - 1 : min(qpos, kn - 1);
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
  const ConstI32Ptr idx_base = (ConstI32Ptr)(uintptr_t)(p.kv_indices + kv_start);
  const unsigned char* k_src = reinterpret_cast<const unsigned char*>(p.k_cache + (int64_t)kvh * kD);
  const unsigned char* v_src = reinterpret_cast<const unsigned char*>(p.v_cache + (int64_t)kvh * kD);
  const uint32_t k_row_bytes = (uint32_t)p.k_stride0 * 2u;
  const uint32_t v_row_bytes = (uint32_t)p.v_stride0 * 2u;
  const uint32_t chunk_off = (uint32_t)(lane & 31) * 16u;
  const bool upper = lane >= 32;
  struct Slots {
    int32_t s[kUPW][2];  // slot ids of the two keys of each of this wave's units (uniform)
  };
  auto slot_load = [&](int base, Slots& sl) {
#pragma unroll
    for (int i = 0; i < kUPW; ++i) {
      sl.s[i][0] = idx_base[min(base + w * kUPW + i, kn - 1)];
      sl.s[i][1] = idx_base[min(base + w * kUPW + i + 16, kn - 1)];
    }
  };
  auto lane_offset = [&](const int32_t (&s)[2], uint32_t row_bytes) -> OffT {
    const OffT a = (OffT)(uint32_t)s[0] * row_bytes;  // uniform: scalar multiplies
    const OffT c = (OffT)(uint32_t)s[1] * row_bytes;
    return (upper ? c : a) + chunk_off;
  };
  OffT k_off[kUPW], v_off[kUPW];
  auto k_offsets = [&](const Slots& sl) {
#pragma unroll
    for (int i = 0; i < kUPW; ++i) k_off[i] = lane_offset(sl.s[i], k_row_bytes);
  };
  auto v_offsets = [&](const Slots& sl) {
#pragma unroll
    for (int i = 0; i < kUPW; ++i) v_off[i] = lane_offset(sl.s[i], v_row_bytes);
  };
  // move number n of a step: the V units first, then the K units
  auto move = [&](int n, uint32_t k_stage, uint32_t v_stage) {
    if (n < kUPW)
      lds_direct_b128(lds0 + v_stage + (uint32_t)(w * kUPW + n) * kVUnit, v_src, v_off[n]);
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
  auto rescale = [&](float alpha) {
    if (__any(alpha != 1.0f)) {
#pragma unroll
      for (int dt = 0; dt < kDT; ++dt)
#pragma unroll
        for (int i = 0; i < 16; ++i) oacc[dt][i] *= alpha;
    }
  };
  // Softmax state of one half, decided as soon as its scores exist:
  //   mul    factor still to be applied to the scores: the softmax scale on interior halves
  //          (max commutes with a positive scale), 1 on boundary halves, which are scaled and
  //          masked in place
  //   m_safe the (lazy) running row max the half's exponentials are taken against
  //   alpha  exp2(previous max - m_safe): what O and l must be multiplied by first
  struct Stats {
    float mul, m_safe, alpha;
  };
  auto mask_in_place = [&](f32x16_t& s, int base) {
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int key = base + 8 * (i >> 2) + 4 * h + (i & 3);
      const float x = s[i] * p.scale_log2e;
      s[i] = (key < row_lo || key > row_hi) ? kNegInf : x;
    }
  };
  auto lane_max = [&](const f32x16_t& s) {
    float m = fmaxf(s[0], s[1]);
#pragma unroll
    for (int i = 2; i < 16; ++i) m = fmaxf(m, s[i]);
    return m;
  };
  auto decide = [&](float mx, Stats& st) {
    const float m = wave_max_xor(mx * st.mul, 32);
    const float m_old = m_run;
    const float m_new = fmaxf(m_old, m);
    const float m_use = (m_new - m_old > kLazy) ? m_new : m_old;
    st.m_safe = (m_use == kNegInf) ? 0.f : m_use;
    st.alpha = fast_exp2(m_old - st.m_safe);
    m_run = m_use;
    pin(st.m_safe);
    pin(st.alpha);
  };
  // One step over halves i-1, i, i+1, cut into four slices by scheduling barriers (inside a
  // slice the compiler interleaves MFMA, LDS reads and VALU freely, across slices nothing
  // moves).  Matrix pipe: scores of half i+1 in slices 0, 1; P V of half i-1 in slices 2, 3.
  // VALU: exponentials and packing of half i in slices 0..2; row max and softmax state of half
  // i+1 in slices 2, 3.  Each slice requests the LDS operands of the next one; slice 3 requests
  // the first K operands of the next step (`kops`, carried between calls).
  auto step = [&](f32x16_t& cur, const Stats& st_cur, f32x16_t& nxt, Stats& st_nxt, bool mask_nxt,
                  int nxt_base, const unsigned char* ks, const unsigned char* vs,
                  const unsigned char* ks_after, bf16x8_t (&kops)[8], const bf16x8_t (&pb_prev)[2],
                  bf16x8_t (&pb_cur)[2], uint32_t k_fill, uint32_t v_fill) {
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
    auto moves = [&](int slice) {
#pragma unroll
      for (int n = slice * 2; n < slice * 2 + 2; ++n) move(n, k_fill, v_fill);
    };
    bf16x8_t ops_a[8], ops_b[8];
    // slice 0
#pragma unroll
    for (int i = 0; i < 16; ++i) nxt[i] = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) ops_a[e] = k_operand(ks, 8 + e);
#pragma unroll
    for (int e = 0; e < 8; ++e) nxt = mfma_32x32x16(kops[e], qreg[e], nxt);
    exp_slice(0);
    moves(0);
    __builtin_amdgcn_sched_barrier(0);
    // slice 1
#pragma unroll
    for (int dt = 0; dt < kDT; ++dt) ops_b[dt] = v_operand(vs, 0, dt);
#pragma unroll
    for (int e = 0; e < 8; ++e) nxt = mfma_32x32x16(ops_a[e], qreg[8 + e], nxt);
    exp_slice(8);
    pack_slice(0);
    moves(1);
    __builtin_amdgcn_sched_barrier(0);
    st_nxt.mul = p.scale_log2e;
    if (mask_nxt) {  // boundary half: scale and mask in place
      asm volatile("" ::: "memory");  // keeps this a branch instead of 64 selects in every step
      mask_in_place(nxt, nxt_base);
      st_nxt.mul = 1.0f;
    }
    // slice 2
#pragma unroll
    for (int dt = 0; dt < kDT; ++dt) ops_a[dt] = v_operand(vs, 1, dt);
#pragma unroll
    for (int dt = 0; dt < kDT; ++dt) oacc[dt] = mfma_32x32x16(ops_b[dt], pb_prev[0], oacc[dt]);
    pack_slice(1);
    float mx = lane_max(nxt);
    pin(mx);
    moves(2);
    __builtin_amdgcn_sched_barrier(0);
    // slice 3
#pragma unroll
    for (int e = 0; e < 8; ++e) kops[e] = k_operand(ks_after, e);
#pragma unroll
    for (int dt = 0; dt < kDT; ++dt) oacc[dt] = mfma_32x32x16(ops_a[dt], pb_prev[1], oacc[dt]);
    l_run = l_run * st_cur.alpha + psum;
    decide(mx, st_nxt);
    moves(3);
    __builtin_amdgcn_sched_barrier(0);
  };

  const bool general_scale = p.scale_log2e <= 0.f;  // the fast path needs a positive scale
  auto needs_mask = [&](int base) {  // some row of this wave sees only part of keys base .. base+31
    return general_scale || (base < w_lo_max) || (base + 31 > w_hi_min);
  };
  if (n_steps > 0) {
    // ---- prologue: K of halves 0..3 and V of half 0 leave; the first four stages are waited for
    Slots sk, sv;
#pragma unroll
    for (int x = 0; x < 3; ++x) {
      slot_load(k_lo + x * kHalf, sk);
      k_offsets(sk);
      if (x == 0) v_offsets(sk);
#pragma unroll
      for (int n = (x == 0 ? 0 : kUPW); n < kMovesPerStep; ++n) move(n, x * kKStage, kVBase);
    }
    slot_load(k_lo + 3 * kHalf, sk);
    k_offsets(sk);
#pragma unroll
    for (int n = kUPW; n < kMovesPerStep; ++n) move(n, 3 * kKStage, 0);
    // slot ids for the moves of step 0: K of half 4, V of half 1
    slot_load(k_lo + 4 * kHalf, sk);
    slot_load(k_lo + 1 * kHalf, sv);
    wait_vm_at_most<kUPW>();
    __syncthreads();

    f32x16_t sa, sb;
    Stats st_a, st_b;
    bf16x8_t pb_a[2], pb_b[2];
    {  // scores of half 0
      const unsigned char* ks = smem + k_lane;
#pragma unroll
      for (int i = 0; i < 16; ++i) sa[i] = 0.f;
#pragma unroll
      for (int kstep = 0; kstep < kKSteps; ++kstep) sa = mfma_32x32x16(k_operand(ks, kstep), qreg[kstep], sa);
    }
    st_a.mul = p.scale_log2e;
    if (needs_mask(k_lo)) {
      mask_in_place(sa, k_lo);
      st_a.mul = 1.0f;
    }
    decide(lane_max(sa), st_a);
    st_b.mul = 1.0f;
    st_b.alpha = 1.0f;
    st_b.m_safe = 0.f;
#pragma unroll
    for (int u = 0; u < 2; ++u) pb_b[u] = as_bf16x8(u32x4_t{0u, 0u, 0u, 0u});

    // Stage rings.  Step i reads K of half i+1 (stage (i+1) % 4), takes the first operands of
    // half i+2, fills stage i % 4 with half i+4; reads V of half i-1 (stage (i-1) % 3; the P
    // of "half -1" is zero, so step 0 may read V of half 0) and fills stage (i+1) % 3.
    uint32_t kr = 0;              // i % 4
    uint32_t v_read = kVBase;     // stage of half i-1
    uint32_t v_mid = kVBase;      // stage of half i (being waited for during step i-1 .. i)
    uint32_t v_fill = kVBase + kVStage;
    uint32_t v_free = kVBase + 2 * kVStage;
    bf16x8_t kops[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) kops[e] = k_operand(smem + kKStage + k_lane, e);

    auto k_stage = [&](uint32_t r) { return (r & 3u) * (uint32_t)kKStage; };
    auto advance = [&](int i) {
      kr = (kr + 1) & 3u;
      const uint32_t freed = (i == 0) ? v_free : v_read;
      v_read = v_mid;
      v_mid = v_fill;
      v_fill = freed;
    };
    for (int i = 0; i < n_steps; i += 2) {
      const int tb = k_lo + i * kHalf;
      // step i: cur = sa
      k_offsets(sk);
      v_offsets(sv);
      slot_load(tb + 5 * kHalf, sk);
      slot_load(tb + 2 * kHalf, sv);
      rescale(st_b.alpha);
      step(sa, st_a, sb, st_b, needs_mask(tb + kHalf), tb + kHalf, smem + k_stage(kr + 1) + k_lane,
           smem + v_read + v_lane, smem + k_stage(kr + 2) + k_lane, kops, pb_b, pb_a, k_stage(kr), v_fill);
      wait_vm_at_most<kMovesPerStep>();
      __syncthreads();
      advance(i);
      // step i+1: cur = sb
      k_offsets(sk);
      v_offsets(sv);
      slot_load(tb + 6 * kHalf, sk);
      slot_load(tb + 3 * kHalf, sv);
      rescale(st_a.alpha);
      step(sb, st_b, sa, st_a, needs_mask(tb + 2 * kHalf), tb + 2 * kHalf, smem + k_stage(kr + 1) + k_lane,
           smem + v_read + v_lane, smem + k_stage(kr + 2) + k_lane, kops, pb_a, pb_b, k_stage(kr), v_fill);
      wait_vm_at_most<kMovesPerStep>();
      __syncthreads();
      advance(i + 1);
    }
    // the last half's P V is still owed: V of half n_steps-1 sits in the stage `v_read`
    rescale(st_b.alpha);
    {
      const unsigned char* vs = smem + v_read + v_lane;
#pragma unroll
      for (int u = 0; u < 2; ++u)
#pragma unroll
        for (int dt = 0; dt < kDT; ++dt) oacc[dt] = mfma_32x32x16(v_operand(vs, u, dt), pb_b[u], oacc[dt]);
    }
    wait_all_vm();     // moves still in flight target the stages the epilogue is about to reuse
    __syncthreads();
  }

  // ---- epilogue: normalise, transpose through LDS, store whole rows ---------------------
  // accumulator i of O^T tile dt is dim 32dt + 8(i/4) + 4h + i%4 of query row c32
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
  return check_launch();
}

}  // namespace msgl
