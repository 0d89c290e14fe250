// LDS-direct loads, counted waits and transposing LDS reads shared by the prefill tile kernels.
#pragma once
#include "msgl_device.h"
#include "prefill_params.h"

namespace msgl {

typedef short s16x4_t __attribute__((ext_vector_type(4)));
typedef int i32x4_t __attribute__((ext_vector_type(4)));
constexpr bf16x2_t kOnes = {(__bf16)1.0f, (__bf16)1.0f};
#define MSGL_LDS_PTR(T, p) ((__attribute__((address_space(3))) T*)(p))

// 64 lanes x 16 bytes: lane l's 16 bytes at `saddr + voff` land at LDS byte lds_addr + 16 l.
// The compiler does not see the LDS write: callers wait on vmcnt and pass a barrier before
// anyone reads the destination.  M0 is written without telling the compiler (it cannot be
// named as a clobber); nothing else in these kernels uses M0.
__device__ __forceinline__ void lds_direct_b128(uint32_t lds_addr, const void* saddr, uint32_t voff) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
               :
               : "s"(lds_addr), "v"(voff), "s"(saddr)
               : "memory");
}
__device__ __forceinline__ void lds_direct_b128(uint32_t lds_addr, const void* saddr, uint64_t voff) {
  const unsigned char* a = static_cast<const unsigned char*>(saddr) + voff;
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off"
               :
               : "s"(lds_addr), "v"(a)
               : "memory");
}
// 64 lanes x 4 bytes: lane l's dword at `saddr + voff` lands at LDS byte lds_addr + 4 l.
__device__ __forceinline__ void lds_direct_b32(uint32_t lds_addr, const void* saddr, uint32_t voff) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2"
               :
               : "s"(lds_addr), "v"(voff), "s"(saddr)
               : "memory");
}
// s_waitcnt vmcnt(0) (expcnt and lgkmcnt fields left at their maxima).  Issued through the
// builtin so that the compiler's own wait bookkeeping sees it.
__device__ __forceinline__ void wait_all_vm() {
  __builtin_amdgcn_s_waitcnt(0x0F70);
  asm volatile("" ::: "memory");
}

// s_waitcnt vmcnt(N): returns once at most N of this wave's vector-memory loads are still in
// flight.  Loads complete in issue order, so this waits for everything older than the last N.
template <int N>
__device__ __forceinline__ void wait_vm_at_most() {
  static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit field");
  __builtin_amdgcn_s_waitcnt(0x0F70 | (N & 15) | ((N >> 4) << 14));
  asm volatile("" ::: "memory");
}

// Lane i of each 16-lane group receives element (i % 4) of the 8 bytes addressed by lanes
// i/4, 4 + i/4, 8 + i/4, 12 + i/4 of its group.
__device__ __forceinline__ u32x2_t lds_read_tr16(const unsigned char* p) {
  const s16x4_t v = __builtin_amdgcn_ds_read_tr16_b64_v4i16(MSGL_LDS_PTR(s16x4_t, p));
  return __builtin_bit_cast(u32x2_t, v);
}

// Workgroup id -> (unit = (request rank, kv head, key split), query block), heaviest query block
// (latest rows) first; `ok` is false for the ids that pad the grid.  Consecutive ids go to
// different XCDs.
struct BlockWork {
  int unit, qblk;
  bool ok;
};
__device__ __forceinline__ BlockWork prefill_block_work(const PrefillParams& p) {
  const int xcd = blockIdx.x & 7;
  const int seq = blockIdx.x >> 3;
  const int n_units = p.n_pairs * p.n_ksplit;
  const int whole_rows = n_units >> 3;  // rows of 8 units, one unit per XCD
  BlockWork w;
  if (seq < whole_rows * p.n_qblk) {  // all query blocks of a unit on one XCD, back to back
    w.unit = (seq / p.n_qblk) * 8 + xcd;
    w.qblk = p.n_qblk - 1 - (seq % p.n_qblk);
    w.ok = true;
  } else {  // the left-over units: each on xcds_per_unit XCDs
    const int side_by_side = 8 / p.xcds_per_unit;
    const int u = xcd % side_by_side;
    const int j = (seq - whole_rows * p.n_qblk) * p.xcds_per_unit + xcd / side_by_side;
    w.unit = whole_rows * 8 + u;
    w.qblk = p.n_qblk - 1 - j;
    w.ok = w.unit < n_units && j < p.n_qblk;
  }
  return w;
}

// ---- ragged shares: which (request, share) is unit `u`? ------------------------------------------
// Visible key range of a request's only query block (rows 0 .. q_len * group - 1), the floor
// rounded down to a tile: the kernels compute the same for their block.
__device__ __forceinline__ void ragged_key_range(const PrefillParams& p, int b, int* k_lo, int* k_hi, int* q_len) {
  const int ql = min(p.qo_indptr[b + 1] - p.qo_indptr[b], p.max_len_extend);
  const int kn = max(p.kv_indptr[b + 1] - p.kv_indptr[b], 0);
  const int prefix = p.prefix_lens[b];
  int hi = p.is_cross ? kn : min(kn, prefix + ql);
  int lo = (p.window > 0) ? max(0, prefix - p.window + 1) : 0;
  lo &= ~(kBN - 1);
  if (hi < lo) hi = lo;
  *k_lo = lo;
  *k_hi = hi;
  *q_len = ql;
}
struct RaggedUnit {
  int request, share, count, first;  // count = shares of the request, first = its first unit
  bool ok;                           // false: `u` lies past the last unit
};
// Every thread of the workgroup calls it.  A request with rows has at least one share (which
// writes zeros if it sees no key); a request without rows has none.
template <int THREADS>
__device__ __forceinline__ RaggedUnit ragged_unit(const PrefillParams& p, int u, int tid) {
  constexpr int kChunks = kRaggedMaxBatch / kWave;
  __shared__ int count[kRaggedMaxBatch];
  __shared__ int chunk_sum[kChunks];  // shares of requests 64 c .. 64 c + 63
  __shared__ int found[4];
  const int lane = tid & (kWave - 1);
  const int wave = tid / kWave;
  if (tid == 0) found[0] = -1;
  for (int i = tid; i < p.batch; i += THREADS) {
    int lo, hi, ql;
    ragged_key_range(p, i, &lo, &hi, &ql);
    const int tiles = (hi - lo + kBN - 1) / kBN;
    count[i] = ql > 0 ? max(1, (tiles + p.ragged_tiles - 1) / p.ragged_tiles) : 0;
  }
  __syncthreads();
  const int n_chunks = (p.batch + kWave - 1) / kWave;
  for (int c = wave; c < n_chunks; c += THREADS / kWave) {
    const int i = c * kWave + lane;
    int v = i < p.batch ? count[i] : 0;
#pragma unroll
    for (int off = 1; off < kWave; off <<= 1) v += __shfl_xor(v, off, kWave);
    if (lane == 0) chunk_sum[c] = v;
  }
  __syncthreads();
  int base = 0, c = 0;  // the chunk that holds unit u: the same for every thread
  for (; c < n_chunks; ++c) {
    const int sum = chunk_sum[c];
    if (u < base + sum) break;
    base += sum;
  }
  if (c < n_chunks && wave == 0) {
    const int i = c * kWave + lane;
    const int v = i < p.batch ? count[i] : 0;
    const int first = base + wave_inclusive_scan(v) - v;
    if (v > 0 && u >= first && u < first + v) {
      found[0] = i;
      found[1] = u - first;
      found[2] = v;
      found[3] = first;
    }
  }
  __syncthreads();
  RaggedUnit r;
  r.request = found[0];
  r.share = found[1];
  r.count = found[2];
  r.first = found[3];
  r.ok = found[0] >= 0;
  return r;
}

// ---- gang ranges: which parts of which units does this workgroup take? ---------------------------
// (prefill_gangs() in prefill_params.h says what they are for.)  Workgroup id -> XCD id % 8, gang
// (id / 8) / n_qblk, member (id / 8) % n_qblk = its query block in every unit.  The XCD's units are
// (request rank, kv head) pairs number i * 8 + xcd, i = 0 .. U - 1, longest requests first; unit i
// is `len` key tiles long (those the member's query block sees).  The units' tiles laid end to end
// are cut at multiples of ceil(total / gangs); a cut that falls within `gang_snap` tiles of either
// end of a unit moves to that end.  The workgroups of one member compute the same plan in every gang.
struct GangPlan {
  int first_unit, last_unit;  // units that overlap this gang's range (first > last: none)
  int lo, hi;                 // the gang's range [lo, hi) in tiles of the XCD's unit stream
};
struct GangLds {
  int order[kRankedBatch];           // request of rank r
  int kv_start[kRankedBatch], kv_len[kRankedBatch], q_start[kRankedBatch], q_len[kRankedBatch],
      prefix[kRankedBatch];          // per request (q_len capped by max_len_extend)
  int len[kGangMaxUnits];            // tiles of unit i
  int start[kGangMaxUnits + 1];      // its place in the stream; start[U] = total
  int cuts[kComputeUnits / 8 + 1];   // cuts[g] .. cuts[g + 1]: range of gang g
  int nonempty_before[kGangMaxUnits + 1];  // units with tiles in front of unit i
  int first_unit, last_unit;
  int cost_at;
};
constexpr int kGangUnitCost = 5;
// Every thread of the workgroup calls it (it holds barriers).
template <int THREADS>
__device__ __forceinline__ GangPlan gang_plan(const PrefillParams& p, GangLds& L, int xcd, int gang, int member,
                                              int block_rows, int tid) {
  __shared__ __attribute__((aligned(16))) int lens[kRankedBatch];
  const int padded = (p.batch + 3) & ~3;
  // every request's geometry in one round trip; the parts of the launch read it from here
  for (int i = tid; i < padded; i += THREADS) {
    int len = (int)0x80000000;
    if (i < p.batch) {
      const int k0 = p.kv_indptr[i], k1 = p.kv_indptr[i + 1], q0 = p.qo_indptr[i], q1 = p.qo_indptr[i + 1];
      len = k1 - k0;
      L.kv_start[i] = k0;
      L.q_start[i] = q0;
      L.q_len[i] = min(q1 - q0, p.max_len_extend);
      L.prefix[i] = p.prefix_lens[i];
    }
    lens[i] = len;
  }
  if (tid == 0) {
    L.first_unit = 0x7fffffff;
    L.last_unit = -1;
  }
  __syncthreads();
  for (int i = tid; i < p.batch; i += THREADS) {  // rank of request i: longer ones, and equal ones before it
    const int len_i = lens[i];
    int rank = 0;
    for (int j = 0; j < padded; j += 4) {
      const i32x4_t l4 = *reinterpret_cast<const i32x4_t*>(&lens[j]);
#pragma unroll
      for (int e = 0; e < 4; ++e) rank += (l4[e] > len_i) || (l4[e] == len_i && j + e < i);
    }
    L.order[rank] = i;
    L.kv_len[i] = max(len_i, 0);
  }
  __syncthreads();
  const int n_units = p.n_pairs / 8;
  for (int i = tid; i < n_units; i += THREADS) {
    const int b = L.order[(i * 8 + xcd) / p.n_kv];
    const int ql = L.q_len[b];
    const int kn = L.kv_len[b];
    // the tiles this workgroup's own query block sees: the members of a gang cut the same unit at
    // (slightly) different tiles, each so that its own work is level with that of its peers in
    // the other gangs (a cut by the longest block would leave the later blocks of every unit,
    // which see more keys, up to n_qblk - 1 tiles per unit behind)
    const int q_hi = min(ql, ((member + 1) * block_rows + p.group - 1) / p.group);  // past its last query
    const int hi = p.is_cross ? kn : min(kn, L.prefix[b] + q_hi);
    // a block with rows but no visible key still has to write its zeros: one (empty) tile
    L.len[i] = member * block_rows < ql * p.group ? max(1, (hi + kBN - 1) / kBN) : 0;
  }
  __syncthreads();
  if (tid < kWave) {  // exclusive prefix sums, 64 units at a time
    int base = 0, base_n = 0;
    for (int i0 = 0; i0 < n_units; i0 += kWave) {
      const int i = i0 + tid;
      const int v = i < n_units ? L.len[i] : 0;
      const int incl = wave_inclusive_scan(v);
      const int incl_n = wave_inclusive_scan(v > 0 ? 1 : 0);
      if (i < n_units) {
        L.start[i] = base + incl - v;
        L.nonempty_before[i] = base_n + incl_n - (v > 0 ? 1 : 0);
      }
      base += __shfl(incl, kWave - 1, kWave);
      base_n += __shfl(incl_n, kWave - 1, kWave);
    }
    if (tid == 0) {
      L.start[n_units] = base;
      L.nonempty_before[n_units] = base_n;
    }
  }
  __syncthreads();
  // Cuts, one after the other, in a stream where every unit also takes kGangUnitCost places in
  // front of its tiles (what a workgroup spends on starting and finishing a unit, in tile times):
  // each cut takes an equal share of what lies behind the cut before it (a cut that moved to a
  // unit's end changes what is left).  cost_at = place of the latest cut in that stream.
  const int total = L.start[n_units];
  if (tid == 0) {
    L.cuts[0] = 0;
    L.cuts[p.gangs] = total;
    L.cost_at = 0;
  }
  __syncthreads();
  // units with tiles in front of unit i (their unit costs precede its place in the cost stream)
  auto cost_start = [&](int i) { return L.start[i] + kGangUnitCost * L.nonempty_before[i]; };
  const int cost_total = total + kGangUnitCost * L.nonempty_before[n_units];
  for (int g = 1; g < p.gangs; ++g) {
    const int prev = L.cost_at;
    const int want = prev + (cost_total - prev + (p.gangs - g)) / (p.gangs - g + 1);
    __syncthreads();  // everyone has read cost_at
    for (int i = tid; i < n_units; i += THREADS) {
      const int n = L.len[i];
      const int c0 = cost_start(i);
      if (n > 0 && want >= c0 && want < c0 + kGangUnitCost + n) {  // exactly one unit holds place `want`
        int o = max(want - c0 - kGangUnitCost, 0);                  // tile of the unit the cut falls on
        o = o < p.gang_snap ? 0 : (n - o < p.gang_snap ? n : o);
        L.cuts[g] = L.start[i] + o;
        L.cost_at = o == 0 ? c0 : (o == n ? c0 + kGangUnitCost + n : c0 + kGangUnitCost + o);
      }
    }
    if (tid == 0 && want >= cost_total) {
      L.cuts[g] = total;
      L.cost_at = cost_total;
    }
    __syncthreads();
  }
  GangPlan plan;
  plan.lo = L.cuts[gang];
  plan.hi = L.cuts[gang + 1];
  for (int i = tid; i < n_units; i += THREADS) {
    const int s0 = L.start[i], n = L.len[i];
    if (n > 0 && s0 < plan.hi && s0 + n > plan.lo) {
      atomicMin(&L.first_unit, i);
      atomicMax(&L.last_unit, i);
    }
  }
  __syncthreads();
  plan.first_unit = L.first_unit;
  plan.last_unit = L.last_unit;
  return plan;
}
// Slot (0 or 1) that gang g's part of the unit starting at stream tile `unit_start` uses: 0 if the
// part begins where the gang's range begins, else 1 (then it is the part the range's end cuts).
__device__ __forceinline__ int gang_slot_of(const GangLds& L, int g, int unit_start) {
  return unit_start <= L.cuts[g] ? 0 : 1;
}

// The request whose kv length has rank `want_rank` in decreasing order (ties: lower index first),
// found by the workgroup itself: lengths into LDS once, then each thread ranks one request
// against all of them with broadcast LDS reads.  (Ranking straight from global memory cost every
// workgroup of a 64-request launch 3.4 us.)  Every thread of the workgroup calls it; beyond
// kRankedBatch requests the order is the batch order.
template <int THREADS>
__device__ __forceinline__ int request_of_rank(const int32_t* kv_indptr, int batch, int want_rank, int tid) {
  if (batch > kRankedBatch) return want_rank;  // many requests balance by their number
  __shared__ __attribute__((aligned(16))) int lens[kRankedBatch];
  __shared__ int found;
  const int padded = (batch + 3) & ~3;
  for (int i = tid; i < padded; i += THREADS)
    lens[i] = i < batch ? kv_indptr[i + 1] - kv_indptr[i] : (int)0x80000000;
  __syncthreads();
  for (int i = tid; i < batch; i += THREADS) {
    const int len_i = lens[i];
    int rank = 0;
    for (int j = 0; j < padded; j += 4) {
      const i32x4_t l4 = *reinterpret_cast<const i32x4_t*>(&lens[j]);
#pragma unroll
      for (int e = 0; e < 4; ++e) rank += (l4[e] > len_i) || (l4[e] == len_i && j + e < i);
    }
    if (rank == want_rank) found = i;
  }
  __syncthreads();
  return found;
}

}  // namespace msgl
