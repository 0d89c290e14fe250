// Attention metadata of one scheduler step, built on the device in one launch.
// Replaces AttnBackend.build_prefill_metadata / build_decode_metadata and their helpers
// (mini_sglang_mlx/attention/backend.py:205-307): per request a Python slice of the slot table,
// a concatenate, two cumulative sums and two list comprehensions.
//
//   kv_indptr  = cumsum([0] + kv_lens)                       qo_indptr = cumsum([0] + extend_lens)
//   kv_indices = concat(page_table[table_rows[b], :kv_lens[b]])
//   prefix_lens[b] = kv_lens[b] - extend_lens[b]             positions = concat(arange(prefix_b, kv_len_b))
//   num_kv_splits[b] = min(max_kv_splits, max(1, ceil(kv_lens[b] / 128)))
//
// Integer copy work, HBM-bound: 8 bytes per kv token (one slot id read, one written) plus 4 per
// query token.  Every workgroup scans the (short) length arrays itself, so there is no second
// launch and no host round trip; element p of an output stream finds its request by binary
// search in the scanned offsets held in LDS, and consecutive lanes handle consecutive elements,
// so reads inside a request and all writes are coalesced.
#include "msgl_device.h"
#include "msgl_internal.h"

namespace msgl {
namespace {

constexpr int kThreads = 256;
constexpr int kItems = 8;  // output elements per thread and stream

struct MetadataParams {
  const int32_t* page_table;
  const int32_t* table_rows;
  const int32_t* kv_lens;
  const int32_t* extend_lens;  // nullptr: one query per request
  int32_t* kv_indptr;
  int32_t* kv_indices;
  int32_t* qo_indptr;      // may be nullptr
  int32_t* prefix_lens;    // may be nullptr
  int32_t* positions;      // may be nullptr
  int32_t* num_kv_splits;  // may be nullptr
  int64_t table_stride0;
  int32_t batch, n_table_rows, max_seq_len;
  int32_t kv_capacity, q_capacity, max_kv_splits;
};

__device__ __forceinline__ int clamp_len(int v, int hi) { return min(max(v, 0), hi); }

// request holding stream position p: largest b with off[b] <= p (off is non-decreasing, off[0] = 0)
__device__ __forceinline__ int find_request(const int32_t* off, int batch, int p) {
  int lo = 0, hi = batch;  // answer in [lo, hi)
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (off[mid] <= p) lo = mid;
    else hi = mid;
  }
  return lo;
}

__global__ __launch_bounds__(kThreads) void build_metadata_kernel(MetadataParams p) {
  extern __shared__ int32_t lds[];
  int32_t* kv_off = lds;                // [batch + 1]
  int32_t* q_off = lds + p.batch + 1;   // [batch + 1]
  const int tid = threadIdx.x;
  // ---- exclusive scans of the clamped lengths (wave 0; chunks of 64 requests) -------------
  if (tid < kWave) {
    int kv_base = 0, q_base = 0;
    for (int b0 = 0; b0 < p.batch; b0 += kWave) {
      const int b = b0 + tid;
      int kl = 0, ql = 0;
      if (b < p.batch) {
        kl = clamp_len(p.kv_lens[b], p.max_seq_len);
        ql = p.extend_lens ? clamp_len(p.extend_lens[b], kl) : min(1, kl);
      }
      const int ki = wave_inclusive_scan(kl), qi = wave_inclusive_scan(ql);
      if (b < p.batch) {
        kv_off[b] = kv_base + ki - kl;
        q_off[b] = q_base + qi - ql;
      }
      kv_base += __shfl(ki, kWave - 1, kWave);
      q_base += __shfl(qi, kWave - 1, kWave);
    }
    if (tid == 0) {
      kv_off[p.batch] = kv_base;
      q_off[p.batch] = q_base;
    }
  }
  __syncthreads();
  const int total_kv = min(kv_off[p.batch], p.kv_capacity);
  const int total_q = min(q_off[p.batch], p.q_capacity);

  // ---- per-request arrays (first workgroup) ----------------------------------------------
  if (blockIdx.x == 0) {
    for (int b = tid; b <= p.batch; b += kThreads) {
      p.kv_indptr[b] = kv_off[b];
      if (p.qo_indptr) p.qo_indptr[b] = q_off[b];
      if (b < p.batch) {
        const int kl = kv_off[b + 1] - kv_off[b];
        const int ql = q_off[b + 1] - q_off[b];
        if (p.prefix_lens) p.prefix_lens[b] = kl - ql;
        if (p.num_kv_splits) p.num_kv_splits[b] = min(p.max_kv_splits, max(1, (kl + 127) / 128));
      }
    }
  }

  // ---- the two streams ----------------------------------------------------------------------
  const int span = kThreads * kItems;
  // a thread's positions grow with i, so the request is searched once and then advanced
  for (int base = blockIdx.x * span; base < total_kv; base += gridDim.x * span) {
    int b = (base + tid < total_kv) ? find_request(kv_off, p.batch, base + tid) : 0;
#pragma unroll
    for (int i = 0; i < kItems; ++i) {
      const int pos = base + i * kThreads + tid;
      if (pos < total_kv) {
        while (pos >= kv_off[b + 1]) ++b;
        const int row = min(max(p.table_rows[b], 0), p.n_table_rows - 1);
        p.kv_indices[pos] = p.page_table[(int64_t)row * p.table_stride0 + (pos - kv_off[b])];
      }
    }
  }
  if (p.positions) {
    for (int base = blockIdx.x * span; base < total_q; base += gridDim.x * span) {
      int b = (base + tid < total_q) ? find_request(q_off, p.batch, base + tid) : 0;
#pragma unroll
      for (int i = 0; i < kItems; ++i) {
        const int pos = base + i * kThreads + tid;
        if (pos < total_q) {
          while (pos >= q_off[b + 1]) ++b;
          const int kl = kv_off[b + 1] - kv_off[b];
          const int ql = q_off[b + 1] - q_off[b];
          p.positions[pos] = kl - ql + (pos - q_off[b]);
        }
      }
    }
  }
}

}  // namespace

int launch_build_metadata(const MetadataArgs& a, hipStream_t stream) {
  MetadataParams p;
  p.page_table = a.page_table;
  p.table_rows = a.table_rows;
  p.kv_lens = a.kv_lens;
  p.extend_lens = a.extend_lens;
  p.kv_indptr = a.kv_indptr;
  p.kv_indices = a.kv_indices;
  p.qo_indptr = a.qo_indptr;
  p.prefix_lens = a.prefix_lens;
  p.positions = a.positions;
  p.num_kv_splits = a.num_kv_splits;
  p.table_stride0 = a.table_stride0;
  p.batch = (int32_t)a.batch;
  p.n_table_rows = (int32_t)a.n_table_rows;
  p.max_seq_len = (int32_t)a.max_seq_len;
  p.kv_capacity = (int32_t)a.kv_capacity;
  p.q_capacity = (int32_t)a.q_capacity;
  p.max_kv_splits = a.max_kv_splits;
  const size_t lds_bytes = (size_t)(2 * (a.batch + 1)) * sizeof(int32_t);
  const int64_t span = kThreads * kItems;
  int64_t blocks = (std::max(a.kv_capacity, a.q_capacity) + span - 1) / span;
  blocks = std::min<int64_t>(std::max<int64_t>(blocks, 1), 4096);
  hipLaunchKernelGGL(build_metadata_kernel, dim3((unsigned)blocks), dim3(kThreads), lds_bytes, stream, p);
  return check_launch();
}

}  // namespace msgl
