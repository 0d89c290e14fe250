// KV-store scatter: k_cache[indices[r]] = k[r], v_cache[indices[r]] = v[r]  (bit copy).
// Restates mini-sglang-mlx-kernel/csrc/store_kv_cache.metal:7-31 for gfx950.
//
// HBM-bound byte mover.  A row (num_kv_heads * head_dim elements, 2 KiB at 8 x 128 bf16)
// is covered by row_bytes / VEC consecutive lanes, so every wave instruction reads and
// writes whole contiguous rows; one thread moves the same chunk of K and of V so the slot
// index is fetched once for both pools.  Algorithmic traffic per stored token:
// 2 * row_bytes read + 2 * row_bytes written + 4 bytes of index.
// A slot id outside [0, num_slots) writes nothing (one compare per thread): a wild store would
// be a GPU memory fault rather than a wrong value.  The reference has no such check
// (store_kv_cache.metal:24-30).
#include "msgl_internal.h"

namespace msgl {
namespace {

template <typename VecT>
__global__ __launch_bounds__(256) void store_kv_cache_kernel(
    char* __restrict__ k_cache, char* __restrict__ v_cache, const int32_t* __restrict__ indices,
    const char* __restrict__ k, const char* __restrict__ v, int64_t length,
    int32_t chunks_per_row, int64_t num_slots, int64_t k_cache_stride, int64_t v_cache_stride,
    int64_t k_stride, int64_t v_stride) {
  const int64_t gid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t row = gid / chunks_per_row;
  if (row >= length) return;
  const int64_t off = (gid - row * chunks_per_row) * (int64_t)sizeof(VecT);
  const int64_t slot = indices[row];
  if ((uint64_t)slot >= (uint64_t)num_slots) return;
  const VecT kv = *reinterpret_cast<const VecT*>(k + row * k_stride + off);
  const VecT vv = *reinterpret_cast<const VecT*>(v + row * v_stride + off);
  *reinterpret_cast<VecT*>(k_cache + slot * k_cache_stride + off) = kv;
  *reinterpret_cast<VecT*>(v_cache + slot * v_cache_stride + off) = vv;
}

template <typename VecT>
int launch(char* kc, char* vc, const int32_t* idx, const char* k, const char* v, int64_t length,
           int64_t num_slots, int64_t row_bytes, int64_t kcs, int64_t vcs, int64_t ks, int64_t vs,
           hipStream_t stream) {
  const int64_t chunks = row_bytes / (int64_t)sizeof(VecT);
  const int64_t total = length * chunks;
  const int64_t blocks = (total + 255) / 256;
  if (blocks > 0x7fffffffLL) return MSGL_ERR_SHAPE;
  hipLaunchKernelGGL(store_kv_cache_kernel<VecT>, dim3((unsigned)blocks), dim3(256), 0, stream,
                     kc, vc, idx, k, v, length, (int32_t)chunks, num_slots, kcs, vcs, ks, vs);
  return check_launch();
}

struct alignas(16) B16 { uint32_t w[4]; };
struct alignas(8) B8 { uint32_t w[2]; };

bool aligned_to(int64_t a, const void* p0, const void* p1, const void* p2, const void* p3,
                int64_t s0, int64_t s1, int64_t s2, int64_t s3, int64_t row) {
  auto ok = [a](const void* p) { return (reinterpret_cast<uintptr_t>(p) % (uintptr_t)a) == 0; };
  return ok(p0) && ok(p1) && ok(p2) && ok(p3) && s0 % a == 0 && s1 % a == 0 && s2 % a == 0 &&
         s3 % a == 0 && row % a == 0;
}

}  // namespace

int launch_store_kv_cache(void* k_cache, void* v_cache, const int32_t* indices, const void* k,
                          const void* v, int64_t length, int64_t num_slots, int64_t row_bytes,
                          int64_t k_cache_stride_bytes, int64_t v_cache_stride_bytes,
                          int64_t k_stride_bytes, int64_t v_stride_bytes, hipStream_t stream) {
  if (length == 0 || row_bytes == 0) return MSGL_OK;
  char* kc = static_cast<char*>(k_cache);
  char* vc = static_cast<char*>(v_cache);
  const char* kk = static_cast<const char*>(k);
  const char* vv = static_cast<const char*>(v);
  // widest vector every pointer, stride and the row length allow
  for (int64_t a : {16, 8, 4, 2}) {
    if (!aligned_to(a, kc, vc, kk, vv, k_cache_stride_bytes, v_cache_stride_bytes,
                    k_stride_bytes, v_stride_bytes, row_bytes))
      continue;
    switch (a) {
      case 16:
        return launch<B16>(kc, vc, indices, kk, vv, length, num_slots, row_bytes, k_cache_stride_bytes,
                           v_cache_stride_bytes, k_stride_bytes, v_stride_bytes, stream);
      case 8:
        return launch<B8>(kc, vc, indices, kk, vv, length, num_slots, row_bytes, k_cache_stride_bytes,
                          v_cache_stride_bytes, k_stride_bytes, v_stride_bytes, stream);
      case 4:
        return launch<uint32_t>(kc, vc, indices, kk, vv, length, num_slots, row_bytes,
                                k_cache_stride_bytes, v_cache_stride_bytes, k_stride_bytes,
                                v_stride_bytes, stream);
      default:
        return launch<uint16_t>(kc, vc, indices, kk, vv, length, num_slots, row_bytes,
                                k_cache_stride_bytes, v_cache_stride_bytes, k_stride_bytes,
                                v_stride_bytes, stream);
    }
  }
  return MSGL_ERR_ALIGNMENT;
}

}  // namespace msgl
