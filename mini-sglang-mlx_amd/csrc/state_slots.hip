// Slot-to-slot copies and zero fills of a recurrent-state pool, all layers in one launch.
// Restates what MambaStatePool.copy / copy_batched / _zero_slot do to their buffers
// (mini_sglang_mlx/kvcache/mamba_pool.py:170-189, 208-213: `buf[dst] = buf[src]` per layer and
// buffer, `buf[slot] = 0`), on a slab laid out (layers, slots, row): the reference issues two
// array updates per layer, this is one launch per slab.
//
// HBM-bound byte mover.  A slot's row of one layer (2 MiB for a 32 x 128 x 128 fp32 state) is
// cut into 16 KiB pieces; a workgroup moves one piece with 16-byte accesses (narrower when the
// row length or the base pointer demand it).  Algorithmic traffic per (pair, layer): row_bytes
// read + row_bytes written (fill: written only) + 8 bytes of slot ids.
#include "msgl_internal.h"

namespace msgl {
namespace {

constexpr int kPieceBytes = 16384;

struct alignas(16) B16 { uint32_t w[4]; };

// grid: (pieces per row, pairs, layers).  A pair whose slot id lies outside [0, num_slots) is
// skipped: ids come from device memory and cannot be checked on the host.
template <typename VecT, bool FILL>
__global__ __launch_bounds__(256) void state_slots_kernel(char* __restrict__ base, int64_t layer_stride,
                                                          int64_t slot_stride, int64_t row_bytes,
                                                          int64_t num_slots,
                                                          const int32_t* __restrict__ src,
                                                          const int32_t* __restrict__ dst) {
  const int pair = blockIdx.y;
  const int64_t d = dst[pair];
  const int64_t s = FILL ? 0 : src[pair];
  if (d < 0 || d >= num_slots || s < 0 || s >= num_slots || (!FILL && s == d)) return;
  char* layer = base + (int64_t)blockIdx.z * layer_stride;
  const int64_t begin = (int64_t)blockIdx.x * kPieceBytes;
  const int64_t end = min(begin + (int64_t)kPieceBytes, row_bytes);
  char* to = layer + d * slot_stride;
  const char* from = layer + s * slot_stride;
  VecT zero{};
  for (int64_t off = begin + (int64_t)threadIdx.x * (int64_t)sizeof(VecT); off < end;
       off += 256 * (int64_t)sizeof(VecT)) {
    if constexpr (FILL) *reinterpret_cast<VecT*>(to + off) = zero;
    else *reinterpret_cast<VecT*>(to + off) = *reinterpret_cast<const VecT*>(from + off);
  }
}

template <typename VecT>
int launch(char* base, int64_t layer_stride, int64_t slot_stride, int64_t row_bytes, int64_t n_layers,
           int64_t num_slots, const int32_t* src, const int32_t* dst, int64_t n_pairs,
           hipStream_t stream) {
  const int64_t pieces = (row_bytes + kPieceBytes - 1) / kPieceBytes;
  if (pieces > 0x7fffffffLL || n_pairs > 65535 || n_layers > 65535) return MSGL_ERR_SHAPE;
  const dim3 grid((unsigned)pieces, (unsigned)n_pairs, (unsigned)n_layers);
  if (src)
    hipLaunchKernelGGL((state_slots_kernel<VecT, false>), grid, dim3(256), 0, stream, base, layer_stride,
                       slot_stride, row_bytes, num_slots, src, dst);
  else
    hipLaunchKernelGGL((state_slots_kernel<VecT, true>), grid, dim3(256), 0, stream, base, layer_stride,
                       slot_stride, row_bytes, num_slots, src, dst);
  return check_launch();
}

}  // namespace

int launch_state_slots(void* base, int64_t layer_stride, int64_t slot_stride, int64_t row_bytes,
                       int64_t n_layers, int64_t num_slots, const int32_t* src, const int32_t* dst,
                       int64_t n_pairs, hipStream_t stream) {
  char* b = static_cast<char*>(base);
  const auto all = [&](int64_t a) {
    return reinterpret_cast<uintptr_t>(b) % (uintptr_t)a == 0 && layer_stride % a == 0 &&
           slot_stride % a == 0 && row_bytes % a == 0;
  };
  if (all(16)) return launch<B16>(b, layer_stride, slot_stride, row_bytes, n_layers, num_slots, src, dst, n_pairs, stream);
  if (all(4)) return launch<uint32_t>(b, layer_stride, slot_stride, row_bytes, n_layers, num_slots, src, dst, n_pairs, stream);
  if (all(2)) return launch<uint16_t>(b, layer_stride, slot_stride, row_bytes, n_layers, num_slots, src, dst, n_pairs, stream);
  return launch<uint8_t>(b, layer_stride, slot_stride, row_bytes, n_layers, num_slots, src, dst, n_pairs, stream);
}

}  // namespace msgl
