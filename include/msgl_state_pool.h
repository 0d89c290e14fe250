/*
 * C ABI of the recurrent-state pool's device operations (part of libmsgl_paged_attention.so).
 *
 * Counterpart of the array updates inside mini_sglang_mlx's MambaStatePool
 * (mini_sglang_mlx/kvcache/mamba_pool.py:170-189 copy / copy_batched, :208-213 _zero_slot): the
 * pool that holds, per slot, the state the gated delta-rule kernel (msgl_gdn_state_inplace)
 * updates in place, and whose slots the hybrid radix cache hands out as prefix snapshots.
 * Error codes are those of msgl_paged_attention.h.
 */
#ifndef MSGL_STATE_POOL_H
#define MSGL_STATE_POOL_H

#include <stddef.h>
#include <stdint.h>

#include "msgl_paged_attention.h"

#ifdef __cplusplus
extern "C" {
#endif

/*
 * copy_state_slots -- for every layer l < n_layers and every pair i < n_pairs
 *     slab[l][dst[i]] = slab[l][src[i]]            (bit copy of row_bytes bytes)
 * or, with src == NULL,
 *     slab[l][dst[i]] = 0.
 * `slab` is one device allocation laid out (layers, slots, row): layer l starts at
 * slab + l * layer_stride_bytes, slot s of it at + s * slot_stride_bytes.  `src` and `dst` are
 * device arrays of int32 slot ids.  Replaces `buf[dst] = buf[src]` over a Python loop of layers
 * and buffers (mamba_pool.py:172-176, 186-189) and `buf[slot] = zeros` (:208-213) by one launch
 * per slab.  As there, all sources are meant to be read before any destination is written: the
 * dst ids must be distinct and no slot may be both a source and a destination of one call
 * (pairs with src[i] == dst[i] are skipped); a pair naming a slot outside [0, num_slots) is
 * skipped.
 */
MSGL_API int msgl_copy_state_slots(void* slab, int64_t layer_stride_bytes, int64_t slot_stride_bytes,
                                   int64_t row_bytes, int64_t n_layers, int64_t num_slots,
                                   const int32_t* src, const int32_t* dst, int64_t n_pairs,
                                   void* stream);

#ifdef __cplusplus
}
#endif
#endif /* MSGL_STATE_POOL_H */
