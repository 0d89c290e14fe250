/*
 * msgl_radix_cache.h -- C ABI of the host-side prefix cache that produces the slot ids the
 * paged-attention path consumes (libmsgl_paged_attention.so, same library as
 * msgl_paged_attention.h).
 *
 * Replaces, behind one tree object,
 *   mini_sglang_mlx::fast_compare_key      mini-sglang-mlx-kernel/csrc/fast_compare_key.cpp:9-45
 *   RadixTreeNode, RadixCacheManager       mini_sglang_mlx/kvcache/radix_manager.py:18-275
 *   HybridRadixCacheManager (tree side)    mini_sglang_mlx/kvcache/radix_manager.py:299-452
 * The Python classes of the same names (mini_sglang_amd/kvcache/radix_manager.py) are thin
 * views over these calls.
 *
 * Everything here is host code: pointers are host pointers, nothing touches a GPU.  Token ids
 * and slot ids ("values", "indices") are int32.  A tree is not thread-safe; the reference
 * drives it from its single scheduler thread.
 *
 * Nodes are named by int64 ids that are never reused; the root is MSGL_RADIX_ROOT.  A call
 * that is handed the id of a node that no longer exists returns MSGL_RADIX_ERR_NODE.
 */
#ifndef MSGL_RADIX_CACHE_H_
#define MSGL_RADIX_CACHE_H_

#include <stddef.h>
#include <stdint.h>

#ifndef MSGL_API
#if defined(__GNUC__)
#define MSGL_API __attribute__((visibility("default")))
#else
#define MSGL_API
#endif
#endif

#ifdef __cplusplus
extern "C" {
#endif

#define MSGL_RADIX_ROOT 0
#define MSGL_RADIX_NO_SLOT (-1)          /* "no mamba snapshot" */

#define MSGL_RADIX_ERR_NODE (-1)         /* unknown or evicted node id */
#define MSGL_RADIX_ERR_ARGUMENT (-2)     /* NULL pointer, negative size, buffer too small */
#define MSGL_RADIX_ERR_SNAPSHOT_ON_ROOT (-3) /* insert of an empty remainder with a snapshot at the root */
#define MSGL_RADIX_ERR_REF_COUNT (-4)    /* unlock of a node that is not locked */
#define MSGL_RADIX_ERR_CANNOT_EVICT (-5) /* more pages requested than are evictable */

/*
 * fast_compare_key (fast_compare_key.cpp:9-45): length of the common prefix of two integer
 * arrays, min(na, nb) if one is a prefix of the other.  elem_bytes is 4 (int32) or 8 (int64);
 * anything else returns 0 with *status = MSGL_RADIX_ERR_ARGUMENT (status may be NULL).
 */
MSGL_API size_t msgl_fast_compare_key(const void* a, size_t na, const void* b, size_t nb,
                                      int32_t elem_bytes, int32_t* status);

/* A tree with only its root, which is permanently locked (radix_manager.py:99-106). */
MSGL_API void* msgl_radix_create(void);
MSGL_API void msgl_radix_destroy(void* tree);

/*
 * RadixCacheManager._walk (radix_manager.py:152-179).  Follows `ids` from the root; a node
 * matched only in part is split at the match (the new upper node inherits timestamp and
 * ref_count, a snapshot stays on the lower node, :73-87); every fully matched node gets
 * timestamp `now_ns`.  Returns the matched length, *node = deepest matched node.
 */
MSGL_API int64_t msgl_radix_walk(void* tree, const int32_t* ids, int64_t n, int64_t now_ns,
                                 int64_t* node);

/*
 * Values along the path root -> node, in order (the concatenation of match_prefix, :127-138).
 * Returns their total length; writes them when cap is large enough, else writes nothing.
 */
MSGL_API int64_t msgl_radix_path_values(void* tree, int64_t node, int32_t* out, int64_t cap);

/*
 * insert_prefix (:140-150, hybrid :362-392).  Walks `ids`; the unmatched remainder, if any,
 * becomes a new leaf holding indices[prefix_len:] and `mamba_slot` (MSGL_RADIX_NO_SLOT for
 * none).  When everything was cached already the deepest node adopts the snapshot if it has
 * none; otherwise *slot_to_free = mamba_slot (the caller returns it to its pool), else
 * MSGL_RADIX_NO_SLOT.  Returns the length that was already cached.
 */
MSGL_API int64_t msgl_radix_insert(void* tree, const int32_t* ids, const int32_t* indices,
                                   int64_t n, int32_t mamba_slot, int64_t now_ns,
                                   int32_t* slot_to_free);

/* lock_handle (:108-125): ref counts and the evictable / protected sizes along node -> root. */
MSGL_API int32_t msgl_radix_lock(void* tree, int64_t node, int32_t unlock);

/*
 * _evict_leaves (:191-237): evicts unlocked leaves, least recently used first (ties: the
 * older node first; the reference leaves ties to its heap), until `size` pages and
 * `num_slots` snapshots are reclaimed, parents that become unlocked leaves included.
 * Requires size <= evictable size (evict, :239-247), else MSGL_RADIX_ERR_CANNOT_EVICT and
 * nothing changes.  Running out of leaves while chasing slots is not an error.
 * Returns the number of evicted values (whole leaves: it may exceed `size`), *n_slots = the
 * number of snapshots that came with them.  The tree keeps both lists until its next evict;
 * msgl_radix_evicted copies them out, values in eviction order.
 */
MSGL_API int64_t msgl_radix_evict(void* tree, int64_t size, int64_t num_slots, int64_t* n_slots);
MSGL_API int32_t msgl_radix_evicted(void* tree, int32_t* out_indices, int64_t cap,
                                    int32_t* out_slots, int64_t slots_cap);

/* size_info (:267-272). */
MSGL_API int32_t msgl_radix_sizes(void* tree, int64_t* evictable, int64_t* protected_size);

/* Node fields (RadixTreeNode, :18-66).  Any out pointer may be NULL. */
MSGL_API int32_t msgl_radix_node_info(void* tree, int64_t node, int64_t* parent, int64_t* length,
                                      int32_t* ref_count, int64_t* timestamp,
                                      int32_t* mamba_slot, int64_t* n_children);
#define MSGL_RADIX_FIELD_TIMESTAMP 0
#define MSGL_RADIX_FIELD_MAMBA_SLOT 1
MSGL_API int32_t msgl_radix_node_set(void* tree, int64_t node, int32_t field, int64_t value);
/* child whose key starts with first_token, or MSGL_RADIX_ERR_NODE */
MSGL_API int64_t msgl_radix_node_child(void* tree, int64_t node, int32_t first_token);
/* children in insertion order; returns their count, fills up to cap entries */
MSGL_API int64_t msgl_radix_node_children(void* tree, int64_t node, int32_t* first_tokens,
                                          int64_t* ids, int64_t cap);
/* key and value of the node itself; returns its length, fills when cap is large enough */
MSGL_API int64_t msgl_radix_node_key_value(void* tree, int64_t node, int32_t* key, int32_t* value,
                                           int64_t cap);

/*
 * _find_mamba_ancestor (:347-358): nearest node on the way up from `node` (matched depth
 * `depth`) that holds a snapshot; the root with *depth_out = 0 if there is none.
 */
MSGL_API int64_t msgl_radix_find_mamba_ancestor(void* tree, int64_t node, int64_t depth,
                                                int64_t* depth_out);
/* collect_mamba_slots (:418-427): returns the count, fills up to cap entries. */
MSGL_API int64_t msgl_radix_collect_mamba_slots(void* tree, int32_t* out, int64_t cap);
/*
 * coldest_snapshot_node (:429-446): least recently used node that holds a snapshot, `exclude`
 * itself skipped (MSGL_RADIX_ERR_NODE for none); returns MSGL_RADIX_ERR_NODE if there is none.
 */
MSGL_API int64_t msgl_radix_coldest_snapshot(void* tree, int64_t exclude);
/* number of live nodes, the root included */
MSGL_API int64_t msgl_radix_node_count(void* tree);

#ifdef __cplusplus
}
#endif
#endif /* MSGL_RADIX_CACHE_H_ */
