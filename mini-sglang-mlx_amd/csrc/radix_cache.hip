// Host-side radix prefix cache behind the C ABI of include/msgl_radix_cache.h: the tree that
// turns token ids into the slot ids of their cached K/V rows.  No device code.
//
// Restates RadixTreeNode / RadixCacheManager / the tree side of HybridRadixCacheManager
// (mini_sglang_mlx/kvcache/radix_manager.py:18-452) and fast_compare_key
// (mini-sglang-mlx-kernel/csrc/fast_compare_key.cpp:9-45) with keys and values held as
// int32 vectors on the host, so that a walk is a few memcmp-like scans instead of one
// interpreter round trip and one array evaluation per node.
#include <algorithm>
#include <cstdint>
#include <cstring>
#include <memory>
#include <queue>
#include <unordered_map>
#include <utility>
#include <vector>

#include "../../include/msgl_radix_cache.h"

namespace {

struct Node {
  std::vector<int32_t> key, value;
  // children in insertion order (the order Python's dict would give); a node rarely has
  // more than a handful, the index map is there for the wide ones (the root)
  std::vector<std::pair<int32_t, int64_t>> children;
  std::unordered_map<int32_t, int64_t> child_index;
  int64_t parent = -1;
  int64_t id = 0;  // creation order
  int64_t timestamp = 0;
  int32_t ref_count = 0;
  int32_t mamba_slot = MSGL_RADIX_NO_SLOT;

  int64_t length() const { return (int64_t)key.size(); }
  bool is_leaf() const { return children.empty(); }
  int64_t child(int32_t tok) const {
    if (children.size() <= 8) {
      for (const auto& c : children)
        if (c.first == tok) return c.second;
      return -1;
    }
    const auto it = child_index.find(tok);
    return it == child_index.end() ? -1 : it->second;
  }
  void set_child(int32_t tok, int64_t node) {
    for (auto& c : children)
      if (c.first == tok) {  // replacing the entry keeps its position, as a dict would
        c.second = node;
        child_index[tok] = node;
        return;
      }
    children.emplace_back(tok, node);
    child_index[tok] = node;
  }
  void erase_child(int32_t tok) {
    for (size_t i = 0; i < children.size(); ++i)
      if (children[i].first == tok) {
        children.erase(children.begin() + (ptrdiff_t)i);
        break;
      }
    child_index.erase(tok);
  }
};

template <typename T>
size_t common_prefix(const T* a, size_t na, const T* b, size_t nb) {
  const size_t n = std::min(na, nb);
  return (size_t)(std::mismatch(a, a + n, b).first - a);
}

class Tree {
 public:
  Tree() {
    Node* root = make_node(0);
    root->ref_count = 1;  // the root is never evicted
  }

  Node* get(int64_t id) {
    const auto it = nodes_.find(id);
    return it == nodes_.end() ? nullptr : it->second.get();
  }
  int64_t node_count() const { return (int64_t)nodes_.size(); }
  int64_t evictable() const { return evictable_; }
  int64_t protected_size() const { return protected_; }

  // radix_manager.py:152-179
  int64_t walk(const int32_t* ids, int64_t n, int64_t now, int64_t* node_out) {
    int64_t prefix = 0;
    Node* node = get(MSGL_RADIX_ROOT);
    while (prefix < n) {
      const int64_t cid = node->child(ids[prefix]);
      if (cid < 0) break;
      node = get(cid);
      const int64_t match = (int64_t)common_prefix(node->key.data(), node->key.size(),
                                                   ids + prefix, (size_t)(n - prefix));
      prefix += match;  // at least one: the child was found by its first token
      if (match != node->length()) {
        node = split_at(node, match);
        break;
      }
      node->timestamp = now;
    }
    *node_out = node->id;
    return prefix;
  }

  // radix_manager.py:140-150 and, with a snapshot, :362-392
  int64_t insert(const int32_t* ids, const int32_t* indices, int64_t n, int32_t mamba_slot,
                 int64_t now, int32_t* slot_to_free) {
    *slot_to_free = MSGL_RADIX_NO_SLOT;
    // the walk may split a node; an insert refused afterwards leaves that split behind, as
    // in the reference, where the assertion fires after _walk
    int64_t nid = 0;
    const int64_t prefix = walk(ids, n, now, &nid);
    Node* node = get(nid);
    if (prefix < n) {
      Node* leaf = make_node(now);
      leaf->key.assign(ids + prefix, ids + n);
      leaf->value.assign(indices + prefix, indices + n);
      leaf->mamba_slot = mamba_slot;
      attach(leaf, node);
      evictable_ += leaf->length();
    } else if (mamba_slot != MSGL_RADIX_NO_SLOT) {
      if (node->id == MSGL_RADIX_ROOT) return MSGL_RADIX_ERR_SNAPSHOT_ON_ROOT;
      if (node->mamba_slot == MSGL_RADIX_NO_SLOT) node->mamba_slot = mamba_slot;
      else *slot_to_free = mamba_slot;
    }
    return prefix;
  }

  // radix_manager.py:108-125
  int32_t lock(int64_t id, bool unlock) {
    Node* node = get(id);
    if (!node) return MSGL_RADIX_ERR_NODE;
    if (unlock) {
      for (Node* c = node; c->id != MSGL_RADIX_ROOT; c = get(c->parent))
        if (c->ref_count <= 0) return MSGL_RADIX_ERR_REF_COUNT;  // checked before anything moves
      for (; node->id != MSGL_RADIX_ROOT; node = get(node->parent)) {
        if (--node->ref_count == 0) {
          evictable_ += node->length();
          protected_ -= node->length();
        }
      }
    } else {
      for (; node->id != MSGL_RADIX_ROOT; node = get(node->parent)) {
        if (node->ref_count == 0) {
          evictable_ -= node->length();
          protected_ += node->length();
        }
        ++node->ref_count;
      }
    }
    return 0;
  }

  // radix_manager.py:191-262.  The evicted values and snapshots are kept until the next call.
  int64_t evict(int64_t size, int64_t num_slots, int64_t* n_slots) {
    evicted_.clear();
    evicted_slots_.clear();
    *n_slots = 0;
    if (size > evictable_) return MSGL_RADIX_ERR_CANNOT_EVICT;
    if (size <= 0 && num_slots <= 0) return 0;
    // least recently used first; among equal timestamps the older node
    using Entry = std::pair<std::pair<int64_t, int64_t>, int64_t>;  // ((timestamp, id), id)
    std::priority_queue<Entry, std::vector<Entry>, std::greater<Entry>> heap;
    for_each_node([&](Node* node) {
      if (node->is_leaf() && node->ref_count == 0) heap.push({{node->timestamp, node->id}, node->id});
    });
    while ((int64_t)evicted_.size() < size || (int64_t)evicted_slots_.size() < num_slots) {
      if (heap.empty()) break;  // only a slot-chasing caller can run the tree dry
      Node* node = get(heap.top().second);
      heap.pop();
      evicted_.insert(evicted_.end(), node->value.begin(), node->value.end());
      evictable_ -= node->length();
      if (node->mamba_slot != MSGL_RADIX_NO_SLOT) evicted_slots_.push_back(node->mamba_slot);
      Node* parent = get(node->parent);
      parent->erase_child(node->key[0]);
      nodes_.erase(node->id);
      // the root is locked for good, so it never enters the heap
      if (parent->is_leaf() && parent->ref_count == 0)
        heap.push({{parent->timestamp, parent->id}, parent->id});
    }
    *n_slots = (int64_t)evicted_slots_.size();
    return (int64_t)evicted_.size();
  }
  const std::vector<int32_t>& evicted() const { return evicted_; }
  const std::vector<int32_t>& evicted_slots() const { return evicted_slots_; }

  // radix_manager.py:347-358
  int64_t find_mamba_ancestor(int64_t id, int64_t depth, int64_t* depth_out) {
    Node* cur = get(id);
    if (!cur) return MSGL_RADIX_ERR_NODE;
    while (cur->id != MSGL_RADIX_ROOT) {
      if (cur->mamba_slot != MSGL_RADIX_NO_SLOT) {
        *depth_out = depth;
        return cur->id;
      }
      depth -= cur->length();
      cur = get(cur->parent);
    }
    *depth_out = 0;
    return MSGL_RADIX_ROOT;
  }

  template <typename F>
  void for_each_node(F&& f) {  // depth first, last child first: the reference's stack order
    std::vector<int64_t> stack{MSGL_RADIX_ROOT};
    while (!stack.empty()) {
      Node* node = get(stack.back());
      stack.pop_back();
      f(node);
      for (const auto& c : node->children) stack.push_back(c.second);
    }
  }

 private:
  Node* make_node(int64_t timestamp) {
    auto node = std::make_unique<Node>();
    node->id = next_id_++;
    node->timestamp = timestamp;
    Node* raw = node.get();
    nodes_.emplace(raw->id, std::move(node));
    return raw;
  }
  void attach(Node* child, Node* parent) {
    child->parent = parent->id;
    parent->set_child(child->key[0], child->id);
  }
  // radix_manager.py:73-87
  Node* split_at(Node* node, int64_t pos) {
    Node* parent = get(node->parent);
    Node* upper = make_node(node->timestamp);
    upper->key.assign(node->key.begin(), node->key.begin() + pos);
    upper->value.assign(node->value.begin(), node->value.begin() + pos);
    upper->ref_count = node->ref_count;
    attach(upper, parent);  // same first token: takes the lower node's place under the parent
    // a snapshot describes the state at the END of the node's key: it stays on the lower part
    node->key.erase(node->key.begin(), node->key.begin() + pos);
    node->value.erase(node->value.begin(), node->value.begin() + pos);
    attach(node, upper);
    return upper;
  }
  std::unordered_map<int64_t, std::unique_ptr<Node>> nodes_;
  int64_t next_id_ = 0;
  int64_t evictable_ = 0, protected_ = 0;
  std::vector<int32_t> evicted_, evicted_slots_;  // what the last evict() took out
};

Tree* as_tree(void* p) { return static_cast<Tree*>(p); }

}  // namespace

extern "C" {

size_t msgl_fast_compare_key(const void* a, size_t na, const void* b, size_t nb, int32_t elem_bytes,
                             int32_t* status) {
  if (status) *status = 0;
  if ((elem_bytes != 4 && elem_bytes != 8) || ((!a || !b) && std::min(na, nb) > 0)) {
    if (status) *status = MSGL_RADIX_ERR_ARGUMENT;
    return 0;
  }
  if (std::min(na, nb) == 0) return 0;
  if (elem_bytes == 8)
    return common_prefix(static_cast<const int64_t*>(a), na, static_cast<const int64_t*>(b), nb);
  return common_prefix(static_cast<const int32_t*>(a), na, static_cast<const int32_t*>(b), nb);
}

void* msgl_radix_create(void) { return new (std::nothrow) Tree(); }
void msgl_radix_destroy(void* tree) { delete as_tree(tree); }

int64_t msgl_radix_walk(void* tree, const int32_t* ids, int64_t n, int64_t now_ns, int64_t* node) {
  if (!tree || !node || n < 0 || (n > 0 && !ids)) return MSGL_RADIX_ERR_ARGUMENT;
  return as_tree(tree)->walk(ids, n, now_ns, node);
}

int64_t msgl_radix_path_values(void* tree, int64_t node, int32_t* out, int64_t cap) {
  if (!tree) return MSGL_RADIX_ERR_ARGUMENT;
  Tree* t = as_tree(tree);
  Node* n = t->get(node);
  if (!n) return MSGL_RADIX_ERR_NODE;
  int64_t total = 0;
  for (Node* c = n; c->id != MSGL_RADIX_ROOT; c = t->get(c->parent)) total += c->length();
  if (out && cap >= total) {
    int64_t end = total;
    for (Node* c = n; c->id != MSGL_RADIX_ROOT; c = t->get(c->parent)) {
      end -= c->length();
      std::memcpy(out + end, c->value.data(), c->value.size() * sizeof(int32_t));
    }
  }
  return total;
}

int64_t msgl_radix_insert(void* tree, const int32_t* ids, const int32_t* indices, int64_t n,
                          int32_t mamba_slot, int64_t now_ns, int32_t* slot_to_free) {
  if (!tree || !slot_to_free || n < 0 || (n > 0 && (!ids || !indices))) return MSGL_RADIX_ERR_ARGUMENT;
  return as_tree(tree)->insert(ids, indices, n, mamba_slot, now_ns, slot_to_free);
}

int32_t msgl_radix_lock(void* tree, int64_t node, int32_t unlock) {
  if (!tree) return MSGL_RADIX_ERR_ARGUMENT;
  return as_tree(tree)->lock(node, unlock != 0);
}

int64_t msgl_radix_evict(void* tree, int64_t size, int64_t num_slots, int64_t* n_slots) {
  if (!tree || !n_slots || size < 0 || num_slots < 0) return MSGL_RADIX_ERR_ARGUMENT;
  return as_tree(tree)->evict(size, num_slots, n_slots);
}

int32_t msgl_radix_evicted(void* tree, int32_t* out_indices, int64_t cap, int32_t* out_slots,
                           int64_t slots_cap) {
  if (!tree) return MSGL_RADIX_ERR_ARGUMENT;
  const std::vector<int32_t>& v = as_tree(tree)->evicted();
  const std::vector<int32_t>& sl = as_tree(tree)->evicted_slots();
  if (cap < (int64_t)v.size() || slots_cap < (int64_t)sl.size() || (!v.empty() && !out_indices) ||
      (!sl.empty() && !out_slots))
    return MSGL_RADIX_ERR_ARGUMENT;
  if (!v.empty()) std::memcpy(out_indices, v.data(), v.size() * sizeof(int32_t));
  if (!sl.empty()) std::memcpy(out_slots, sl.data(), sl.size() * sizeof(int32_t));
  return 0;
}

int32_t msgl_radix_sizes(void* tree, int64_t* evictable, int64_t* protected_size) {
  if (!tree) return MSGL_RADIX_ERR_ARGUMENT;
  if (evictable) *evictable = as_tree(tree)->evictable();
  if (protected_size) *protected_size = as_tree(tree)->protected_size();
  return 0;
}

int32_t msgl_radix_node_info(void* tree, int64_t node, int64_t* parent, int64_t* length,
                             int32_t* ref_count, int64_t* timestamp, int32_t* mamba_slot,
                             int64_t* n_children) {
  if (!tree) return MSGL_RADIX_ERR_ARGUMENT;
  Node* n = as_tree(tree)->get(node);
  if (!n) return MSGL_RADIX_ERR_NODE;
  if (parent) *parent = n->parent;
  if (length) *length = n->length();
  if (ref_count) *ref_count = n->ref_count;
  if (timestamp) *timestamp = n->timestamp;
  if (mamba_slot) *mamba_slot = n->mamba_slot;
  if (n_children) *n_children = (int64_t)n->children.size();
  return 0;
}

int32_t msgl_radix_node_set(void* tree, int64_t node, int32_t field, int64_t value) {
  if (!tree) return MSGL_RADIX_ERR_ARGUMENT;
  Node* n = as_tree(tree)->get(node);
  if (!n) return MSGL_RADIX_ERR_NODE;
  if (field == MSGL_RADIX_FIELD_TIMESTAMP) n->timestamp = value;
  else if (field == MSGL_RADIX_FIELD_MAMBA_SLOT) n->mamba_slot = (int32_t)value;
  else return MSGL_RADIX_ERR_ARGUMENT;
  return 0;
}

int64_t msgl_radix_node_child(void* tree, int64_t node, int32_t first_token) {
  if (!tree) return MSGL_RADIX_ERR_ARGUMENT;
  Node* n = as_tree(tree)->get(node);
  if (!n) return MSGL_RADIX_ERR_NODE;
  return n->child(first_token);
}

int64_t msgl_radix_node_children(void* tree, int64_t node, int32_t* first_tokens, int64_t* ids,
                                 int64_t cap) {
  if (!tree || cap < 0) return MSGL_RADIX_ERR_ARGUMENT;
  Node* n = as_tree(tree)->get(node);
  if (!n) return MSGL_RADIX_ERR_NODE;
  const int64_t count = (int64_t)n->children.size();
  for (int64_t i = 0; i < std::min(count, cap); ++i) {
    if (first_tokens) first_tokens[i] = n->children[(size_t)i].first;
    if (ids) ids[i] = n->children[(size_t)i].second;
  }
  return count;
}

int64_t msgl_radix_node_key_value(void* tree, int64_t node, int32_t* key, int32_t* value, int64_t cap) {
  if (!tree) return MSGL_RADIX_ERR_ARGUMENT;
  Node* n = as_tree(tree)->get(node);
  if (!n) return MSGL_RADIX_ERR_NODE;
  if (cap >= n->length()) {
    if (key) std::memcpy(key, n->key.data(), n->key.size() * sizeof(int32_t));
    if (value) std::memcpy(value, n->value.data(), n->value.size() * sizeof(int32_t));
  }
  return n->length();
}

int64_t msgl_radix_find_mamba_ancestor(void* tree, int64_t node, int64_t depth, int64_t* depth_out) {
  if (!tree || !depth_out) return MSGL_RADIX_ERR_ARGUMENT;
  return as_tree(tree)->find_mamba_ancestor(node, depth, depth_out);
}

int64_t msgl_radix_collect_mamba_slots(void* tree, int32_t* out, int64_t cap) {
  if (!tree || cap < 0) return MSGL_RADIX_ERR_ARGUMENT;
  int64_t count = 0;
  as_tree(tree)->for_each_node([&](Node* n) {
    if (n->mamba_slot == MSGL_RADIX_NO_SLOT) return;
    if (out && count < cap) out[count] = n->mamba_slot;
    ++count;
  });
  return count;
}

int64_t msgl_radix_coldest_snapshot(void* tree, int64_t exclude) {
  if (!tree) return MSGL_RADIX_ERR_ARGUMENT;
  Node* best = nullptr;
  as_tree(tree)->for_each_node([&](Node* n) {
    if (n->mamba_slot == MSGL_RADIX_NO_SLOT || n->id == exclude) return;
    if (!best || n->timestamp < best->timestamp ||
        (n->timestamp == best->timestamp && n->id < best->id))
      best = n;
  });
  return best ? best->id : MSGL_RADIX_ERR_NODE;
}

int64_t msgl_radix_node_count(void* tree) {
  if (!tree) return MSGL_RADIX_ERR_ARGUMENT;
  return as_tree(tree)->node_count();
}

}  // extern "C"
