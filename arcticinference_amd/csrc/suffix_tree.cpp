// Suffix-tree speculation (SuffixDecoding), CPU.
//
// Replaces the reference's SuffixTree (csrc/suffix_decoding/suffix_tree.{h,cc}, with its Int32Map,
// csrc/suffix_decoding/int32_map.h) behind the C ABI of include/arctic_suffix.h.  Same tree, same
// drafts; different machinery:
//
//  * Nodes, child buckets and endpoint records live in three arenas and refer to each other by 32-bit
//    index (the reference uses heap nodes, unique_ptr children maps and shared_ptr groups).
//  * One open-addressing table per tree maps (parent, first token) -> child; the reference keeps a hash
//    map inside every node.  The endpoints of a node (which suffixes end there) are a short linked list
//    of records; a suffix that is still growing carries its record along, so the hot path never searches
//    for it, and only a node that collects many endpoints gets them indexed in a second table.
//  * Sequences sit in numbered slots; nodes and endpoint records name a slot, not a sequence id, so
//    reading a node's tokens takes no hash lookup.
//  * The children of a node are kept in decreasing order of count as a list of buckets, one per
//    distinct count, each holding its nodes in order (the O(1) frequency-list layout).  The reference
//    keeps one sibling list plus "group" records that point at the first node of each run of equal
//    counts; where a node lands among equal counts after a count changes by one is the same in both,
//    and that order decides which continuation a draft follows, so it is part of the contract:
//      new child (count 1)            -> last of all children
//      count c -> c+1, node was first of the c-run   -> first of the (c+1)-run
//      count c -> c+1, node was not first            -> last of the (c+1)-run
//      count c -> c-1                                -> first of the (c-1)-run
//    (suffix_tree.cc:31-296).
#include "../../include/arctic_suffix.h"

#include <algorithm>
#include <cstdio>
#include <cstring>
#include <deque>
#include <new>
#include <queue>
#include <string>
#include <unordered_map>
#include <utility>
#include <vector>

namespace {

constexpr uint32_t NIL = 0xffffffffu;

// uint64 -> uint32, linear probing over a power-of-two table, deletion by backward shift.
class FlatMap {
 public:
  FlatMap() : slots_(16), mask_(15) {}

  uint32_t find(uint64_t key) const {
    for (size_t i = hash(key) & mask_;; i = (i + 1) & mask_) {
      const Slot &s = slots_[i];
      if (!s.used) return NIL;
      if (s.key == key) return s.value;
    }
  }

  void set(uint64_t key, uint32_t value) {
    if ((size_ + 1) * 10 > slots_.size() * 7) grow();
    for (size_t i = hash(key) & mask_;; i = (i + 1) & mask_) {
      Slot &s = slots_[i];
      if (!s.used) {
        s.key = key;
        s.value = value;
        s.used = 1;
        ++size_;
        return;
      }
      if (s.key == key) {
        s.value = value;
        return;
      }
    }
  }

  bool erase(uint64_t key) {
    size_t i = hash(key) & mask_;
    for (;; i = (i + 1) & mask_) {
      if (!slots_[i].used) return false;
      if (slots_[i].key == key) break;
    }
    // close the gap: pull back every later entry of the run whose home slot is not after the gap
    size_t gap = i;
    for (size_t j = (i + 1) & mask_; slots_[j].used; j = (j + 1) & mask_) {
      const size_t home = hash(slots_[j].key) & mask_;
      const bool between = gap <= j ? (gap < home && home <= j) : (gap < home || home <= j);
      if (!between) {
        slots_[gap] = slots_[j];
        gap = j;
      }
    }
    slots_[gap].used = 0;
    --size_;
    return true;
  }

  size_t size() const { return size_; }
  size_t bytes() const { return slots_.capacity() * sizeof(Slot); }

 private:
  struct Slot {
    uint64_t key = 0;
    uint32_t value = 0;
    uint32_t used = 0;
  };
  static size_t hash(uint64_t k) {
    k ^= k >> 33;
    k *= 0xff51afd7ed558ccdULL;
    k ^= k >> 33;
    k *= 0xc4ceb9fe1a85ec53ULL;
    k ^= k >> 33;
    return (size_t)k;
  }
  void grow() {
    std::vector<Slot> old;
    old.swap(slots_);
    slots_.assign(old.size() * 2, Slot());
    mask_ = slots_.size() - 1;
    size_ = 0;
    for (const Slot &s : old)
      if (s.used) set(s.key, s.value);
  }
  std::vector<Slot> slots_;
  size_t size_ = 0;
  size_t mask_;
};

struct Node {
  int64_t count = 0;          // suffixes that end at or pass through this node
  int32_t token = 0;          // first token of the node's label
  int32_t length = 0;         // tokens in the label
  int32_t ref_seq = 0;        // the label is tokens [ref_idx, ref_idx + length) of the sequence in slot ref_seq
  int32_t ref_idx = -1;
  uint32_t parent = NIL;
  uint32_t first_bucket = NIL;  // children, highest count first
  uint32_t last_bucket = NIL;
  uint32_t bucket = NIL;        // the bucket of the parent this node sits in
  uint32_t next = NIL;          // neighbours inside that bucket
  uint32_t prev = NIL;
  uint32_t first_endpoint = NIL;
  uint32_t num_children = 0;
  uint32_t num_endpoints = 0;
  bool endpoints_indexed = false;  // true once the node held more than kIndexAbove endpoints
};

constexpr uint32_t kIndexAbove = 16;

// The children of one node that share one count, in order.
struct Bucket {
  int64_t count = 0;
  uint32_t head = NIL;
  uint32_t tail = NIL;
  uint32_t next = NIL;  // bucket with the next lower count
  uint32_t prev = NIL;
};

// "A suffix of the sequence in slot seq ends in this node, at position end of the sequence."
struct Endpoint {
  uint32_t node = NIL;
  int32_t seq = 0;
  int32_t end = 0;
  uint32_t next = NIL;  // other endpoints of the same node
  uint32_t prev = NIL;
};

// Where one of the last max_depth suffixes of a sequence currently ends, and its endpoint record.
struct Growing {
  uint32_t node;
  uint32_t endpoint;
};

struct Sequence {
  int32_t id = 0;
  std::vector<int32_t> tokens;
  std::deque<Growing> active;  // oldest (deepest) first
};

struct Draft {
  std::vector<int32_t> token_ids;
  std::vector<int32_t> parents;
  std::vector<float> probs;
  float score = 0.0f;
  int match_len = 0;
};

template <typename T>
class Arena {
 public:
  uint32_t make() {
    if (!free_.empty()) {
      const uint32_t i = free_.back();
      free_.pop_back();
      items_[i] = T();
      return i;
    }
    items_.emplace_back();
    return (uint32_t)(items_.size() - 1);
  }
  void release(uint32_t i) { free_.push_back(i); }
  T &operator[](uint32_t i) { return items_[i]; }
  const T &operator[](uint32_t i) const { return items_[i]; }
  size_t live() const { return items_.size() - free_.size(); }
  size_t bytes() const { return items_.capacity() * sizeof(T) + free_.capacity() * sizeof(uint32_t); }

 private:
  std::vector<T> items_;
  std::vector<uint32_t> free_;
};

inline uint64_t pair_key(uint32_t a, int32_t b) { return ((uint64_t)a << 32) | (uint32_t)b; }

}  // namespace

struct arctic_suffix_tree {
  explicit arctic_suffix_tree(int max_depth) : max_depth_(max_depth) { root_ = nodes_.make(); }
  ~arctic_suffix_tree() {
    for (Sequence *s : slots_) delete s;
  }
  arctic_suffix_tree(const arctic_suffix_tree &) = delete;
  arctic_suffix_tree &operator=(const arctic_suffix_tree &) = delete;

  int num_seqs() const { return (int)slot_of_.size(); }
  void append(int seq_id, int32_t token);
  void remove(int seq_id);
  Draft speculate(const int32_t *context, int64_t n, int max_spec_tokens, float max_spec_factor,
                  float max_spec_offset, float min_token_prob, bool use_tree_spec);
  std::string check_integrity();
  size_t estimate_memory() const;

 private:
  // ---- sequences ---------------------------------------------------------------------------------
  int32_t slot_for(int seq_id) {
    auto it = slot_of_.find(seq_id);
    if (it != slot_of_.end()) return it->second;
    int32_t slot;
    if (!free_slots_.empty()) {
      slot = free_slots_.back();
      free_slots_.pop_back();
    } else {
      slot = (int32_t)slots_.size();
      slots_.push_back(nullptr);
    }
    slots_[slot] = new Sequence();
    slots_[slot]->id = seq_id;
    slot_of_.emplace(seq_id, slot);
    return slot;
  }
  const int32_t *label(uint32_t node) const {
    const Node &n = nodes_[node];
    return slots_[n.ref_seq]->tokens.data() + n.ref_idx;
  }

  // ---- children table --------------------------------------------------------------------------
  uint32_t child_of(uint32_t parent, int32_t token) const { return children_.find(pair_key(parent, token)); }
  // the same answer without touching the table where the node itself tells it
  uint32_t find_child(uint32_t parent, int32_t token) const {
    const Node &p = nodes_[parent];
    if (p.num_children == 0) return NIL;
    if (p.num_children == 1) {
      const uint32_t only = buckets_[p.first_bucket].head;
      return nodes_[only].token == token ? only : NIL;
    }
    return child_of(parent, token);
  }
  void set_child(uint32_t parent, int32_t token, uint32_t child) { children_.set(pair_key(parent, token), child); }
  void drop_child_key(uint32_t parent, int32_t token) { children_.erase(pair_key(parent, token)); }

  // ---- endpoints -------------------------------------------------------------------------------
  uint32_t find_endpoint(uint32_t node, int32_t slot) const {
    const Node &n = nodes_[node];
    if (n.endpoints_indexed) return endpoint_index_.find(pair_key(node, slot));
    for (uint32_t e = n.first_endpoint; e != NIL; e = endpoints_[e].next)
      if (endpoints_[e].seq == slot) return e;
    return NIL;
  }
  void link_endpoint(uint32_t e, uint32_t node) {
    Endpoint &r = endpoints_[e];
    Node &n = nodes_[node];
    r.node = node;
    r.prev = NIL;
    r.next = n.first_endpoint;
    if (r.next != NIL) endpoints_[r.next].prev = e;
    n.first_endpoint = e;
    n.num_endpoints++;
    if (n.endpoints_indexed) {
      endpoint_index_.set(pair_key(node, r.seq), e);
    } else if (n.num_endpoints > kIndexAbove) {
      n.endpoints_indexed = true;
      for (uint32_t x = n.first_endpoint; x != NIL; x = endpoints_[x].next)
        endpoint_index_.set(pair_key(node, endpoints_[x].seq), x);
    }
  }
  void unlink_endpoint(uint32_t e) {
    const Endpoint &r = endpoints_[e];
    Node &n = nodes_[r.node];
    if (r.prev != NIL) endpoints_[r.prev].next = r.next; else n.first_endpoint = r.next;
    if (r.next != NIL) endpoints_[r.next].prev = r.prev;
    n.num_endpoints--;
    if (n.endpoints_indexed) endpoint_index_.erase(pair_key(r.node, r.seq));
  }
  // a record for a suffix that (the caller knows) has none in `node` yet
  uint32_t add_endpoint(uint32_t node, int32_t slot, int32_t end) {
    const uint32_t e = endpoints_.make();
    endpoints_[e].seq = slot;
    endpoints_[e].end = end;
    link_endpoint(e, node);
    return e;
  }
  void drop_endpoint(uint32_t e) {
    unlink_endpoint(e);
    endpoints_.release(e);
  }
  // The growing suffix `g` now ends in `node` at `end`.  A node holds one record per sequence: if an
  // earlier suffix of the same sequence already ended there (possible only at the depth limit, where
  // suffixes stop growing), that record is taken over, as assigning endpoints[seq] does in the reference.
  void move_endpoint(Growing &g, uint32_t node, int32_t end, bool may_exist) {
    if (may_exist) {
      const uint32_t there = find_endpoint(node, endpoints_[g.endpoint].seq);
      if (there != NIL) {
        drop_endpoint(g.endpoint);
        g.endpoint = there;
        endpoints_[there].end = end;
        g.node = node;
        return;
      }
    }
    unlink_endpoint(g.endpoint);
    endpoints_[g.endpoint].end = end;
    link_endpoint(g.endpoint, node);
    g.node = node;
  }
  void drop_all_endpoints(uint32_t node) {
    Node &n = nodes_[node];
    for (uint32_t e = n.first_endpoint; e != NIL;) {
      const uint32_t next = endpoints_[e].next;
      if (n.endpoints_indexed) endpoint_index_.erase(pair_key(node, endpoints_[e].seq));
      endpoints_.release(e);
      e = next;
    }
    n.first_endpoint = NIL;
    n.num_endpoints = 0;
  }

  // ---- ordered children ------------------------------------------------------------------------
  uint32_t head_child(uint32_t node) const {
    const uint32_t b = nodes_[node].first_bucket;
    return b == NIL ? NIL : buckets_[b].head;
  }
  uint32_t next_sibling(uint32_t node) const {
    const Node &n = nodes_[node];
    if (n.next != NIL) return n.next;
    const uint32_t b = buckets_[n.bucket].next;
    return b == NIL ? NIL : buckets_[b].head;
  }
  // a fresh bucket holding only `node`, linked between buckets `before` and `after` of `parent`
  void bucket_alone(uint32_t parent, uint32_t node, uint32_t before, uint32_t after) {
    const uint32_t b = buckets_.make();
    Bucket &k = buckets_[b];
    k.count = nodes_[node].count;
    k.head = k.tail = node;
    k.prev = before;
    k.next = after;
    if (before != NIL) buckets_[before].next = b; else nodes_[parent].first_bucket = b;
    if (after != NIL) buckets_[after].prev = b; else nodes_[parent].last_bucket = b;
    Node &n = nodes_[node];
    n.bucket = b;
    n.prev = n.next = NIL;
  }
  void bucket_push_front(uint32_t b, uint32_t node) {
    Node &n = nodes_[node];
    n.bucket = b;
    n.prev = NIL;
    n.next = buckets_[b].head;
    nodes_[n.next].prev = node;
    buckets_[b].head = node;
  }
  void bucket_push_back(uint32_t b, uint32_t node) {
    Node &n = nodes_[node];
    n.bucket = b;
    n.next = NIL;
    n.prev = buckets_[b].tail;
    nodes_[n.prev].next = node;
    buckets_[b].tail = node;
  }
  // take `node` out of its parent's order; an emptied bucket disappears
  void unlink(uint32_t node) {
    Node &n = nodes_[node];
    const uint32_t b = n.bucket;
    Bucket &k = buckets_[b];
    if (n.prev != NIL) nodes_[n.prev].next = n.next; else k.head = n.next;
    if (n.next != NIL) nodes_[n.next].prev = n.prev; else k.tail = n.prev;
    if (k.head == NIL) {
      Node &p = nodes_[n.parent];
      if (k.prev != NIL) buckets_[k.prev].next = k.next; else p.first_bucket = k.next;
      if (k.next != NIL) buckets_[k.next].prev = k.prev; else p.last_bucket = k.prev;
      buckets_.release(b);
    }
    n.bucket = n.prev = n.next = NIL;
  }
  // `fresh` (same parent, same count) takes the exact place of `old`
  void take_place(uint32_t old, uint32_t fresh) {
    Node &o = nodes_[old];
    Node &f = nodes_[fresh];
    f.bucket = o.bucket;
    f.prev = o.prev;
    f.next = o.next;
    Bucket &k = buckets_[o.bucket];
    if (o.prev != NIL) nodes_[o.prev].next = fresh; else k.head = fresh;
    if (o.next != NIL) nodes_[o.next].prev = fresh; else k.tail = fresh;
    o.bucket = o.prev = o.next = NIL;
  }
  void add_last_child(uint32_t parent, uint32_t node) {  // node.count == 1
    const uint32_t last = nodes_[parent].last_bucket;
    if (last != NIL && buckets_[last].count == 1) bucket_push_back(last, node);
    else bucket_alone(parent, node, last, NIL);
    nodes_[parent].num_children++;
  }
  void count_up(uint32_t node);
  void count_down(uint32_t node);

  void release_subtree(uint32_t top);
  bool match(const int32_t *context, int64_t n, uint32_t &node, int &idx) const;
  Draft draft_path(uint32_t node, int idx, int max_tokens, float min_token_prob) const;
  Draft draft_tree(uint32_t node, int idx, int max_tokens, float min_token_prob) const;

  int max_depth_;
  uint32_t root_;
  Arena<Node> nodes_;
  Arena<Bucket> buckets_;
  Arena<Endpoint> endpoints_;
  FlatMap children_;
  FlatMap endpoint_index_;                        // (node, slot) -> record, for nodes with many endpoints
  std::vector<Sequence *> slots_;                 // sequences by slot; nullptr = free
  std::vector<int32_t> free_slots_;
  std::unordered_map<int32_t, int32_t> slot_of_;  // sequence id -> slot
};

// count c -> c+1 (suffix_tree.cc:171-215)
void arctic_suffix_tree::count_up(uint32_t node) {
  Node &n = nodes_[node];
  const uint32_t b = n.bucket;
  Bucket &k = buckets_[b];
  const uint32_t above = k.prev;
  const bool first = k.head == node;
  const bool alone = first && k.tail == node;
  const bool joins = above != NIL && buckets_[above].count == n.count + 1;
  if (alone && !joins) {  // nothing to reorder
    n.count += 1;
    k.count += 1;
    return;
  }
  const uint32_t parent = n.parent;
  unlink(node);
  nodes_[node].count += 1;
  if (joins) {
    if (first) bucket_push_front(above, node); else bucket_push_back(above, node);
  } else {
    bucket_alone(parent, node, above, b);  // b survives: it holds other nodes
  }
}

// count c -> c-1, c >= 2 (suffix_tree.cc:217-294)
void arctic_suffix_tree::count_down(uint32_t node) {
  Node &n = nodes_[node];
  const uint32_t b = n.bucket;
  Bucket &k = buckets_[b];
  const uint32_t below = k.next;
  const bool alone = k.head == node && k.tail == node;
  const bool joins = below != NIL && buckets_[below].count == n.count - 1;
  if (alone && !joins) {
    n.count -= 1;
    k.count -= 1;
    return;
  }
  const uint32_t parent = n.parent;
  unlink(node);
  nodes_[node].count -= 1;
  if (joins) bucket_push_front(below, node);
  else bucket_alone(parent, node, b, below);  // b survives here: it was not alone
}

// Free `top` and everything below it.  `top` must already be out of its parent's order and table.
void arctic_suffix_tree::release_subtree(uint32_t top) {
  std::vector<uint32_t> todo{top};
  while (!todo.empty()) {
    const uint32_t node = todo.back();
    todo.pop_back();
    for (uint32_t b = nodes_[node].first_bucket; b != NIL;) {
      for (uint32_t c = buckets_[b].head; c != NIL; c = nodes_[c].next) {
        drop_child_key(node, nodes_[c].token);
        todo.push_back(c);
      }
      const uint32_t next = buckets_[b].next;
      buckets_.release(b);
      b = next;
    }
    drop_all_endpoints(node);
    nodes_.release(node);
  }
}

// suffix_tree.cc:297-490
void arctic_suffix_tree::append(int seq_id, int32_t token) {
  const int32_t slot = slot_for(seq_id);
  Sequence &seq = *slots_[slot];
  // a new suffix starts at the root
  seq.active.push_back(Growing{root_, add_endpoint(root_, slot, (int32_t)seq.tokens.size())});
  nodes_[root_].count += 1;
  if (seq.active.size() > (size_t)max_depth_) seq.active.pop_front();  // keeps its endpoint: a truncated suffix
  seq.tokens.push_back(token);
  const int32_t len = (int32_t)seq.tokens.size();
  // only the oldest suffix of a full window reaches the depth limit, where records of the same
  // sequence can already be waiting
  const bool window_full = seq.active.size() == (size_t)max_depth_;

  bool oldest = true;
  for (Growing &g : seq.active) {
    const bool at_limit = oldest && window_full;
    oldest = false;
    const uint32_t node = g.node;
    if (nodes_[node].count == 1 && node != root_) {
      // only this suffix ends here and nothing passes through: a leaf, which grows by one token
      nodes_[node].length += 1;
      endpoints_[g.endpoint].end += 1;
      continue;
    }
    const uint32_t child = find_child(node, token);
    if (child == NIL) {
      {
        const uint32_t fresh = nodes_.make();
        Node &f = nodes_[fresh];
        f.count = 1;
        f.token = token;
        f.length = 1;
        f.ref_seq = slot;
        f.ref_idx = len - 1;
        f.parent = node;
        set_child(node, token, fresh);
        move_endpoint(g, fresh, len, false);
        add_last_child(node, fresh);
      }
    } else if (nodes_[node].count == nodes_[child].count + 1 && node != root_) {
      // this suffix is the only one that ends here; every other one continues into the single child
      Node &n = nodes_[node];
      Node &c = nodes_[child];
      if (c.length == 1) {
        // with the new token the suffix covers the child entirely: the two nodes become one
        c.count += 1;  // now equal to the node's count, whose place it takes
        c.token = n.token;
        c.length = n.length + 1;
        c.ref_seq = slot;
        c.ref_idx = len - c.length;
        c.parent = n.parent;
        buckets_.release(n.first_bucket);
        take_place(node, child);
        drop_child_key(node, token);
        set_child(c.parent, c.token, child);  // overwrites the entry that led to `node`
        move_endpoint(g, child, len, at_limit);
        nodes_.release(node);                 // its only endpoint was this suffix's, now moved
      } else {
        // the node takes over the child's first token
        n.length += 1;
        endpoints_[g.endpoint].end += 1;
        n.ref_seq = slot;
        n.ref_idx = len - n.length;
        c.length -= 1;
        c.ref_idx += 1;
        const int32_t first = slots_[c.ref_seq]->tokens[c.ref_idx];
        if (first != token) {
          drop_child_key(node, token);
          set_child(node, first, child);
        }
        c.token = first;
      }
    } else {
      // the suffix moves down into the child
      if (nodes_[child].length == 1) {
        move_endpoint(g, child, len, at_limit);
        count_up(child);
      } else {
        // the child's first token splits off into a node of its own, which the suffix enters
        const uint32_t mid = nodes_.make();
        Node &c = nodes_[child];
        Node &m = nodes_[mid];
        m.count = c.count;
        m.token = token;
        m.length = 1;
        m.ref_seq = slot;
        m.ref_idx = len - 1;
        m.parent = node;
        take_place(child, mid);
        set_child(node, token, mid);
        c.length -= 1;
        c.ref_idx += 1;
        c.token = slots_[c.ref_seq]->tokens[c.ref_idx];
        c.parent = mid;
        set_child(mid, c.token, child);
        bucket_alone(mid, child, NIL, NIL);
        m.num_children = 1;
        move_endpoint(g, mid, len, false);
        count_up(mid);
      }
    }
  }
}

// suffix_tree.cc:500-581
void arctic_suffix_tree::remove(int seq_id) {
  auto found = slot_of_.find(seq_id);
  if (found == slot_of_.end()) return;
  const int32_t slot = found->second;
  const std::vector<int32_t> &seq = slots_[slot]->tokens;
  const int32_t len = (int32_t)seq.size();
  std::vector<uint32_t> path;
  for (int32_t start = 0; start < len; ++start) {
    uint32_t node = root_;
    nodes_[root_].count -= 1;
    int32_t idx = start;
    path.clear();
    while (idx < len) {
      const int32_t token = seq[idx];
      const uint32_t child = find_child(node, token);
      if (child == NIL) break;
      if (nodes_[child].count > 1) {
        count_down(child);
      } else {
        // only this suffix went there
        unlink(child);
        drop_child_key(node, token);
        nodes_[node].num_children--;
        release_subtree(child);
        break;
      }
      const uint32_t e = find_endpoint(child, slot);
      if (e != NIL) drop_endpoint(e);
      idx += nodes_[child].length;
      node = child;
      path.push_back(node);
    }
    // a node left with one child that carries every suffix of the node is folded into that child
    if (node != root_ && nodes_[node].num_children == 1) {
      const uint32_t child = head_child(node);
      if (nodes_[node].count == nodes_[child].count) {
        Node &n = nodes_[node];
        Node &c = nodes_[child];
        drop_child_key(node, c.token);
        c.token = n.token;
        c.length += n.length;
        c.ref_idx -= n.length;
        c.parent = n.parent;
        buckets_.release(n.first_bucket);
        take_place(node, child);
        set_child(c.parent, c.token, child);
        drop_all_endpoints(node);
        nodes_.release(node);
        path.back() = node = child;
      }
    }
    // nodes on the path whose label refers to the departing sequence borrow the position of a suffix
    // that ends in some leaf below
    uint32_t leaf = node;
    int32_t distance = 0;
    for (uint32_t c = head_child(leaf); c != NIL; c = head_child(leaf)) {
      leaf = c;
      distance += nodes_[leaf].length;
    }
    if (nodes_[leaf].num_endpoints == 0 || find_endpoint(leaf, slot) != NIL) continue;  // comes by again later
    const Endpoint &ref = endpoints_[nodes_[leaf].first_endpoint];
    const int32_t ref_seq = ref.seq;
    int32_t ref_idx = ref.end - distance;
    while (!path.empty()) {
      Node &n = nodes_[path.back()];
      path.pop_back();
      ref_idx -= n.length;
      if (n.ref_seq == slot) {
        n.ref_seq = ref_seq;
        n.ref_idx = ref_idx;
      }
    }
  }
  delete slots_[slot];
  slots_[slot] = nullptr;
  free_slots_.push_back(slot);
  slot_of_.erase(found);
}

// Walk `context` down from the root (suffix_tree.cc:815-838).
bool arctic_suffix_tree::match(const int32_t *context, int64_t n, uint32_t &node, int &idx) const {
  node = root_;
  idx = 0;
  int32_t length = 0;
  const int32_t *text = nullptr;
  for (int64_t i = 0; i < n; ++i) {
    if (idx >= length) {
      node = find_child(node, context[i]);
      if (node == NIL) return false;
      text = label(node);
      length = nodes_[node].length;
      idx = 0;
    }
    if (text[idx] != context[i]) return false;
    ++idx;
  }
  return true;
}

// The single most frequent continuation (suffix_tree.cc:840-869).
Draft arctic_suffix_tree::draft_path(uint32_t node, int idx, int max_tokens, float min_token_prob) const {
  Draft d;
  float prob = 1.0f;
  const int32_t *text = node == root_ ? nullptr : label(node);
  while ((int)d.token_ids.size() < max_tokens && prob >= min_token_prob) {
    if (idx < nodes_[node].length) {
      d.parents.push_back((int32_t)d.token_ids.size() - 1);
      d.token_ids.push_back(text[idx]);
      d.probs.push_back(prob);
      d.score += prob;
      ++idx;
    } else {
      const uint32_t child = head_child(node);
      if (child == NIL) break;
      prob *= static_cast<float>(nodes_[child].count) / nodes_[node].count;
      node = child;
      text = label(node);
      idx = 0;
    }
  }
  return d;
}

namespace {
struct Candidate {
  float prob;
  uint32_t node;
  int idx;
  int parent;  // position in the draft of the token this one follows, -1 for none
};
struct LowerProb {
  bool operator()(const Candidate &a, const Candidate &b) const { return a.prob < b.prob; }
};
}  // namespace

// A tree of continuations, most probable first (suffix_tree.cc:871-905).
Draft arctic_suffix_tree::draft_tree(uint32_t node, int idx, int max_tokens, float min_token_prob) const {
  Draft d;
  std::priority_queue<Candidate, std::vector<Candidate>, LowerProb> best;
  best.push(Candidate{1.0f, node, idx, -1});
  while ((int)d.token_ids.size() < max_tokens && !best.empty()) {
    const Candidate c = best.top();
    best.pop();
    const Node &n = nodes_[c.node];
    if (c.idx < n.length) {
      d.token_ids.push_back(label(c.node)[c.idx]);
      d.parents.push_back(c.parent);
      d.probs.push_back(c.prob);
      d.score += c.prob;
      best.push(Candidate{c.prob, c.node, c.idx + 1, (int)d.token_ids.size() - 1});
    } else {
      for (uint32_t child = head_child(c.node); child != NIL; child = next_sibling(child)) {
        const float prob = c.prob * nodes_[child].count / static_cast<float>(n.count);
        if (prob < min_token_prob) break;
        best.push(Candidate{prob, child, 0, c.parent});
      }
    }
  }
  return d;
}

// suffix_tree.cc:583-612.  The reference tries every suffix of the context from the shortest up, stops at
// the first that is not in the tree, and keeps the draft with the highest score, the longest match
// winning a tie.  The same answer with less work: the suffixes that are in the tree are exactly those up
// to some length (a tree of suffixes holds every tail of what it holds), found by bisection; the drafts
// are then built from the longest match down, a shorter one replacing the best only with a strictly
// higher score, and the walk ends as soon as no remaining token budget could reach that score (a score
// is a sum of probabilities, so it never exceeds the number of tokens).
Draft arctic_suffix_tree::speculate(const int32_t *context, int64_t n, int max_spec_tokens, float max_spec_factor,
                                    float max_spec_offset, float min_token_prob, bool use_tree_spec) {
  Draft best;
  uint32_t node;
  int idx;
  int64_t longest = 0, beyond = n;  // suffixes of length <= longest match; those of length >= beyond do not
  while (beyond - longest > 1) {
    const int64_t mid = longest + (beyond - longest) / 2;
    if (match(context + (n - mid), mid, node, idx)) longest = mid; else beyond = mid;
  }
  if (longest == 0) return best;
  std::vector<int> budget((size_t)longest + 1, 0), budget_below((size_t)longest + 1, 0);
  for (int64_t m = 1; m <= longest; ++m) {
    const int tokens =
        std::min(max_spec_tokens, static_cast<int>((int)m * max_spec_factor + max_spec_offset + 1e-6));
    budget[m] = std::max(tokens, 0);
    budget_below[m] = std::max(budget_below[m - 1], budget[m - 1]);  // largest budget of any shorter match
  }
  bool have = false;
  for (int64_t m = longest; m >= 1; --m) {
    if (have && (float)budget[m] <= best.score) {
      if ((float)budget_below[m] <= best.score) break;
      continue;
    }
    match(context + (n - m), m, node, idx);
    Draft d = use_tree_spec ? draft_tree(node, idx, budget[m], min_token_prob)
                            : draft_path(node, idx, budget[m], min_token_prob);
    if (!have || d.score > best.score) {
      best = std::move(d);
      best.match_len = (int)m;
      have = true;
    }
    if ((float)budget_below[m] <= best.score) break;
  }
  return best;
}

#define ARCTIC_EXPECT(cond)                                                                              \
  do {                                                                                                   \
    if (!(cond)) return std::string("suffix tree invariant broken (line ") + std::to_string(__LINE__) + \
                        "): " #cond;                                                                     \
  } while (0)

std::string arctic_suffix_tree::check_integrity() {
  // 1. every node: links, order of children, labels, endpoints
  std::vector<uint32_t> order{root_};
  size_t endpoint_records = 0;
  for (size_t at = 0; at < order.size(); ++at) {
    const uint32_t node = order[at];
    const Node &n = nodes_[node];
    uint32_t seen = 0;
    int64_t last_count = -1;
    uint32_t prev_bucket = NIL;
    for (uint32_t b = n.first_bucket; b != NIL; b = buckets_[b].next) {
      const Bucket &k = buckets_[b];
      ARCTIC_EXPECT(k.prev == prev_bucket);
      ARCTIC_EXPECT(k.head != NIL && k.tail != NIL);
      ARCTIC_EXPECT(last_count < 0 || k.count < last_count);  // buckets in strictly decreasing count
      last_count = k.count;
      uint32_t prev = NIL;
      for (uint32_t c = k.head; c != NIL; c = nodes_[c].next) {
        const Node &ch = nodes_[c];
        ARCTIC_EXPECT(ch.bucket == b && ch.prev == prev && ch.parent == node);
        ARCTIC_EXPECT(ch.count == k.count);
        ARCTIC_EXPECT(child_of(node, ch.token) == c);
        ARCTIC_EXPECT(node == root_ || ch.count < n.count);  // else the two should be one node
        prev = c;
        ++seen;
        order.push_back(c);
      }
      ARCTIC_EXPECT(k.tail == prev);
      prev_bucket = b;
    }
    ARCTIC_EXPECT(n.last_bucket == prev_bucket);
    ARCTIC_EXPECT(seen == n.num_children);
    if (node == root_) {
      ARCTIC_EXPECT(n.count >= 0 && n.parent == NIL && n.length == 0 && n.num_endpoints == 0 && n.ref_idx == -1);
      continue;
    }
    ARCTIC_EXPECT(n.length > 0 && n.count > 0);
    ARCTIC_EXPECT(n.ref_seq >= 0 && (size_t)n.ref_seq < slots_.size() && slots_[n.ref_seq] != nullptr);
    const std::vector<int32_t> &ref = slots_[n.ref_seq]->tokens;
    ARCTIC_EXPECT(n.ref_idx >= 0 && (size_t)(n.ref_idx + n.length) <= ref.size());
    ARCTIC_EXPECT(n.token == ref[n.ref_idx]);
    uint32_t listed = 0;
    for (uint32_t e = n.first_endpoint; e != NIL; e = endpoints_[e].next) {
      const Endpoint &r = endpoints_[e];
      ++listed;
      ARCTIC_EXPECT(r.node == node && find_endpoint(node, r.seq) == e);  // also: one record per sequence
      ARCTIC_EXPECT(r.seq >= 0 && (size_t)r.seq < slots_.size() && slots_[r.seq] != nullptr);
      const std::vector<int32_t> &s = slots_[r.seq]->tokens;
      ARCTIC_EXPECT(r.end > 0 && (size_t)r.end <= s.size());
      // the tokens before the endpoint spell the path from the root to here
      int32_t idx = r.end;
      for (uint32_t up = node; up != root_; up = nodes_[up].parent) {
        const Node &u = nodes_[up];
        ARCTIC_EXPECT(u.length <= idx);
        idx -= u.length;
        const int32_t *text = label(up);
        for (int32_t i = 0; i < u.length; ++i) ARCTIC_EXPECT(s[idx + i] == text[i]);
      }
    }
    ARCTIC_EXPECT(listed == n.num_endpoints);
    endpoint_records += listed;
  }
  ARCTIC_EXPECT(order.size() == nodes_.live());
  ARCTIC_EXPECT(endpoint_records == endpoints_.live());
  // 2. every suffix of every sequence is in the tree, and the counts are the number of visits
  std::unordered_map<uint32_t, int64_t> visits;
  for (const auto &entry : slot_of_) {
    ARCTIC_EXPECT(slots_[entry.second] != nullptr && slots_[entry.second]->id == entry.first);
    const std::vector<int32_t> &seq = slots_[entry.second]->tokens;
    for (size_t start = 0; start < seq.size(); ++start) {
      size_t idx = start;
      uint32_t node = root_;
      visits[node]++;
      while (idx < seq.size() && idx - start < (size_t)max_depth_) {
        node = child_of(node, seq[idx]);
        ARCTIC_EXPECT(node != NIL);
        visits[node]++;
        const Node &n = nodes_[node];
        ARCTIC_EXPECT(idx + n.length <= seq.size());
        const int32_t *text = label(node);
        for (int32_t i = 0; i < n.length; ++i) ARCTIC_EXPECT(seq[idx + i] == text[i]);
        idx += n.length;
      }
      ARCTIC_EXPECT(find_endpoint(node, entry.second) != NIL);
    }
    // the growing suffixes point at their own records
    for (const Growing &g : slots_[entry.second]->active) {
      ARCTIC_EXPECT(endpoints_[g.endpoint].node == g.node && endpoints_[g.endpoint].seq == entry.second);
    }
  }
  for (uint32_t node : order) ARCTIC_EXPECT(nodes_[node].count == visits[node]);
  return std::string();
}

size_t arctic_suffix_tree::estimate_memory() const {
  size_t total = sizeof(*this) + nodes_.bytes() + buckets_.bytes() + endpoints_.bytes() + children_.bytes() +
                 endpoint_index_.bytes() + slots_.capacity() * sizeof(Sequence *) +
                 slot_of_.size() * (sizeof(std::pair<int32_t, int32_t>) + 2 * sizeof(void *));
  for (const Sequence *s : slots_)
    if (s) total += sizeof(*s) + s->tokens.capacity() * sizeof(int32_t) + s->active.size() * sizeof(Growing);
  return total;
}

// ---- C ABI -----------------------------------------------------------------------------------------
extern "C" {

int arctic_suffix_abi_version(void) { return ARCTIC_SUFFIX_ABI_VERSION; }

arctic_suffix_tree *arctic_suffix_tree_create(int max_depth) {
  if (max_depth < 1) return nullptr;
  return new (std::nothrow) arctic_suffix_tree(max_depth);
}

void arctic_suffix_tree_destroy(arctic_suffix_tree *tree) { delete tree; }

int arctic_suffix_tree_num_seqs(const arctic_suffix_tree *tree) { return tree ? tree->num_seqs() : 0; }

int arctic_suffix_tree_append(arctic_suffix_tree *tree, int seq_id, int32_t token) {
  if (!tree) return ARCTIC_SUFFIX_ERR_INVALID_ARGUMENT;
  try {
    tree->append(seq_id, token);
  } catch (const std::bad_alloc &) {
    return ARCTIC_SUFFIX_ERR_NO_MEMORY;
  }
  return 0;
}

int arctic_suffix_tree_extend(arctic_suffix_tree *tree, int seq_id, const int32_t *tokens, int64_t num_tokens) {
  if (!tree || num_tokens < 0 || (num_tokens > 0 && !tokens)) return ARCTIC_SUFFIX_ERR_INVALID_ARGUMENT;
  try {
    for (int64_t i = 0; i < num_tokens; ++i) tree->append(seq_id, tokens[i]);
  } catch (const std::bad_alloc &) {
    return ARCTIC_SUFFIX_ERR_NO_MEMORY;
  }
  return 0;
}

int arctic_suffix_tree_remove(arctic_suffix_tree *tree, int seq_id) {
  if (!tree) return ARCTIC_SUFFIX_ERR_INVALID_ARGUMENT;
  try {
    tree->remove(seq_id);
  } catch (const std::bad_alloc &) {
    return ARCTIC_SUFFIX_ERR_NO_MEMORY;
  }
  return 0;
}

int arctic_suffix_tree_speculate(arctic_suffix_tree *tree, const int32_t *context, int64_t context_len,
                                 int max_spec_tokens, float max_spec_factor, float max_spec_offset,
                                 float min_token_prob, int use_tree_spec, int32_t *token_ids, int32_t *parents,
                                 float *probs, float *score, int *match_len) {
  if (!tree || context_len < 0 || (context_len > 0 && !context)) return ARCTIC_SUFFIX_ERR_INVALID_ARGUMENT;
  if (max_spec_tokens > 0 && (!token_ids || !parents || !probs)) return ARCTIC_SUFFIX_ERR_INVALID_ARGUMENT;
  try {
    const Draft d = tree->speculate(context, context_len, max_spec_tokens, max_spec_factor, max_spec_offset,
                                    min_token_prob, use_tree_spec != 0);
    const size_t n = d.token_ids.size();
    if (n) {
      std::memcpy(token_ids, d.token_ids.data(), n * sizeof(int32_t));
      std::memcpy(parents, d.parents.data(), n * sizeof(int32_t));
      std::memcpy(probs, d.probs.data(), n * sizeof(float));
    }
    if (score) *score = d.score;
    if (match_len) *match_len = d.match_len;
    return (int)n;
  } catch (const std::bad_alloc &) {
    return ARCTIC_SUFFIX_ERR_NO_MEMORY;
  }
}

int arctic_suffix_tree_check_integrity(arctic_suffix_tree *tree, char *message, int capacity) {
  if (!tree) return ARCTIC_SUFFIX_ERR_INVALID_ARGUMENT;
  const std::string problem = tree->check_integrity();
  if (message && capacity > 0) std::snprintf(message, (size_t)capacity, "%s", problem.c_str());
  return problem.empty() ? 0 : 1;
}

size_t arctic_suffix_tree_estimate_memory(const arctic_suffix_tree *tree) {
  return tree ? tree->estimate_memory() : 0;
}

}  // extern "C"
