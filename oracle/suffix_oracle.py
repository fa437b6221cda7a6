"""CPU restatement of the reference's suffix-tree speculation - TEST INFRASTRUCTURE ONLY.

Restates csrc/suffix_decoding/suffix_tree.cc of the reference as a plain, UNCOMPRESSED trie (one trie
node per token; the reference compresses chains into nodes with a length), in pure Python, for small
cases.  What must agree with the reference is the observable behaviour: the drafts.  They depend on

* the counts (how many suffixes, each cut at max_depth tokens, pass through a trie node), which are
  canonical, and
* the order of a node's children: by decreasing count, and among equal counts by the history of
  changes (suffix_tree.cc:31-296: a new child goes last; a child whose count rises joins the run of the
  higher count at its front if it was the first of its old run, at its back otherwise; a child whose
  count falls goes to the front of the run of the lower count).  A chain inside one of the reference's
  compressed nodes has single children, so compression does not change any order.

The tree-shaped draft additionally depends on the order in which std::priority_queue returns
candidates of equal probability; `_Heap` below restates libstdc++'s push_heap / pop_heap (GCC's
bits/stl_heap.h, the standard library the reference is built with) and the candidates are pushed in
the reference's order (one per token inside a compressed node, one "expand" step at its end;
suffix_tree.cc:871-905).  Probabilities are computed in fp32 with the reference's expressions.

Pinned by tests/test_suffix_tree.py: against the reference's own code compiled into oracle/_ref (when
that has been built), against fixtures that build wrote (tests/golden/suffix_tree.json), and against
brute-force suffix counting.
"""
from __future__ import annotations

from typing import Dict, List, Optional, Sequence

import numpy as np

f32 = np.float32


class _Trie:
    __slots__ = ("token", "count", "children", "order", "parent")

    def __init__(self, token: int, parent: Optional["_Trie"]):
        self.token = token
        self.count = 0
        self.children: Dict[int, _Trie] = {}
        self.order: List[_Trie] = []     # children, highest count first
        self.parent = parent

    def ends_compressed_node(self) -> bool:
        """True where the reference's compressed node ends: anything but exactly one child that carries
        every suffix of this node (the integrity rule "child count < node count", suffix_tree.cc:723-728)."""
        return not (len(self.order) == 1 and self.order[0].count == self.count)


def _count_up(parent: _Trie, child: _Trie) -> None:
    # suffix_tree.cc:171-215
    order = parent.order
    i = order.index(child)
    c = child.count
    j = i
    while j > 0 and order[j - 1].count == c:
        j -= 1                                    # start of the run of count c
    first_of_run = i == j
    has_higher_run = j > 0 and order[j - 1].count == c + 1
    order.pop(i)
    if first_of_run:
        if has_higher_run:
            k = j - 1
            while k > 0 and order[k - 1].count == c + 1:
                k -= 1
            order.insert(k, child)                # front of the (c+1)-run
        else:
            order.insert(i, child)                # stays where it is
    else:
        order.insert(j, child)                    # right behind the (c+1)-run, if any
    child.count = c + 1


def _count_down(parent: _Trie, child: _Trie) -> None:
    # suffix_tree.cc:217-294
    order = parent.order
    i = order.index(child)
    c = child.count
    order.pop(i)
    j = i
    while j < len(order) and order[j].count == c:
        j += 1                                    # just behind the run of count c
    order.insert(j, child)
    child.count = c - 1


class _Heap:
    """std::priority_queue<T, std::vector<T>, Cmp> of libstdc++ (bits/stl_heap.h: __push_heap,
    __adjust_heap, __pop_heap), with less(a, b) = a[0] < b[0]."""

    def __init__(self):
        self.v: list = []

    @staticmethod
    def _less(a, b) -> bool:
        return a[0] < b[0]

    def _push_up(self, hole: int, top: int, value) -> None:
        v = self.v
        parent = (hole - 1) // 2
        while hole > top and self._less(v[parent], value):
            v[hole] = v[parent]
            hole = parent
            parent = (hole - 1) // 2
        v[hole] = value

    def push(self, value) -> None:
        self.v.append(value)
        self._push_up(len(self.v) - 1, 0, value)

    def pop(self):
        v = self.v
        top = v[0]
        value = v[-1]
        v[-1] = v[0]
        n = len(v) - 1                            # heap length without the element being removed
        hole = 0
        second = 0
        while second < (n - 1) // 2:
            second = 2 * (second + 1)
            if self._less(v[second], v[second - 1]):
                second -= 1
            v[hole] = v[second]
            hole = second
        if n % 2 == 0 and second == (n - 2) // 2:
            second = 2 * (second + 1)
            v[hole] = v[second - 1]
            hole = second - 1
        if n > 0:
            self._push_up(hole, 0, value)
        v.pop()
        return top

    def __len__(self) -> int:
        return len(self.v)


class SuffixTreeOracle:
    def __init__(self, max_depth: int):
        self.max_depth = max_depth
        self.root = _Trie(0, None)
        self.seqs: Dict[int, List[int]] = {}
        self.active: Dict[int, List[_Trie]] = {}

    def num_seqs(self) -> int:
        return len(self.seqs)

    # suffix_tree.cc:297-490
    def append(self, seq_id: int, token: int) -> None:
        seq = self.seqs.setdefault(seq_id, [])
        active = self.active.setdefault(seq_id, [])
        active.append(self.root)
        self.root.count += 1
        if len(active) > self.max_depth:
            active.pop(0)
        seq.append(token)
        for k, node in enumerate(active):
            child = node.children.get(token)
            if child is None:
                child = _Trie(token, node)
                child.count = 1
                node.children[token] = child
                node.order.append(child)
            else:
                _count_up(node, child)
            active[k] = child

    def extend(self, seq_id: int, tokens: Sequence[int]) -> None:
        for t in tokens:
            self.append(seq_id, int(t))

    # suffix_tree.cc:500-581
    def remove(self, seq_id: int) -> None:
        seq = self.seqs.get(seq_id)
        if seq is None:
            return
        for start in range(len(seq)):
            node = self.root
            node.count -= 1
            for idx in range(start, min(len(seq), start + self.max_depth)):
                child = node.children.get(seq[idx])
                if child is None:
                    break
                if child.count > 1:
                    _count_down(node, child)
                else:
                    node.order.remove(child)
                    del node.children[seq[idx]]
                    break
                node = child
        del self.seqs[seq_id]
        del self.active[seq_id]

    # suffix_tree.cc:815-838
    def _match(self, context: Sequence[int]) -> Optional[_Trie]:
        node = self.root
        for t in context:
            node = node.children.get(int(t))
            if node is None:
                return None
        return node

    # suffix_tree.cc:840-869
    def _path(self, node: _Trie, max_tokens: int, min_token_prob: float):
        tokens, parents, probs = [], [], []
        score = f32(0.0)
        prob = f32(1.0)
        lo = f32(min_token_prob)
        while len(tokens) < max_tokens and prob >= lo:
            if not node.order:
                break
            child = node.order[0]
            if node.ends_compressed_node():
                prob = f32(prob * f32(f32(child.count) / f32(node.count)))
                if not prob >= lo:
                    break
            parents.append(len(tokens) - 1)
            tokens.append(child.token)
            probs.append(float(prob))
            score = f32(score + prob)
            node = child
        return tokens, parents, probs, float(score)

    # suffix_tree.cc:871-905
    def _tree(self, node: _Trie, max_tokens: int, min_token_prob: float):
        tokens, parents, probs = [], [], []
        score = f32(0.0)
        lo = f32(min_token_prob)
        heap = _Heap()
        # candidates: (prob, "emit", trie node whose token comes next, parent) or (prob, "expand", node, parent)
        first = ("expand", node) if node.ends_compressed_node() else ("emit", node.order[0])
        heap.push((f32(1.0),) + first + (-1,))
        while len(tokens) < max_tokens and len(heap):
            prob, kind, at, parent = heap.pop()
            if kind == "emit":
                tokens.append(at.token)
                parents.append(parent)
                probs.append(float(prob))
                score = f32(score + prob)
                here = len(tokens) - 1
                if at.ends_compressed_node():
                    heap.push((prob, "expand", at, here))
                else:
                    heap.push((prob, "emit", at.order[0], here))
            else:
                for child in at.order:
                    p = f32(f32(prob * f32(child.count)) / f32(at.count))
                    if p < lo:
                        break
                    heap.push((p, "emit", child, parent))
        return tokens, parents, probs, float(score)

    # suffix_tree.cc:583-612
    def speculate(self, context: Sequence[int], max_spec_tokens: int, max_spec_factor: float,
                  max_spec_offset: float, min_token_prob: float, use_tree_spec: bool):
        """(token_ids, parents, probs, score, match_len)"""
        best = ([], [], [], 0.0, 0)
        n = len(context)
        for match_len in range(1, n):
            node = self._match(context[n - match_len:])
            if node is None:
                break
            limit = int(float(f32(f32(f32(match_len) * f32(max_spec_factor)) + f32(max_spec_offset))) + 1e-6)
            max_tokens = max(min(max_spec_tokens, limit), 0)
            draft = (self._tree if use_tree_spec else self._path)(node, max_tokens, min_token_prob)
            if f32(draft[3]) >= f32(best[3]):
                best = draft + (match_len,)
        return best
