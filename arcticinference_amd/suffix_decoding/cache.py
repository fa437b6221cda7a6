"""Request-level cache for SuffixDecoding: one suffix tree per active request (its prompt and its
response so far) and one global tree over the responses of recent requests.

Drop-in counterpart of the reference's ``arctic_inference/suffix_decoding/cache.py`` (``SuffixDecodingDraft``
:26-58, ``SuffixDecodingCache`` :61-357): same constructor, properties, methods, defaults and errors.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, Hashable, KeysView, List, Optional, Sequence, Union

import numpy as np

from ._tree import Draft, SuffixTree

Tokens = Union[np.ndarray, Sequence[int]]
_SEQ_ID_MASK = 0x7FFFFFFF


@dataclass
class SuffixDecodingDraft:
    """A speculation: ``token_ids[i]`` follows ``token_ids[parents[i]]`` (``-1``: follows the context),
    ``probs[i]`` is its estimated probability, ``score`` the sum of the probabilities and ``match_len`` the
    length of the context suffix that was matched (reference cache.py:26-58)."""
    token_ids: List[int] = field(default_factory=list)
    parents: List[int] = field(default_factory=list)
    probs: List[float] = field(default_factory=list)
    score: float = 0.0
    match_len: int = 0

    @staticmethod
    def from_native(draft: Draft) -> "SuffixDecodingDraft":
        return SuffixDecodingDraft(token_ids=draft.token_ids, parents=draft.parents, probs=draft.probs,
                                   score=draft.score, match_len=draft.match_len)


def _validated(tokens: Tokens) -> Tokens:
    # reference cache.py:347-357
    if isinstance(tokens, np.ndarray):
        if tokens.ndim != 1:
            raise ValueError(f"ndarray input must have ndim=1, got ndim={tokens.ndim}")
        if tokens.dtype != np.int32:
            raise ValueError(f"ndarray input must have dtype=int32, got dtype={tokens.dtype.name}")
        if not tokens.flags["CONTIGUOUS"]:
            raise ValueError("ndarray input must be contiguous")
    return tokens


def _extend(tree: SuffixTree, seq_id: int, tokens: Tokens) -> None:
    if isinstance(tokens, np.ndarray):
        tree.extend_ndarray(seq_id, tokens)
    else:
        tree.extend(seq_id, tokens)


class SuffixDecodingCache:

    def __init__(self, max_tree_depth: int = 64, max_cached_requests: int = -1):
        """``max_tree_depth``: depth limit of every tree.  ``max_cached_requests``: how many responses the
        global tree keeps (oldest evicted first); ``-1`` for no limit, ``0`` to switch the global tree off
        (reference cache.py:63-96)."""
        if max_cached_requests > 0x7FFFFFFF:
            raise ValueError("max_cached_requests must be at most 2^31")
        self._max_tree_depth = max_tree_depth
        self._max_cached_requests = max_cached_requests
        self._global_tree = SuffixTree(max_tree_depth)
        self._local_trees: Dict[Hashable, SuffixTree] = {}
        # request id <-> sequence id in the global tree, for every cached response
        self._req_to_seq_id: Dict[Hashable, int] = {}
        self._seq_to_req_id: Dict[int, Hashable] = {}
        self._next_seq_id = 0

    @property
    def max_tree_depth(self) -> int:
        return self._max_tree_depth

    @property
    def max_cached_requests(self) -> int:
        return self._max_cached_requests

    @property
    def active_requests(self) -> KeysView:
        """Requests between ``start_request`` and ``stop_request`` (their prompts are held)."""
        return self._local_trees.keys()

    @property
    def cached_requests(self) -> KeysView:
        """Requests whose responses are in the global tree."""
        return self._req_to_seq_id.keys()

    def start_request(self, req_id: Hashable, prompt_token_ids: Tokens):
        """Begin a request: its prompt goes into a tree of its own, and (unless the global tree is switched
        off) a slot for its response is taken in the global tree, evicting the oldest response if the
        limit is reached (reference cache.py:120-157)."""
        if req_id in self._local_trees:
            raise ValueError(f"Request '{req_id}' is already active")
        prompt_token_ids = _validated(prompt_token_ids)
        tree = SuffixTree(self._max_tree_depth)
        self._local_trees[req_id] = tree
        _extend(tree, 0, prompt_token_ids)
        if self._max_cached_requests != 0:
            if req_id in self._req_to_seq_id:
                self.evict_cached_response(req_id)
            self._generate_seq_id(req_id)

    def stop_request(self, req_id: Hashable):
        """End a request: its prompt tree is dropped; its response stays cached until evicted
        (reference cache.py:159-175)."""
        if req_id not in self._local_trees:
            raise ValueError(f"Request '{req_id}' is not active")
        del self._local_trees[req_id]

    def add_active_response(self, req_id: Hashable, token_ids: Tokens):
        """Append generated tokens to the request's own tree and to its response in the global tree
        (reference cache.py:177-207)."""
        if req_id not in self._local_trees:
            raise ValueError(f"Request '{req_id}' is not active")
        token_ids = _validated(token_ids)
        _extend(self._local_trees[req_id], 0, token_ids)
        seq_id = self._req_to_seq_id.get(req_id)
        if seq_id is not None:
            _extend(self._global_tree, seq_id, token_ids)

    def evict_cached_response(self, req_id: Hashable):
        """Remove the request's response from the global tree (reference cache.py:209-226)."""
        if req_id not in self._req_to_seq_id:
            raise ValueError(f"Request '{req_id}' is not cached")
        seq_id = self._req_to_seq_id.pop(req_id)
        self._seq_to_req_id.pop(seq_id)
        self._global_tree.remove(seq_id)

    def speculate(self, req_id: Hashable, context: Tokens, max_spec_tokens: Optional[int] = None,
                  max_spec_factor: float = 1.0, max_spec_offset: float = 0.0, min_token_prob: float = 0.1,
                  use_tree_spec: bool = False) -> SuffixDecodingDraft:
        """The better of the drafts from the request's own tree and from the global tree for the last
        ``max_tree_depth`` tokens of ``context``; at most ``max_spec_tokens`` tokens (default: the tree
        depth) and at most ``max_spec_factor * match_len + max_spec_offset``, each with an estimated
        probability of at least ``min_token_prob`` (reference cache.py:228-304; a tie goes to the
        request's own tree)."""
        if req_id not in self._local_trees:
            raise ValueError(f"Request '{req_id}' is not active")
        context = _validated(context)
        if max_spec_tokens is None:
            max_spec_tokens = self._max_tree_depth
        if len(context) > self._max_tree_depth:
            context = context[-self._max_tree_depth:]
        drafts = []
        for tree in (self._local_trees[req_id], self._global_tree):
            if isinstance(context, np.ndarray):
                drafts.append(tree.speculate_ndarray(np.ascontiguousarray(context), max_spec_tokens, max_spec_factor,
                                                     max_spec_offset, min_token_prob, use_tree_spec))
            else:
                drafts.append(tree.speculate(context, max_spec_tokens, max_spec_factor, max_spec_offset,
                                             min_token_prob, use_tree_spec))
        own, shared = drafts
        return SuffixDecodingDraft.from_native(own if own.score >= shared.score else shared)

    def _generate_seq_id(self, req_id: Hashable) -> int:
        # the next sequence id (mod 2^31) that is free or belongs to a response of a finished request,
        # which is then evicted (reference cache.py:306-334)
        while True:
            seq_id = self._next_seq_id
            self._next_seq_id = (self._next_seq_id + 1) & _SEQ_ID_MASK
            holder = self._seq_to_req_id.get(seq_id)
            if holder is None or holder not in self._local_trees:
                break
        if seq_id in self._seq_to_req_id:
            del self._req_to_seq_id[self._seq_to_req_id[seq_id]]
            del self._seq_to_req_id[seq_id]
            self._global_tree.remove(seq_id)
        self._req_to_seq_id[req_id] = seq_id
        self._seq_to_req_id[seq_id] = req_id
        self._maybe_evict_requests(seq_id)
        return seq_id

    def _maybe_evict_requests(self, new_seq_id: int):
        # oldest first (dict order = order of insertion), never the slot just taken (reference cache.py:336-345)
        if self._max_cached_requests < 0:
            return
        assert self._max_cached_requests != 0
        while len(self._req_to_seq_id) > self._max_cached_requests:
            victim = next(r for r, s in self._req_to_seq_id.items() if s != new_seq_id)
            self.evict_cached_response(victim)
