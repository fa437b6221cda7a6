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


class _ResponseSlots:
    """Which sequence of the global tree holds which request's response.

    Sequence numbers are 31-bit and handed out by a counter that wraps; ``by_request`` keeps the
    responses in the order they were given a sequence, which is the order of eviction."""

    def __init__(self, limit: int):
        self.limit = limit                            # < 0: no limit
        self.by_request: Dict[Hashable, int] = {}     # insertion order = age
        self.holder: Dict[int, Hashable] = {}
        self.counter = 0

    def release(self, req_id: Hashable) -> int:
        seq = self.by_request.pop(req_id)
        del self.holder[seq]
        return seq

    def take(self, req_id: Hashable, is_active) -> List[int]:
        """Give ``req_id`` the next sequence number that is free or whose holder has finished, then apply
        the limit.  Returns the sequences whose responses have to leave the tree, in that order: a finished
        holder of the number taken first, then the oldest responses beyond the limit (never the one just
        added).  Reference cache.py:306-345."""
        while True:
            seq = self.counter
            self.counter = (seq + 1) & _SEQ_ID_MASK
            previous = self.holder.get(seq)
            if previous is None or not is_active(previous):
                break
        leaving = []
        if previous is not None:
            leaving.append(self.release(previous))
        self.by_request[req_id] = seq
        self.holder[seq] = req_id
        if self.limit >= 0:
            assert self.limit != 0   # with a limit of 0 no response is ever given a sequence
            excess = len(self.by_request) - self.limit
            if excess > 0:
                oldest = [r for r in self.by_request if r != req_id][:excess]
                leaving.extend(self.release(r) for r in oldest)
        return leaving


class SuffixDecodingCache:

    def __init__(self, max_tree_depth: int = 64, max_cached_requests: int = -1):
        """``max_tree_depth``: depth limit of every tree.  ``max_cached_requests``: how many responses the
        global tree keeps (oldest evicted first); ``-1`` for no limit, ``0`` to switch the global tree off
        (reference cache.py:63-96)."""
        if max_cached_requests > 0x7FFFFFFF:
            raise ValueError("max_cached_requests must be at most 2^31")
        self._max_tree_depth = max_tree_depth
        self._max_cached_requests = max_cached_requests
        self._global_tree = SuffixTree(max_tree_depth)   # the reference's simulator reads this attribute
        self._prompt_trees: Dict[Hashable, SuffixTree] = {}
        self._slots = _ResponseSlots(max_cached_requests)

    @property
    def max_tree_depth(self) -> int:
        return self._max_tree_depth

    @property
    def max_cached_requests(self) -> int:
        return self._max_cached_requests

    @property
    def active_requests(self) -> KeysView:
        """Requests between ``start_request`` and ``stop_request`` (their prompts are held)."""
        return self._prompt_trees.keys()

    @property
    def cached_requests(self) -> KeysView:
        """Requests whose responses are in the global tree."""
        return self._slots.by_request.keys()

    def _active_tree(self, req_id: Hashable) -> SuffixTree:
        try:
            return self._prompt_trees[req_id]
        except KeyError:
            raise ValueError(f"Request '{req_id}' is not active") from None

    def start_request(self, req_id: Hashable, prompt_token_ids: Tokens):
        """Begin a request: its prompt goes into a tree of its own, and (unless the global tree is switched
        off) a sequence for its response is taken in the global tree, evicting the oldest response if the
        limit is reached (reference cache.py:120-157)."""
        if req_id in self._prompt_trees:
            raise ValueError(f"Request '{req_id}' is already active")
        tokens = _validated(prompt_token_ids)
        tree = self._prompt_trees[req_id] = SuffixTree(self._max_tree_depth)
        _extend(tree, 0, tokens)
        if self._max_cached_requests == 0:
            return
        if req_id in self._slots.by_request:     # an earlier response under the same id
            self.evict_cached_response(req_id)
        for seq in self._slots.take(req_id, self._prompt_trees.__contains__):
            self._global_tree.remove(seq)

    def stop_request(self, req_id: Hashable):
        """End a request: its prompt tree is dropped; its response stays cached until evicted
        (reference cache.py:159-175)."""
        self._active_tree(req_id)
        del self._prompt_trees[req_id]

    def add_active_response(self, req_id: Hashable, token_ids: Tokens):
        """Append generated tokens to the request's own tree and to its response in the global tree
        (reference cache.py:177-207)."""
        own = self._active_tree(req_id)
        tokens = _validated(token_ids)
        _extend(own, 0, tokens)
        seq = self._slots.by_request.get(req_id)
        if seq is not None:
            _extend(self._global_tree, seq, tokens)

    def evict_cached_response(self, req_id: Hashable):
        """Remove the request's response from the global tree (reference cache.py:209-226)."""
        if req_id not in self._slots.by_request:
            raise ValueError(f"Request '{req_id}' is not cached")
        self._global_tree.remove(self._slots.release(req_id))

    def speculate(self, req_id: Hashable, context: Tokens, max_spec_tokens: Optional[int] = None,
                  max_spec_factor: float = 1.0, max_spec_offset: float = 0.0, min_token_prob: float = 0.1,
                  use_tree_spec: bool = False) -> SuffixDecodingDraft:
        """The better of the drafts from the request's own tree and from the global tree for the last
        ``max_tree_depth`` tokens of ``context``; at most ``max_spec_tokens`` tokens (default: the tree
        depth) and at most ``max_spec_factor * match_len + max_spec_offset``, each with an estimated
        probability of at least ``min_token_prob`` (reference cache.py:228-304; a tie goes to the
        request's own tree)."""
        own_tree = self._active_tree(req_id)
        context = _validated(context)
        depth = self._max_tree_depth
        budget = depth if max_spec_tokens is None else max_spec_tokens
        if len(context) > depth:
            context = context[-depth:]
        limits = (budget, max_spec_factor, max_spec_offset, min_token_prob, use_tree_spec)
        if isinstance(context, np.ndarray):
            context = np.ascontiguousarray(context)
            own, shared = (t.speculate_ndarray(context, *limits) for t in (own_tree, self._global_tree))
        else:
            own, shared = (t.speculate(context, *limits) for t in (own_tree, self._global_tree))
        return SuffixDecodingDraft.from_native(shared if shared.score > own.score else own)
