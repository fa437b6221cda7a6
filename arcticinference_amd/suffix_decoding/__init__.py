"""SuffixDecoding: suffix-tree speculation over prompts and previous responses (CPU).

Counterpart of the reference's ``arctic_inference.suffix_decoding`` package: ``SuffixDecodingCache`` and
``SuffixDecodingDraft`` (cache.py) over ``SuffixTree`` / ``Draft`` from ``libarctic_suffix.so``.
"""
from ._tree import Draft, SuffixTree
from .cache import SuffixDecodingCache, SuffixDecodingDraft

__all__ = ["Draft", "SuffixTree", "SuffixDecodingCache", "SuffixDecodingDraft"]
