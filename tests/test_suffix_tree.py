"""Suffix-tree speculation (CPU): libarctic_suffix.so and the Python oracle against the reference's own
code (golden fixtures written from it; the compiled reference itself where oracle/_ref has been built),
against brute-force suffix counting, and the request-level cache on top."""
import ctypes
import json
import os
import re
import subprocess

import numpy as np
import pytest

from arcticinference_amd.suffix_decoding import SuffixDecodingCache, SuffixDecodingDraft, SuffixTree
from arcticinference_amd.suffix_decoding import _tree
from oracle.suffix_oracle import SuffixTreeOracle, _Heap
from suffix_helpers import ROOT, RefTree, make_script, run_script

GOLDEN = os.path.join(ROOT, "tests", "golden", "suffix_tree.json")


def as_ops(script):
    return [tuple(op) for op in script]


def golden_cases():
    with open(GOLDEN) as f:
        return json.load(f)["cases"]


def tupled(drafts):
    return [(list(d[0]), list(d[1]), [float(p) for p in d[2]], float(d[3]), int(d[4])) for d in drafts]


def assert_intact(tree):
    assert tree.check_integrity() == ""


# ---- pinned by the reference's answers ---------------------------------------------------------------
def test_library_reproduces_the_reference_fixtures():
    cases = golden_cases()
    assert len(cases) == 40 and sum(len(c["drafts"]) for c in cases) > 500
    for case in cases:
        tree = SuffixTree(case["max_depth"])
        got = run_script(tree, as_ops(case["script"]), check=assert_intact)
        assert got == tupled(case["drafts"]), f"seed {case['seed']}"


def test_oracle_reproduces_the_reference_fixtures():
    for case in golden_cases():
        got = run_script(SuffixTreeOracle(case["max_depth"]), as_ops(case["script"]))
        assert got == tupled(case["drafts"]), f"seed {case['seed']}"


@pytest.mark.skipif(not RefTree.available(), reason="oracle/_ref is not built here (needs the reference's sources)")
def test_against_the_compiled_reference():
    for seed in range(150):
        depth, script = make_script(seed)
        want = run_script(RefTree(depth), script)
        assert run_script(SuffixTree(depth), script, check=assert_intact) == want, f"library, seed {seed}"
        assert run_script(SuffixTreeOracle(depth), script) == want, f"oracle, seed {seed}"


def test_library_against_oracle_on_fresh_scripts():
    # scripts the fixtures do not hold; longer, more sequences
    for seed in range(5000, 5060):
        depth, script = make_script(seed, steps=120, max_seq=30)
        assert run_script(SuffixTree(depth), script, check=assert_intact) == \
            run_script(SuffixTreeOracle(depth), script), f"seed {seed}"


# ---- pinned by what the definition fixes ---------------------------------------------------------------
def brute_force_counts(seqs, depth):
    """How often each token string of length <= depth occurs as the start of a suffix."""
    counts = {}
    for seq in seqs:
        for start in range(len(seq)):
            for end in range(start + 1, min(len(seq), start + depth) + 1):
                key = tuple(seq[start:end])
                counts[key] = counts.get(key, 0) + 1
    return counts


def oracle_counts(node, prefix=()):
    out = {}
    for child in node.order:
        key = prefix + (child.token,)
        out[key] = child.count
        out.update(oracle_counts(child, key))
    return out


def test_oracle_counts_are_suffix_counts_and_children_are_sorted():
    rng = np.random.default_rng(3)
    for depth, vocab in ((3, 2), (5, 3), (8, 4)):
        tree = SuffixTreeOracle(depth)
        seqs = {}
        for step in range(40):
            sid = int(rng.integers(0, 6))
            if sid in seqs and rng.random() < 0.25:
                tree.remove(sid)
                del seqs[sid]
            else:
                toks = rng.integers(0, vocab, int(rng.integers(1, 12))).tolist()
                tree.extend(sid, toks)
                seqs.setdefault(sid, []).extend(toks)
            assert oracle_counts(tree.root) == brute_force_counts(seqs.values(), depth)
            assert tree.root.count == sum(len(s) for s in seqs.values())
            stack = [tree.root]
            while stack:
                n = stack.pop()
                assert [c.count for c in n.order] == sorted((c.count for c in n.order), reverse=True)
                assert set(n.children.values()) == set(n.order)
                stack.extend(n.order)


def test_path_draft_follows_the_most_frequent_continuation():
    # "1 2 3" three times, "1 2 4" once: after (1, 2) the draft must say 3 with probability 3/4
    for make in (SuffixTree, SuffixTreeOracle):
        tree = make(8)
        tree.extend(0, [1, 2, 3, 9, 1, 2, 3, 8, 1, 2, 3, 7, 1, 2, 4])
        d = run_script(tree, [("speculate", [5, 1, 2], 1, 1.0, 0.0, 0.0, False)])[0]
        assert d[0] == [3] and d[1] == [-1] and d[4] == 2
        assert d[2] == [0.75] and d[3] == 0.75
        # the whole context is never used as the match (match_len < len(context)): (1, 2) alone gives match_len 1
        d = run_script(tree, [("speculate", [1, 2], 4, 1.0, 0.0, 0.0, False)])[0]
        assert d[4] == 1 and d[0][:1] == [3]
        # min_token_prob cuts the draft where the estimate falls below it
        d = run_script(tree, [("speculate", [5, 1, 2], 8, 4.0, 0.0, 0.8, False)])[0]
        assert d[0] == []
        # tree draft: both continuations, the likelier first, both hanging off the context
        d = run_script(tree, [("speculate", [5, 1, 2], 2, 1.0, 0.0, 0.0, True)])[0]
        assert d[0] == [3, 4] and d[1] == [-1, -1] and d[2] == [0.75, 0.25]


def test_token_budget_formula():
    # max tokens = min(max_spec_tokens, int(match_len * factor + offset + 1e-6)), never negative
    for make in (SuffixTree, SuffixTreeOracle):
        tree = make(16)
        tree.extend(0, list(range(1, 15)))
        for k, factor, offset, want in ((32, 1.0, 0.0, 3), (32, 2.0, 0.0, 6), (32, 0.5, 0.0, 1), (2, 2.0, 0.0, 2),
                                        (32, 1.0, -5.0, 0), (32, 0.7, 0.9, 3), (0, 1.0, 0.0, 0)):
            d = run_script(tree, [("speculate", [0, 1, 2, 3], k, factor, offset, 0.0, False)])[0]
            assert len(d[0]) == want and d[0] == list(range(4, 4 + want)), (k, factor, offset)


def test_heap_restatement_matches_a_sorted_order_and_breaks_ties_like_libstdcxx():
    rng = np.random.default_rng(0)
    h = _Heap()
    items = [(float(rng.integers(0, 5)), i) for i in range(200)]
    for it in items:
        h.push(it)
    out = [h.pop() for _ in range(len(items))]
    assert [o[0] for o in out] == sorted((i[0] for i in items), reverse=True)
    # known answers, taken from std::priority_queue itself (g++ 11, the same push / pop sequence)
    h = _Heap()
    for i in range(5):
        h.push((1.0, i))
    assert [h.pop()[1] for _ in range(5)] == [0, 2, 4, 1, 3]
    h = _Heap()
    for i, p in enumerate((0.5, 1.0, 0.5, 0.25, 1.0, 0.5, 0.25, 1.0)):
        h.push((p, i))
    assert [h.pop()[1] for _ in range(8)] == [1, 4, 7, 2, 5, 0, 3, 6]


# ---- edge cases ---------------------------------------------------------------------------------------
def test_empty_and_unknown():
    tree = SuffixTree(4)
    assert tree.num_seqs() == 0 and tree.check_integrity() == ""
    tree.remove(7)                                       # unknown id: ignored
    d = tree.speculate([], 4, 1.0, 0.0, 0.1, False)
    assert (d.token_ids, d.parents, d.probs, d.score, d.match_len) == ([], [], [], 0.0, 0)
    tree.extend(3, [])                                   # no tokens: no sequence yet
    tree.extend(3, [5])
    assert tree.num_seqs() == 1
    d = tree.speculate([5, 5], 4, 1.0, 0.0, 0.1, True)    # matches, but nothing follows
    assert d.token_ids == [] and d.match_len == 1
    tree.remove(3)
    assert tree.num_seqs() == 0 and tree.check_integrity() == ""
    assert tree.estimate_memory() > 0
    with pytest.raises(ValueError):
        SuffixTree(0)


def test_long_repetitive_sequence_and_depth_limit():
    # one token repeated: every suffix is cut at max_depth, so many suffixes of one sequence end in one node
    for depth in (1, 2, 5):
        tree, oracle = SuffixTree(depth), SuffixTreeOracle(depth)
        script = [("extend", 0, [7] * 50), ("extend", 1, [7, 8] * 20), ("speculate", [1, 7, 7], 8, 3.0, 0.0, 0.0, False),
                  ("speculate", [7, 8, 7], 8, 3.0, 0.0, 0.0, True), ("remove", 0),
                  ("speculate", [7, 8, 7], 8, 3.0, 0.0, 0.0, True), ("remove", 1)]
        assert run_script(tree, script, check=assert_intact) == run_script(oracle, script)
        assert tree.num_seqs() == 0


def test_append_equals_extend_and_ndarray_entry_points():
    a, b, c = SuffixTree(8), SuffixTree(8), SuffixTree(8)
    toks = [3, 1, 4, 1, 5, 9, 2, 6, 5, 3, 5, 8, 9, 7, 9, 3]
    a.extend(0, toks)
    for t in toks:
        b.append(0, t)
    c.extend_ndarray(0, np.array(toks, dtype=np.int32))
    ctx = [9, 3, 5]
    drafts = [t.speculate(ctx, 6, 2.0, 0.0, 0.0, True) for t in (a, b)]
    drafts.append(c.speculate_ndarray(np.array(ctx, dtype=np.int32), 6, 2.0, 0.0, 0.0, True))
    assert len({(tuple(d.token_ids), tuple(d.parents), tuple(d.probs), d.score, d.match_len) for d in drafts}) == 1


# ---- the request-level cache (reference cache.py) -------------------------------------------------------
def test_cache_prompt_and_response_sharing():
    cache = SuffixDecodingCache(max_tree_depth=8)
    cache.start_request("a", [1, 2, 3, 4, 5, 6])
    assert list(cache.active_requests) == ["a"] and list(cache.cached_requests) == ["a"]
    d = cache.speculate("a", [9, 2, 3], max_spec_tokens=3)          # from the request's own prompt
    assert isinstance(d, SuffixDecodingDraft) and d.token_ids == [4, 5] and d.match_len == 2
    cache.add_active_response("a", np.array([7, 8, 9, 10], dtype=np.int32))
    cache.stop_request("a")
    cache.start_request("b", [0])
    d = cache.speculate("b", [0, 7, 8], max_spec_tokens=4)          # from a's cached response
    assert d.token_ids == [9, 10] and d.score == 2.0
    assert cache.speculate("b", [0, 2, 3]).token_ids == []          # a's prompt went with stop_request
    with pytest.raises(ValueError, match="already active"):
        cache.start_request("b", [1])
    with pytest.raises(ValueError, match="not active"):
        cache.speculate("a", [1, 2])
    with pytest.raises(ValueError, match="not active"):
        cache.add_active_response("zz", [1])
    with pytest.raises(ValueError, match="not active"):
        cache.stop_request("zz")
    with pytest.raises(ValueError, match="not cached"):
        cache.evict_cached_response("zz")
    cache.evict_cached_response("a")
    assert cache.speculate("b", [0, 7, 8]).token_ids == []


def test_cache_eviction_is_first_in_first_out_and_limits():
    cache = SuffixDecodingCache(max_tree_depth=4, max_cached_requests=2)
    for name in ("r0", "r1", "r2"):
        cache.start_request(name, [1])
        cache.add_active_response(name, [10, 11, 12])
        cache.stop_request(name)
    assert list(cache.cached_requests) == ["r1", "r2"]              # r0 evicted first
    assert cache._global_tree.num_seqs() == 2
    off = SuffixDecodingCache(max_tree_depth=4, max_cached_requests=0)   # global tree switched off
    off.start_request("x", [1, 2, 3, 1, 2])
    off.add_active_response("x", [3])
    assert list(off.cached_requests) == [] and off._global_tree.num_seqs() == 0
    assert off.speculate("x", [5, 1, 2], max_spec_tokens=2).token_ids == [3, 1]
    with pytest.raises(ValueError, match="at most 2\\^31"):
        SuffixDecodingCache(max_cached_requests=1 << 31)
    # restarting a cached request drops its old response first
    cache.start_request("r2", [1])
    assert list(cache.cached_requests) == ["r1", "r2"] and cache._global_tree.num_seqs() == 1


def test_cache_sequence_numbers_wrap_skip_active_holders_and_displace_finished_ones():
    # reference cache.py:306-334: 31-bit numbers from a wrapping counter; a number whose holder is still active is
    # passed over, a number whose holder has finished is taken and that response leaves the tree
    cache = SuffixDecodingCache(max_tree_depth=4)
    cache._slots.counter = 0x7FFFFFFE
    for name in ("a", "b", "c"):                      # numbers 2^31-2, 2^31-1, 0
        cache.start_request(name, [1])
        cache.add_active_response(name, [20, 21, 22])
    assert [cache._slots.by_request[n] for n in "abc"] == [0x7FFFFFFE, 0x7FFFFFFF, 0]
    cache.stop_request("b")
    cache._slots.counter = 0x7FFFFFFE                 # the counter comes round again
    cache.start_request("d", [1])                     # a is active: passed over; b has finished: displaced
    assert cache._slots.by_request["d"] == 0x7FFFFFFF and "b" not in cache.cached_requests
    assert list(cache.cached_requests) == ["a", "c", "d"]
    assert cache._global_tree.num_seqs() == 2             # a and c: b has left, d has no tokens yet
    cache.start_request("e", [1])                     # c (number 0) is active: passed over as well
    assert cache._slots.by_request["e"] == 1
    cache.add_active_response("d", [30, 31])
    assert cache._global_tree.num_seqs() == 3
    assert cache.speculate("e", [1, 30], max_spec_tokens=1).token_ids == [31]
    assert cache._global_tree.check_integrity() == ""


def test_cache_validates_ndarrays_and_truncates_context():
    cache = SuffixDecodingCache(max_tree_depth=4)
    with pytest.raises(ValueError, match="dtype=int32"):
        cache.start_request("a", np.array([1, 2, 3]))
    with pytest.raises(ValueError, match="ndim=1"):
        cache.start_request("a", np.zeros((2, 2), dtype=np.int32))
    with pytest.raises(ValueError, match="contiguous"):
        cache.start_request("a", np.arange(10, dtype=np.int32)[::2])
    cache.start_request("a", np.arange(20, dtype=np.int32))
    d = cache.speculate("a", np.arange(3, 12, dtype=np.int32), max_spec_tokens=2)
    # only the last 4 tokens are looked at, and a depth-4 tree holds 2 more tokens behind a match of 2
    assert d.match_len == 2 and d.token_ids == [12, 13]
    same = cache.speculate("a", np.arange(8, 12, dtype=np.int32), max_spec_tokens=2)
    assert same == d


# ---- the C ABI -------------------------------------------------------------------------------------------
def test_library_exports_what_the_header_declares():
    header = open(os.path.join(ROOT, "include", "arctic_suffix.h")).read()
    declared = set(re.findall(r"\b(arctic_suffix_\w+)\s*\(", header))
    assert declared == set(_tree.EXPORTED_SYMBOLS)
    lib = ctypes.CDLL(_tree.library_path())
    for sym in declared:
        assert hasattr(lib, sym), sym
    needed = subprocess.run(["readelf", "-d", _tree.library_path()], capture_output=True, text=True).stdout
    assert "libamdhip64" not in needed and "libtorch" not in needed and "libpython" not in needed


def test_c_abi_rejects_bad_arguments():
    lib = _tree._lib
    assert lib.arctic_suffix_tree_create(0) is None
    assert lib.arctic_suffix_tree_append(None, 0, 1) == -1
    h = lib.arctic_suffix_tree_create(4)
    assert lib.arctic_suffix_tree_extend(h, 0, None, 3) == -1
    assert lib.arctic_suffix_tree_extend(h, 0, None, 0) == 0
    ctx = np.array([1, 2], dtype=np.int32)
    assert lib.arctic_suffix_tree_speculate(h, ctx.ctypes.data, 2, 4, 1.0, 0.0, 0.1, 0, None, None, None, None, None) == -1
    lib.arctic_suffix_tree_destroy(h)
    lib.arctic_suffix_tree_destroy(None)


def test_ndarray_entry_points_turn_away_what_is_not_an_int32_vector():
    import numpy as np
    from arcticinference_amd.suffix_decoding import SuffixTree
    tree = SuffixTree(8)
    tree.extend_ndarray(0, np.array([1, 2, 3, 1, 2], dtype=np.int32))
    for bad in (np.array([1, 2, 3], dtype=np.int64), np.zeros((2, 2), dtype=np.int32),
                np.arange(10, dtype=np.int32)[::2], [1, 2, 3]):
        with pytest.raises(TypeError):
            tree.extend_ndarray(1, bad)
        with pytest.raises(TypeError):
            tree.speculate_ndarray(bad, 4, 1.0, 0.0, 0.1, False)
    assert tree.speculate_ndarray(np.array([1, 2], dtype=np.int32), 4, 1.0, 0.0, 0.1, False).token_ids[:1] == [3]
    assert tree.check_integrity() == ""
