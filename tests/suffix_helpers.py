"""Shared pieces of the suffix-tree tests: seeded scripts of operations, and runners for the three
implementations (libarctic_suffix.so, the Python oracle, the reference's own code in oracle/_ref)."""
import os
import random

from oracle.suffix_ref import RefTree  # noqa: F401  (re-exported for the tests)

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def make_script(seed: int, steps: int = 80, max_seq: int = 12):
    """A list of operations: ("extend", seq_id, tokens) | ("remove", seq_id) |
    ("speculate", context, max_spec_tokens, factor, offset, min_prob, use_tree)."""
    rnd = random.Random(seed)
    depth = rnd.choice([2, 3, 4, 8, 16, 64])
    vocab = rnd.choice([2, 3, 5, 20, 1000])
    live, hist, script = [], {}, []
    for _ in range(steps):
        op = rnd.random()
        if op < 0.55 or not live:
            sid = rnd.choice(live) if live and rnd.random() < 0.6 else rnd.randint(0, max_seq)
            toks = [rnd.randrange(vocab) for _ in range(rnd.randint(1, 30))]
            script.append(("extend", sid, toks))
            if sid not in live:
                live.append(sid)
            hist.setdefault(sid, []).extend(toks)
        elif op < 0.7:
            sid = rnd.choice(live)
            live.remove(sid)
            hist.pop(sid)
            script.append(("remove", sid))
        else:
            src = hist[rnd.choice(live)]
            st = rnd.randrange(len(src))
            ctx = src[st:st + rnd.randint(1, depth + 3)]
            if rnd.random() < 0.2:
                ctx = ctx + [rnd.randrange(vocab)]
            script.append(("speculate", ctx, rnd.choice([0, 1, 4, 8, 32]), rnd.choice([0.5, 1.0, 2.0, 3.7]),
                           rnd.choice([0.0, -1.0, 2.5]), rnd.choice([0.0, 0.1, 0.3, 0.9]), rnd.random() < 0.5))
    return depth, script


def run_script(tree, script, check=None):
    """Apply the script to an object with extend / remove / speculate; returns the list of drafts as
    (token_ids, parents, probs, score, match_len) tuples."""
    drafts = []
    for op in script:
        if op[0] == "extend":
            tree.extend(op[1], op[2])
        elif op[0] == "remove":
            tree.remove(op[1])
        else:
            d = tree.speculate(*op[1:])
            if not isinstance(d, tuple):
                d = (d.token_ids, d.parents, d.probs, d.score, d.match_len)
            drafts.append((list(d[0]), list(d[1]), [float(p) for p in d[2]], float(d[3]), int(d[4])))
        if check is not None:
            check(tree)
    return drafts
