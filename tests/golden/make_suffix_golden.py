"""Writes tests/golden/suffix_tree.json: seeded scripts of suffix-tree operations and the drafts the
REFERENCE's own code returns for them.

The reference's csrc/suffix_decoding/suffix_tree.cc is compiled, from where it lies, by
`make -C oracle ref` (oracle/_ref/libsuffix_ref.so); this script drives that library and records what it
answers.  The fixture holds inputs and outputs only.  Run from the repository root:

    make -C oracle ref && python tests/golden/make_suffix_golden.py
"""
import json
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))                    # tests/
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))   # repository root (the oracle package)
from suffix_helpers import RefTree, make_script, run_script  # noqa: E402


def main():
    if not RefTree.available():
        sys.exit("oracle/_ref/libsuffix_ref.so is missing: run `make -C oracle ref` first")
    cases = []
    for seed in range(1000, 1040):
        depth, script = make_script(seed, steps=60)
        tree = RefTree(depth)
        drafts = run_script(tree, script)
        assert tree.check_integrity() == ""
        cases.append({"seed": seed, "max_depth": depth, "script": script, "drafts": drafts})
    out = os.path.join(HERE, "suffix_tree.json")
    with open(out, "w") as f:
        json.dump({"source": "reference csrc/suffix_decoding/suffix_tree.cc, g++ -O3 -DNDEBUG -std=c++20",
                   "cases": cases}, f, separators=(",", ":"))
    print(out, os.path.getsize(out), "bytes;", sum(len(c["drafts"]) for c in cases), "drafts")


if __name__ == "__main__":
    main()
