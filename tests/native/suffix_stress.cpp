// Stress driver for libarctic_suffix's C ABI, meant to be built together with suffix_tree.cpp under
// AddressSanitizer and UndefinedBehaviorSanitizer (tests/test_suffix_sanitizers.py does that): seeded random
// appends, extends, removals and drafts over many sequences and several depth limits, the tree's own integrity
// check after every batch, and a brute-force count of how often the draft's first token follows the matched
// suffix in the live sequences.  Exits 0 and prints "ok" if nothing is reported.
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <map>
#include <random>
#include <vector>

#include "arctic_suffix.h"

static int fail(const char *what, int round) {
  std::fprintf(stderr, "suffix_stress: %s (round %d)\n", what, round);
  return 1;
}

int main(int argc, char **argv) {
  const unsigned seed = argc > 1 ? (unsigned)std::atoi(argv[1]) : 1u;
  const int rounds = argc > 2 ? std::atoi(argv[2]) : 400;
  std::mt19937 rng(seed);
  auto pick = [&](int n) { return (int)(rng() % (unsigned)n); };
  for (int depth : {1, 2, 5, 16, 64}) {
    arctic_suffix_tree *tree = arctic_suffix_tree_create(depth);
    if (!tree) return fail("create returned NULL", 0);
    std::map<int, std::vector<int32_t>> live;
    const int vocab = depth <= 2 ? 3 : 6;   // small alphabets: long shared suffixes, many splits and merges
    for (int round = 0; round < rounds; ++round) {
      const int op = pick(10);
      const int seq = pick(12) + (pick(20) == 0 ? 0x7ffffff0 : 0);
      if (op < 4) {
        const int n = pick(40);
        std::vector<int32_t> toks(n);
        for (auto &t : toks) t = pick(vocab);
        if (arctic_suffix_tree_extend(tree, seq, toks.data(), n) != 0) return fail("extend failed", round);
        auto &s = live[seq];
        s.insert(s.end(), toks.begin(), toks.end());
      } else if (op < 6) {
        const int32_t t = pick(vocab);
        if (arctic_suffix_tree_append(tree, seq, t) != 0) return fail("append failed", round);
        live[seq].push_back(t);
      } else if (op < 7) {
        if (arctic_suffix_tree_remove(tree, seq) != 0) return fail("remove failed", round);
        live.erase(seq);
      } else {
        const int clen = pick(depth + 3);
        std::vector<int32_t> ctx(clen);
        for (auto &t : ctx) t = pick(vocab);
        const int budget = pick(12);
        std::vector<int32_t> ids(budget + 1), parents(budget + 1);
        std::vector<float> probs(budget + 1);
        float score = -1.f;
        int match_len = -1;
        const int n = arctic_suffix_tree_speculate(tree, ctx.data(), clen, budget, 1.0f + pick(3), (float)pick(3),
                                                   0.05f * pick(4), pick(2), ids.data(), parents.data(),
                                                   probs.data(), &score, &match_len);
        if (n < 0 || n > budget) return fail("speculate returned a count outside [0, budget]", round);
        if (match_len < 0 || match_len > clen || match_len > depth) return fail("match_len out of range", round);
        float sum = 0.f;
        for (int i = 0; i < n; ++i) {
          if (parents[i] < -1 || parents[i] >= i) return fail("parent does not precede its child", round);
          if (!(probs[i] > 0.f && probs[i] <= 1.0001f)) return fail("probability outside (0, 1]", round);
          sum += probs[i];
        }
        if (n > 0 && !(sum > score - 1e-3f && sum < score + 1e-3f)) return fail("score is not the sum of the probabilities", round);
        if (n > 0) {
          // the first draft token must follow the matched suffix somewhere in a live sequence
          bool seen = false;
          for (auto &kv : live) {
            const auto &s = kv.second;
            for (size_t at = 0; !seen && at + match_len < s.size(); ++at) {
              bool same = true;
              for (int j = 0; j < match_len && same; ++j) same = s[at + j] == ctx[clen - match_len + j];
              if (same && s[at + match_len] == ids[0]) seen = true;
            }
          }
          if (parents[0] != -1 || !seen) return fail("first draft token never follows the matched suffix", round);
        }
      }
      if (round % 16 == 15) {
        char msg[256];
        if (arctic_suffix_tree_check_integrity(tree, msg, sizeof msg) != 0) {
          std::fprintf(stderr, "suffix_stress: integrity: %s\n", msg);
          return fail("integrity check failed", round);
        }
        int nonempty = 0;
        for (auto &kv : live) nonempty += !kv.second.empty();
        if (arctic_suffix_tree_num_seqs(tree) != nonempty) return fail("num_seqs differs from the live sequences", round);
        (void)arctic_suffix_tree_estimate_memory(tree);
      }
    }
    arctic_suffix_tree_destroy(tree);
  }
  std::puts("ok");
  return 0;
}
