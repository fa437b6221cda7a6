// Test infrastructure: C entry points around the REFERENCE's own SuffixTree class, so that the tests can
// drive it next to libarctic_suffix.so.  Compiled by `make -C oracle ref` together with the reference's
// csrc/suffix_decoding/suffix_tree.cc, taken from where it lies (REFERENCE=/root/reference by default),
// into oracle/_ref/libsuffix_ref.so.  Nothing of the reference is copied into this repository; the
// product never loads this library.
#include <cstdint>
#include <cstring>
#include <span>
#include <string>

#include "suffix_tree.h"  // the reference's header, found through -I$(REFERENCE)/csrc/suffix_decoding

extern "C" {

void *ref_suffix_tree_create(int max_depth) { return new SuffixTree(max_depth); }
void ref_suffix_tree_destroy(void *t) { delete static_cast<SuffixTree *>(t); }
int ref_suffix_tree_num_seqs(void *t) { return static_cast<SuffixTree *>(t)->num_seqs(); }

int ref_suffix_tree_extend(void *t, int seq_id, const int32_t *tokens, int64_t n) {
  static_cast<SuffixTree *>(t)->extend(seq_id, std::span<const int32_t>(tokens, (size_t)n));
  return 0;
}

int ref_suffix_tree_remove(void *t, int seq_id) {
  static_cast<SuffixTree *>(t)->remove(seq_id);
  return 0;
}

int ref_suffix_tree_speculate(void *t, const int32_t *context, int64_t n, int max_spec_tokens, float max_spec_factor,
                              float max_spec_offset, float min_token_prob, int use_tree_spec, int32_t *token_ids,
                              int32_t *parents, float *probs, float *score, int *match_len) {
  Draft d = static_cast<SuffixTree *>(t)->speculate(std::span<const int32_t>(context, (size_t)n), max_spec_tokens,
                                                    max_spec_factor, max_spec_offset, min_token_prob,
                                                    use_tree_spec != 0);
  const size_t k = d.token_ids.size();
  if (k) {
    std::memcpy(token_ids, d.token_ids.data(), k * sizeof(int32_t));
    std::memcpy(parents, d.parents.data(), k * sizeof(int32_t));
    std::memcpy(probs, d.probs.data(), k * sizeof(float));
  }
  *score = d.score;
  *match_len = d.match_len;
  return (int)k;
}

int ref_suffix_tree_check_integrity(void *t, char *message, int capacity) {
  const std::string problem = static_cast<SuffixTree *>(t)->check_integrity();
  if (message && capacity > 0) std::snprintf(message, (size_t)capacity, "%s", problem.c_str());
  return problem.empty() ? 0 : 1;
}

size_t ref_suffix_tree_estimate_memory(void *t) { return static_cast<SuffixTree *>(t)->estimate_memory(); }

}  // extern "C"
