/*
 * arctic_suffix.h - C ABI of libarctic_suffix.so
 *
 * Suffix-tree speculation (SuffixDecoding) of ArcticInference: the native half of
 * arctic_inference.suffix_decoding.  CPU only; no GPU, torch or Python types cross
 * this boundary.  Each function below names the member of the reference's
 * SuffixTree class (csrc/suffix_decoding/suffix_tree.h:119-179, bound to Python in
 * csrc/suffix_decoding/bindings.cc:79-102) that it replaces.  Results - draft
 * tokens, parents, probabilities, score and match length - are those of the
 * reference on the same sequence of calls.
 *
 * A tree is not thread safe; different trees may be used from different threads.
 * Functions that can fail return 0 on success and a negative ARCTIC_SUFFIX_ERR_*.
 */
#ifndef ARCTIC_SUFFIX_H
#define ARCTIC_SUFFIX_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define ARCTIC_SUFFIX_ABI_VERSION 1

#define ARCTIC_SUFFIX_ERR_INVALID_ARGUMENT (-1)
#define ARCTIC_SUFFIX_ERR_NO_MEMORY (-2)

typedef struct arctic_suffix_tree arctic_suffix_tree;

int arctic_suffix_abi_version(void);

/* SuffixTree::SuffixTree(int max_depth)           suffix_tree.cc:27-29.  NULL if max_depth < 1. */
arctic_suffix_tree *arctic_suffix_tree_create(int max_depth);
void arctic_suffix_tree_destroy(arctic_suffix_tree *tree);

/* SuffixTree::num_seqs()                          suffix_tree.h:124-126 */
int arctic_suffix_tree_num_seqs(const arctic_suffix_tree *tree);

/* SuffixTree::append(seq_id, token)               suffix_tree.cc:297-490 */
int arctic_suffix_tree_append(arctic_suffix_tree *tree, int seq_id, int32_t token);

/* SuffixTree::extend(seq_id, tokens)              suffix_tree.cc:493-497 (extend / extend_ndarray,
 * bindings.cc:29-43) */
int arctic_suffix_tree_extend(arctic_suffix_tree *tree, int seq_id, const int32_t *tokens, int64_t num_tokens);

/* SuffixTree::remove(seq_id)                      suffix_tree.cc:500-581.  Unknown ids are ignored. */
int arctic_suffix_tree_remove(arctic_suffix_tree *tree, int seq_id);

/* SuffixTree::speculate(...)                      suffix_tree.cc:583-612 with _match_context,
 * _speculate_path and _speculate_tree (:815-905); speculate / speculate_ndarray, bindings.cc:46-76.
 *
 * The draft (Draft, suffix_tree.h:101-117) is written to the caller's arrays: token_ids, parents and
 * probs must each hold max(max_spec_tokens, 0) entries.  Returns the number of draft tokens (>= 0) or
 * a negative error.  *score and *match_len receive Draft::score and Draft::match_len. */
int arctic_suffix_tree_speculate(arctic_suffix_tree *tree, const int32_t *context, int64_t context_len,
                                 int max_spec_tokens, float max_spec_factor, float max_spec_offset,
                                 float min_token_prob, int use_tree_spec, int32_t *token_ids, int32_t *parents,
                                 float *probs, float *score, int *match_len);

/* SuffixTree::check_integrity()                   suffix_tree.cc:614-681, 683-813.  Returns 0 and an
 * empty message if every invariant holds, 1 and a message (truncated to capacity) otherwise. */
int arctic_suffix_tree_check_integrity(arctic_suffix_tree *tree, char *message, int capacity);

/* SuffixTree::estimate_memory()                   suffix_tree.cc:907-933.  Bytes held by this tree. */
size_t arctic_suffix_tree_estimate_memory(const arctic_suffix_tree *tree);

#ifdef __cplusplus
}
#endif
#endif /* ARCTIC_SUFFIX_H */
