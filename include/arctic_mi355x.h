/*
 * arctic_mi355x.h - C ABI of libarctic_mi355x.so
 *
 * MI355X (gfx950) replacement for the native half of ArcticInference's
 * csrc/custom_ops library: the SwiftKV bulk KV-cache write and the Arctic
 * speculator's fused element-wise operators.  Plain pointers and sizes only; no
 * torch, ATen or pybind types cross this boundary.  Every pointer named "device"
 * is an address in the current HIP device's memory; `stream` is a hipStream_t
 * passed as void* (NULL = the default stream).
 *
 * All entry points are asynchronous with respect to the host: they enqueue work
 * on `stream` and return.  They never allocate, free or synchronise, so they can
 * be recorded into a HIP graph.  They return 0 on success and a non-zero
 * ARCTIC_ERR_* code on failure; arctic_last_error() then holds a message for the
 * calling thread.  The library keeps no reference to any argument after return.
 *
 * Sizes are checked before anything is computed from them: row and token counts
 * must be below 2^31, widths (hidden, D_gate, columns, num_heads * head_size) at
 * most 2^30 / 2^28 / 2^30 / 2^24, block_size at most 2^20, num_blocks at most
 * 2^40, and every pitch non-negative and small enough that its last row still
 * starts inside a 2^47-byte address space.  A call outside these limits returns
 * ARCTIC_ERR_INVALID_ARGUMENT and launches nothing.
 *
 * Reference paths below are relative to the ArcticInference source tree.
 */
#ifndef ARCTIC_MI355X_H
#define ARCTIC_MI355X_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define ARCTIC_ABI_VERSION 2

/* element types of source / activation tensors */
#define ARCTIC_DTYPE_F32 0
#define ARCTIC_DTYPE_F16 1
#define ARCTIC_DTYPE_BF16 2

/* KV-cache storage types: the reference's Fp8KVCacheDataType
 * (csrc/custom_ops/dtype_fp8.cuh:14-18) selected from the strings
 * "auto" | "fp8" / "fp8_e4m3" | "fp8_e5m2" (csrc/custom_ops/quant_utils.cuh:532-567). */
#define ARCTIC_KV_AUTO 0
#define ARCTIC_KV_FP8_E4M3 1
#define ARCTIC_KV_FP8_E5M2 2

/* activation codes of arctic_speculator_add_ln_act */
#define ARCTIC_ACT_NONE 0
#define ARCTIC_ACT_GELU 1      /* erf form, nn.GELU() */
#define ARCTIC_ACT_GELU_TANH 2 /* tanh form */

#define ARCTIC_OK 0
#define ARCTIC_ERR_INVALID_ARGUMENT 1
#define ARCTIC_ERR_UNSUPPORTED 2
#define ARCTIC_ERR_LAUNCH 3

/* Largest num_layers one call accepts. */
#define ARCTIC_MAX_LAYERS 512

int arctic_abi_version(void);

/* Message of the last failure on the calling thread ("" if none). The pointer
 * stays valid until the next failing call on the same thread. */
const char *arctic_last_error(void);

/*
 * Bulk KV-cache write.  Replaces the host launcher + kernel
 *   reshape_and_cache_flash_bulk()            csrc/custom_ops/reshape_and_cache_flash_bulk.cu:77-144
 *   reshape_and_cache_flash_bulk_kernel<>     csrc/custom_ops/reshape_and_cache_flash_bulk.cu:12-60
 *   fp8::scaled_convert<>                     csrc/custom_ops/quant_utils.cuh:456-489,515-526
 * (declared in csrc/custom_ops/custom_ops.h:9-17, bound at torch_bindings.cpp:7-18).
 *
 * For every layer l < num_layers and token t < num_tokens with
 * slot = slot_mapping[t] >= 0 (negative slots are padding and are skipped):
 *   dst = cache_l + (slot / block_size) * block_stride + (slot % block_size) * n
 *   dst[i] = cvt(src[t * stride + l * n + i])   for i < n = num_heads * head_size
 * for both (keys, key_cache_ptrs, k_scale_ptrs) and (values, value_cache_ptrs,
 * v_scale_ptrs).  cvt is a raw copy for ARCTIC_KV_AUTO (cache element type ==
 * src_dtype) and fp8(float(x) / *scale_l) otherwise: IEEE fp32 division, round to
 * nearest even into OCP e4m3fn / e5m2, saturating to the largest finite value.
 *
 *   keys, values        device; [num_tokens, >= num_layers*n], row strides
 *                       key_stride / value_stride in ELEMENTS, inner dim dense
 *   key_cache_ptrs ...  HOST arrays of num_layers DEVICE pointers (the reference
 *                       builds the same four tables on its host stack, :104-118);
 *                       they are copied into the kernel arguments, so nothing is
 *                       uploaded separately and they may be freed on return.
 *                       Scale pointers address one fp32 each; they are read on the
 *                       device at execution time.  May be NULL for ARCTIC_KV_AUTO.
 *   slot_mapping        device int64[num_tokens]
 *   block_stride        ELEMENTS between consecutive cache blocks (same for K and
 *                       V); inside a block the layout is [block_size][n] dense
 *   num_blocks          blocks in every cache; a slot >= num_blocks * block_size
 *                       moves nothing, like a negative one (the reference writes
 *                       out of bounds there).  0 = unknown, slots are not checked.
 * Distinct valid slots are required for a deterministic result (as in the
 * reference).  num_layers == 0 or num_tokens == 0 is a successful no-op.
 */
int arctic_reshape_and_cache_flash_bulk(
    const void *keys, const void *values, int64_t key_stride,
    int64_t value_stride, const void *const *key_cache_ptrs,
    const void *const *value_cache_ptrs, const float *const *k_scale_ptrs,
    const float *const *v_scale_ptrs, const int64_t *slot_mapping,
    int64_t num_tokens, int num_layers, int num_heads, int head_size,
    int block_size, int64_t block_stride, int64_t num_blocks, int src_dtype,
    int kv_cache_dtype, void *stream);

/*
 * Helper of arctic_reshape_and_cache_flash_bulk_select: the inverse of an index list.
 *   row_map[t] = j where indices[j] == t, -1 for every other t < num_tokens
 * in one launch (indices outside [0, num_tokens) are ignored; of repeated indices one wins).  No counterpart in
 * the reference, whose index_select calls take logits_indices as it is (llama_swiftkv.py:663-679).
 *   row_map    device int64[num_tokens], written
 *   indices    device, num_indices entries of index_bytes (4 or 8) each, signed
 */
int arctic_build_row_map(int64_t *row_map, int64_t num_tokens, const void *indices, int index_bytes,
                         int64_t num_indices, void *stream);

/* Longest index list that arctic_reshape_and_cache_flash_bulk_select serves without a row map. */
#define ARCTIC_SELECT_SCAN_MAX_INDICES 2048

/*
 * The bulk KV-cache write with the row selection that follows it in the caller folded in.  Everything
 * arctic_reshape_and_cache_flash_bulk does, and in the same pass over the source
 *   keys_out[j] = keys[indices[j]],  values_out[j] = values[indices[j]]        for j < num_indices
 * which is
 *   index_fn("k_states", k_states, logits_indices), index_fn("v_states", v_states, logits_indices)
 *        arctic_inference/vllm/swiftkv/llama_swiftkv.py:663-679
 * so k_states and v_states are read once for both steps.  No single function of the reference corresponds to it.
 * The result is torch.index_select's for EVERY index in [0, num_src_rows), repeated ones included; a token is
 * copied whether or not its slot is padding.  Output rows whose index lies outside [0, num_src_rows) are left as
 * they were (index_select would raise).
 *
 *   indices            device, num_indices entries of index_bytes (4 or 8) each.
 *   row_map            NULL, or device int64[num_tokens] as arctic_build_row_map leaves it for `indices`.
 *                      NULL (num_indices <= ARCTIC_SELECT_SCAN_MAX_INDICES: one index per request of a serving
 *                      batch): every token's workgroup scans the index list itself for the output rows that name
 *                      its token; one launch, no workspace.  Given: a token's workgroup looks its output row up
 *                      in the map, whatever the list's length; rows that the map cannot serve (an index that is
 *                      repeated, a source row at or beyond num_tokens) are copied from the source by a few index
 *                      workgroups of the same launch.  With a row map `indices` may be NULL: the caller then
 *                      vouches that the indices are distinct and below num_tokens.
 *   num_src_rows       rows of keys / values (>= num_tokens)
 *   keys_out, values_out   device; num_indices rows of num_layers*n elements of src_dtype, out_*_stride ELEMENTS apart
 *   other arguments as arctic_reshape_and_cache_flash_bulk
 */
int arctic_reshape_and_cache_flash_bulk_select(
    const void *keys, const void *values, int64_t key_stride, int64_t value_stride,
    const void *const *key_cache_ptrs, const void *const *value_cache_ptrs,
    const float *const *k_scale_ptrs, const float *const *v_scale_ptrs,
    const int64_t *slot_mapping, int64_t num_tokens, int num_layers, int num_heads,
    int head_size, int block_size, int64_t block_stride, int64_t num_blocks, int src_dtype,
    int kv_cache_dtype, const int64_t *row_map, const void *indices, int index_bytes, int64_t num_indices,
    int64_t num_src_rows, void *keys_out, void *values_out, int64_t out_key_stride, int64_t out_value_stride,
    void *stream);

/* Most tokens one call of arctic_reshape_and_cache_flash_bulk_select_static accepts. */
#define ARCTIC_SELECT_STATIC_MAX_TOKENS 262144

/*
 * arctic_reshape_and_cache_flash_bulk_select for callers that cannot allocate device memory (code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc) and whose index lists may be longer than
 * ARCTIC_SELECT_SCAN_MAX_INDICES.  It has no counterpart in the reference.  The same result as
 * arctic_reshape_and_cache_flash_bulk_select; where that needs a row map (lists beyond
 * ARCTIC_SELECT_SCAN_MAX_INDICES) the map is built by this call and kept in a device array inside the library
 * (8 bytes x ARCTIC_SELECT_STATIC_MAX_TOKENS = 2 MiB on each GPU the library runs on, held until the process ends)
 * instead of a workspace of the caller's.  The call allocates and frees nothing; it enqueues one or two kernels on
 * `stream`.
 *
 *   num_tokens   at most ARCTIC_SELECT_STATIC_MAX_TOKENS, else ARCTIC_ERR_INVALID_ARGUMENT
 *   indices      device, num_indices entries of index_bytes (4 or 8) each; required when num_indices > 0
 *   other arguments as arctic_reshape_and_cache_flash_bulk_select
 *
 * Every argument is checked before the first kernel is enqueued; a call that is refused has launched nothing.
 *
 * All calls on one GPU share that GPU's array.  Calls on one stream use it one after the other.  A call on another
 * stream than the previous one first makes its stream wait (hipStreamWaitEvent) for an event that the library
 * recorded behind the previous call's kernels, so calls on streams that nothing else orders take turns at the
 * array instead of racing on it.  Under stream capture neither the wait nor the event is recorded: replays of graphs
 * that hold such a call must not overlap on one GPU, with each other or with an eager call; use the workspace form
 * where they may.
 * The first call with a long list on a device looks the array's address up (hipGetSymbolAddress) and creates that
 * event; make that call outside graph capture.
 */
int arctic_reshape_and_cache_flash_bulk_select_static(
    const void *keys, const void *values, int64_t key_stride, int64_t value_stride,
    const void *const *key_cache_ptrs, const void *const *value_cache_ptrs,
    const float *const *k_scale_ptrs, const float *const *v_scale_ptrs,
    const int64_t *slot_mapping, int64_t num_tokens, int num_layers, int num_heads,
    int head_size, int block_size, int64_t block_stride, int64_t num_blocks, int src_dtype,
    int kv_cache_dtype, const void *indices, int index_bytes, int64_t num_indices, int64_t num_src_rows,
    void *keys_out, void *values_out, int64_t out_key_stride, int64_t out_value_stride, void *stream);

/*
 * NVFP4-style KV-cache write for ONE layer: e2m1 values, two per byte (first element
 * in the low nibble), plus one e4m3 scale byte per 16 elements.  Replaces
 *   reshape_and_cache_flash_fp4()             csrc/custom_ops/reshape_and_cache_flash_fp4.cu:256-337
 *   reshape_and_cache_flash_kernel_fp4<>, quantize_16_to_fp4<>   :104-254
 * (custom_ops.h:19-27, torch_bindings.cpp:20-32).
 *
 * For every token t with slot = slot_mapping[t] >= 0, head h and group g of 16 elements:
 *   amax = max |x|;  scale byte = e4m3(amax / 6) (saturating);  SF = value of that byte
 *   nibble_i = e2m1(x_i / SF), round to nearest even, saturating at +-6 (0 if SF == 0)
 *   packed -> cache      + blk*block_stride     + off*page_stride     + h*head_stride     + g*8
 *   scale  -> scale cache + blk*(block_stride/8) + off*(page_stride/8) + h*(head_stride/8) + g
 * with blk = slot / block_size, off = slot % block_size.  Strides are in BYTES of the packed
 * cache: NHD [NB, block_size, H, D/2] passes page_stride = stride(1), head_stride = stride(2);
 * HND [NB, H, block_size, D/2] passes page_stride = stride(2), head_stride = stride(1).  The
 * reference's per-tensor k_scale / v_scale and kv_cache_dtype arguments have no effect there
 * and are not part of this call.  The two reciprocals (1/6, 1/SF) are correctly rounded here
 * and approximate (rcp.approx.ftz) in the reference.
 *
 *   key, value   device; [num_tokens, num_heads*head_size] F16 or BF16, row strides in ELEMENTS,
 *                16-byte aligned rows; head_size % 16 == 0
 *   num_blocks   blocks in each cache; a slot >= num_blocks * block_size moves nothing.
 *                0 = unknown, slots are not checked.
 */
int arctic_reshape_and_cache_flash_fp4(
    const void *key, const void *value, int64_t key_stride, int64_t value_stride,
    void *key_cache, void *value_cache, void *key_scale_cache,
    void *value_scale_cache, const int64_t *slot_mapping, int64_t num_tokens,
    int num_heads, int head_size, int block_size, int64_t block_stride,
    int64_t page_stride, int64_t head_stride, int64_t num_blocks, int dtype,
    void *stream);

/*
 * Speculator "LayerNorm" (an RMS norm with optional scale and shift).  Replaces
 *   speculator_ln_cuda()                      csrc/custom_ops/speculator_ln.cu:152-252
 *   spec_ln_vec_kernel<> / spec_ln_scalar_kernel<>   csrc/custom_ops/speculator_ln.cu:21-150
 * (custom_ops.h:29-32, torch_bindings.cpp:33-37).
 *
 *   y = x * rsqrt(mean(x^2) + eps);  if (weight) y *= weight;  if (bias) y += bias
 * in fp32, rounded to nearest even into `dtype` (F16 or BF16).
 *
 *   in       device; rows of `hidden` elements, in_row_stride ELEMENTS apart
 *   out      device; rows * hidden elements, dense
 *   weight, bias   device [hidden] or NULL
 */
int arctic_speculator_ln(void *out, const void *in, const void *weight,
                         const void *bias, int64_t rows, int hidden,
                         int64_t in_row_stride, float eps, int dtype,
                         void *stream);

/*
 * The same norm with the element-wise steps the speculator runs around it folded
 * in.  No single function of the reference corresponds to it; it stands for the
 * PyTorch sequences
 *   states.add_(z, alpha=emb_weight / state_weight); activation(ln(states))
 *        arctic_inference/vllm/spec_dec/arctic_speculator.py:296-307, 809-816
 *   ln0(previous_hidden_states) / SQRT2
 *        arctic_inference/vllm/spec_dec/arctic_speculator.py:296-297, 733-734
 * and rounds to `dtype` wherever those sequences hold a tensor of that type:
 *   x = z ? round(in + alpha * z) : in
 *   y = round(x * rsqrt(mean(x^2) + eps) [* weight] [+ bias])
 *   if (activation) y = round(gelu(y));   if (out_scale != 1) y = round(y * out_scale)
 * `in` is not modified.
 *
 *   z            device; rows of `hidden` elements, z_row_stride ELEMENTS apart, or NULL
 *   activation   ARCTIC_ACT_*
 *   other arguments as arctic_speculator_ln
 */
int arctic_speculator_add_ln_act(void *out, const void *in, const void *z,
                                 const void *weight, const void *bias,
                                 int64_t rows, int hidden, int64_t in_row_stride,
                                 int64_t z_row_stride, float alpha, float eps,
                                 int activation, float out_scale, int dtype,
                                 void *stream);

/*
 * arctic_speculator_add_ln_act with z looked up in an embedding table: row r adds
 * emb_table[clamp(token_ids[r], 0, num_embeddings - 1)], which is
 *   z = self.emb[i](last_tokens); states.add_(z, alpha=...); activation(ln(states))
 *        arctic_inference/vllm/spec_dec/arctic_speculator.py:301-309
 * with the clamp the caller applies to last_tokens (:845, :862) in the same launch, and no z tensor.
 *
 *   emb_table    device; num_embeddings rows of `hidden` elements, emb_row_stride ELEMENTS apart
 *   token_ids    device, int64 [rows]
 */
int arctic_speculator_embed_add_ln_act(void *out, const void *in, const void *emb_table,
                                       const int64_t *token_ids, const void *weight,
                                       const void *bias, int64_t rows, int hidden,
                                       int64_t in_row_stride, int64_t emb_row_stride,
                                       int64_t num_embeddings, float alpha, float eps,
                                       int activation, float out_scale, int dtype,
                                       void *stream);

/*
 * Fused LSTM-style gate / cell / state update.  Replaces
 *   sum_lstm_cuda()                           csrc/custom_ops/sum_lstm.cu:293-473
 *   sum_lstm_vec_kernel<> / sum_lstm_scalar_kernel<>   csrc/custom_ops/sum_lstm.cu:28-291
 * (custom_ops.h:34-41, torch_bindings.cpp:39-50).
 *
 * Per row, with gate order f | i | o | c along the 4*D dimension:
 *   pre_g    = states_g + alpha * z4_g
 *   c_new    = prev_cell * sigmoid(pre_f)
 *              + gelu(rmsnorm(pre_c; w_cell, b_cell, eps_cell)) * sigmoid(pre_i)
 *   out_cell = round(c_new)
 *   out_state = round(gelu(rmsnorm(out_cell; w_state, b_state, eps_state)) * sigmoid(pre_o))
 * where rmsnorm(v; w, b, eps) = v * rsqrt(mean(v^2) + eps) [* w] [+ b]; the mean
 * for the state norm is taken over the unrounded c_new while the normalised
 * values are the rounded out_cell, as in the reference (:136-137,:163,:174).
 * gelu is the exact erf form, or the tanh form when fast_gelu != 0.
 *
 *   states, z4     device; rows of 4*D elements, s_stride / z_stride apart
 *   prev_cell      device; rows of D elements, pc_stride apart.  NULL = a cell of zeros, which is what the
 *                  speculator starts every proposal round from (arctic_speculator.py:899-903): the result is that
 *                  of a zero tensor bit for bit, without the tensor, its clearing or its read; pc_stride is ignored
 *   out_state, out_cell   device; rows of D elements, out_stride apart
 *   w_cell, b_cell, w_state, b_state   device [>= D] or NULL
 * All strides are in ELEMENTS.  dtype is F16 or BF16.
 */
int arctic_sum_lstm(void *out_state, void *out_cell, const void *states,
                    const void *z4, const void *prev_cell, const void *w_cell,
                    const void *b_cell, const void *w_state,
                    const void *b_state, int64_t rows, int D, int64_t s_stride,
                    int64_t z_stride, int64_t pc_stride, int64_t out_stride,
                    float alpha, float eps_cell, float eps_state, int fast_gelu,
                    int dtype, void *stream);

/*
 * sum_lstm with the embedding term given ONCE per token.  The speculator builds
 *   z4 = forget_emb(tokens).repeat(1, 1, 4)       arctic_inference/vllm/spec_dec/arctic_speculator.py:744
 * i.e. the same [rows, D] row under all four gates, and passes it to sum_lstm.  This entry
 * point takes that [rows, D] row itself (z, rows z_stride ELEMENTS apart) and adds it to every
 * gate; everything else, and every output bit, is as arctic_sum_lstm with z4 = repeat(z, 4).
 * It fuses the caller's repeat() into the operator (6*D fewer bytes read per row and no z4
 * tensor); the reference has no operator of this shape.
 */
int arctic_sum_lstm_shared_z(void *out_state, void *out_cell, const void *states,
                             const void *z, const void *prev_cell, const void *w_cell,
                             const void *b_cell, const void *w_state,
                             const void *b_state, int64_t rows, int D, int64_t s_stride,
                             int64_t z_stride, int64_t pc_stride, int64_t out_stride,
                             float alpha, float eps_cell, float eps_state, int fast_gelu,
                             int dtype, void *stream);

/*
 * arctic_sum_lstm_shared_z with the embedding lookup folded in: row r uses
 * emb_table[clamp(token_ids[r], 0, num_embeddings - 1)] as its z, which is
 *   z4 = self.forget_emb[i](last_tokens).repeat(1, 1, 4)
 *        arctic_inference/vllm/spec_dec/arctic_speculator.py:744
 * and the clamp of last_tokens (:845, :862) inside the operator: no z and no z4 tensor, one launch less.
 *
 *   emb_table    device; num_embeddings rows of D elements, emb_stride ELEMENTS apart
 *   token_ids    device, int64 [rows]
 */
int arctic_sum_lstm_embedded(void *out_state, void *out_cell, const void *states,
                             const void *emb_table, const int64_t *token_ids,
                             const void *prev_cell, const void *w_cell, const void *b_cell,
                             const void *w_state, const void *b_state, int64_t rows, int D,
                             int64_t s_stride, int64_t emb_stride, int64_t pc_stride,
                             int64_t out_stride, int64_t num_embeddings, float alpha,
                             float eps_cell, float eps_state, int fast_gelu, int dtype,
                             void *stream);

/*
 * Row gather / scatter over up to 8 tensors in one launch.  No native function of
 * the reference corresponds to it; it stands for the PyTorch calls either side of
 * the bulk KV write in LlamaSwiftKVModel:
 *   gather   torch.index_select(tensor, 0, logits_indices, out=buffer[:batch]) for
 *            hidden_states, residual, positions, k_states, v_states
 *            arctic_inference/vllm/swiftkv/llama_swiftkv.py:663-679
 *   scatter  orig_hidden_states[logits_indices] = hidden_states[:batch_size]
 *            arctic_inference/vllm/swiftkv/llama_swiftkv.py:733-742
 *
 * gather  (scatter == 0): dst_t row r           <- src_t row indices[r]
 * scatter (scatter != 0): dst_t row indices[r]  <- src_t row r
 * for r in [0, num_indices) and every tensor t.  Bytes are copied as they are.  An
 * index outside [0, num_indexed_rows) moves nothing (torch raises a device-side
 * assertion there).  Equal indices in a scatter race, as in torch.
 *
 *   src, dst            HOST arrays [num_tensors] of device pointers (row 0 of each tensor)
 *   row_bytes           HOST array: bytes per row of each tensor (0 skips the tensor)
 *   *_row_stride_bytes  HOST arrays: bytes between rows
 *   indices             device, num_indices entries of index_bytes (4 or 8) each, signed
 *   num_indices         number of rows moved per tensor (any count; more than 65535 are walked by a loop in the kernel)
 *   num_indexed_rows    rows of the indexed side (sources of a gather, destinations of a scatter)
 */
int arctic_gather_rows(int num_tensors, const void *const *src, void *const *dst,
                       const int64_t *row_bytes, const int64_t *src_row_stride_bytes,
                       const int64_t *dst_row_stride_bytes, const void *indices,
                       int index_bytes, int64_t num_indices, int64_t num_indexed_rows,
                       int scatter, void *stream);

/*
 * Row-wise argmax with clamping.  No native function of the reference corresponds to it; it stands for the
 * token selection that ends every speculator step,
 *   last_tokens = torch.argmax(logits, dim=-1); last_tokens.clamp_(0, vocab_size - 1)
 *        arctic_inference/vllm/spec_dec/arctic_speculator.py:846-848, 862
 * with torch's rules: the largest value wins, the lowest index among equal values, and a NaN beats every
 * number (the first NaN wins).
 *
 *   out         device int64[rows]: min(argmax_j logits[r][j], max_index)
 *   logits      device; rows of `cols` elements (F32, F16 or BF16), row_stride ELEMENTS apart
 */
int arctic_argmax_clamp(int64_t *out, const void *logits, int64_t rows, int cols,
                        int64_t row_stride, int64_t max_index, int dtype, void *stream);

#ifdef __cplusplus
}
#endif

#endif /* ARCTIC_MI355X_H */
