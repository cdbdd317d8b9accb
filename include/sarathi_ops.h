/*
 * sarathi_ops.h -- C ABI of the gfx950 (MI355X) op library that stands in for
 * Sarathi-Serve's csrc/ ops.
 *
 * Conventions, all entry points:
 *   - plain pointers to DEVICE memory, sizes in ELEMENTS, strides in ELEMENTS;
 *   - `stream` is a hipStream_t passed as void* (NULL = the null stream); the
 *     call enqueues its kernel(s) on that stream and returns without waiting;
 *   - nothing is allocated or freed, no global state is mutated, calls are
 *     re-entrant; the current HIP device must be the one owning the pointers;
 *   - the return value is 0 on success or a negative SARATHI_ERR_* code; no
 *     exceptions cross this boundary.  A size of zero tokens is a successful
 *     no-op.
 *   - `dtype` is a SARATHI_DTYPE_* code and applies to every floating tensor of
 *     the call.  16-byte vector paths are chosen when pointers and strides
 *     allow; otherwise an element-wise path computes the same results.
 */
#ifndef SARATHI_OPS_H_
#define SARATHI_OPS_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SARATHI_OPS_ABI_VERSION 1

/* element types of the floating tensors (csrc/dispatch_utils.h:7-14) */
#define SARATHI_DTYPE_F32 0
#define SARATHI_DTYPE_F16 1
#define SARATHI_DTYPE_BF16 2

/* element types of topk_ids (csrc/dispatch_utils.h:16-24) */
#define SARATHI_IDTYPE_U8 0
#define SARATHI_IDTYPE_I8 1
#define SARATHI_IDTYPE_I16 2
#define SARATHI_IDTYPE_I32 3
#define SARATHI_IDTYPE_I64 4

#define SARATHI_OK 0
#define SARATHI_ERR_INVALID_ARG (-1) /* null pointer, negative size, bad stride */
#define SARATHI_ERR_UNSUPPORTED (-2) /* unknown dtype code or shape outside limits */
#define SARATHI_ERR_LAUNCH (-3)      /* the HIP runtime rejected the launch */
#define SARATHI_ERR_SCRATCH_LIMIT (-4) /* input needs more than the fixed scratch of a *_static entry */

/* Largest num_experts accepted by the two MoE routing entry points. */
#define SARATHI_MOE_MAX_EXPERTS 1024

int sarathi_ops_abi_version(void);
const char* sarathi_ops_strerror(int code);

/*
 * Replaces rms_norm(out, input, weight, epsilon): csrc/layernorm.cpp:3-14,
 * host csrc/layernorm_kernels.cu:39-62.
 *   out[t,i] = T( T(x[t,i] * rsqrt(mean_i(x[t,:]^2) + eps)) * w[i] ),
 * sum of squares in fp32.  Rows of `input`/`out` start row_stride elements
 * apart (the reference assumes hidden_size; pass hidden_size for that).
 */
int sarathi_rms_norm(void* out, const void* input, const void* weight, float epsilon,
                     int64_t num_tokens, int64_t hidden_size, int64_t input_row_stride,
                     int64_t out_row_stride, int dtype, void* stream);

/*
 * New entry next to rms_norm; fuses the reference decoder layer's
 * `hidden = residual + hidden; residual = hidden; hidden = rms_norm(hidden)`
 * (sarathi/model_executor/models/llama.py:248-252).  In place on both tensors:
 *   residual <- T(input + residual);  input <- rms_norm(residual).
 */
int sarathi_fused_add_rms_norm(void* input, void* residual, const void* weight, float epsilon,
                               int64_t num_tokens, int64_t hidden_size,
                               int64_t input_row_stride, int64_t residual_row_stride,
                               int dtype, void* stream);

/*
 * Replaces silu_and_mul(out, input): csrc/activation.cpp:3-19, host
 * csrc/activation_kernels.cu:29-48.  input [num_tokens, 2*d], out
 * [num_tokens, d]; out = T( T(silu(x)) * y ) with x = input[:, :d],
 * y = input[:, d:].
 */
int sarathi_silu_and_mul(void* out, const void* input, int64_t num_tokens, int64_t d,
                         int64_t input_row_stride, int64_t out_row_stride, int dtype,
                         void* stream);

/*
 * Replace gelu_new(out, input) and gelu_fast(out, input):
 * csrc/activation.cpp:7-28, csrc/activation_kernels.cu:86-114.
 * Contiguous [num_tokens, d] in and out.
 * 16-bit dtypes, 12 Mi elements or more: the result is read from a table of the op over all
 * 65536 bit patterns (same bits as the arithmetic path).  The library keeps the four tables
 * (two ops x two dtypes, 128 KiB each) in a file-scope device array; the first such call on a
 * device launches the kernel that fills the table on its stream, and until that kernel has
 * finished, calls on other streams and calls under stream capture use the arithmetic path.
 * Nothing is allocated on the device and nothing waits.
 */
int sarathi_gelu_new(void* out, const void* input, int64_t num_tokens, int64_t d, int dtype,
                     void* stream);
int sarathi_gelu_fast(void* out, const void* input, int64_t num_tokens, int64_t d, int dtype,
                      void* stream);

/*
 * Replaces rotary_embedding(positions, query, key, head_size, cos_sin_cache,
 * is_neox): csrc/pos_encoding.cpp:3-16, host csrc/pos_encoding_kernels.cu:80-127.
 * In place on query [num_tokens, num_heads*head_size] and key
 * [num_tokens, num_kv_heads*head_size], whose rows start query_stride /
 * key_stride elements apart (views of a packed qkv buffer are the normal
 * case).  cos_sin_cache is [max_position, rot_dim] = cos[0:rot/2] || sin[0:rot/2]
 * per row, in the tensors' dtype; positions are int64 row numbers of that
 * cache and are not range-checked.  Elements at or above rot_dim in each head
 * are left untouched.
 */
int sarathi_rotary_embedding(const int64_t* positions, void* query, void* key,
                             const void* cos_sin_cache, int64_t num_tokens, int num_heads,
                             int num_kv_heads, int head_size, int rot_dim,
                             int64_t query_stride, int64_t key_stride, int is_neox, int dtype,
                             void* stream);

/*
 * Replaces topk_softmax(topk_weights, topk_indices, token_expert_indices,
 * gating_output): csrc/moe.cpp:3-8, host csrc/moe_topk_softmax_kernels.cu:476-503.
 * gating_output fp32 [num_tokens, num_experts]; outputs [num_tokens, topk] in
 * descending probability order, lower expert index first on equal
 * probabilities; token_expert_indices[t,j] = j*num_tokens + t.  No workspace
 * is needed for any num_experts in [1, SARATHI_MOE_MAX_EXPERTS]; topk must be
 * in [1, num_experts].  renormalize = 0 reproduces the reference op (raw
 * softmax probabilities); renormalize = 1 additionally divides each row's
 * weights by their sum, which the reference's caller does as a separate
 * tensor op (sarathi/model_executor/layers/fused_moe/fused_moe.py:371-372).
 */
int sarathi_topk_softmax(float* topk_weights, int32_t* topk_indices,
                         int32_t* token_expert_indices, const float* gating_output,
                         int64_t num_tokens, int num_experts, int topk, int renormalize,
                         void* stream);

/*
 * Replaces moe_align_block_size(topk_ids, num_experts, block_size,
 * sorted_token_ids, experts_ids, num_tokens_post_pad): csrc/moe.cpp:10-17, host
 * csrc/moe_align_block_size_kernels.cu:112-135.  Stable counting sort of the
 * `numel` flat ids by expert, each expert's run padded to a multiple of
 * block_size.  sorted_token_ids has sorted_len >= numel + E*(block_size-1)
 * int32 slots, expert_ids has expert_ids_len >= ceil(that / block_size).
 * Slots of sorted_token_ids that hold no token keep the caller's contents
 * when fill_pad = 0 (the reference's contract: the caller pre-fills with
 * numel, fused_moe.py:195) or are set to numel by this call when fill_pad = 1.
 * expert_ids entries at or above num_tokens_post_pad / block_size are left
 * untouched.  Ids outside [0, num_experts) are skipped (the reference's
 * behaviour for them is undefined).
 *
 * `workspace` is optional device scratch of `workspace_bytes` bytes (4-byte
 * aligned, contents irrelevant on entry and exit).  Up to 32 768 ids of at most 256 experts the
 * sort is one launch of several independent workgroups and uses no scratch.  Beyond that, with a
 * workspace of at least sarathi_moe_align_workspace_bytes() bytes, the input is spread over the
 * whole GPU in three launches; without one the sort runs in a single workgroup.  Results are
 * identical either way.
 */
int sarathi_moe_align_block_size(const void* topk_ids, int id_dtype, int64_t numel,
                                 int num_experts, int block_size, int32_t* sorted_token_ids,
                                 int64_t sorted_len, int32_t* expert_ids,
                                 int64_t expert_ids_len, int32_t* num_tokens_post_pad,
                                 int fill_pad, void* workspace, int64_t workspace_bytes,
                                 void* stream);

/*
 * Scratch bytes sarathi_moe_align_block_size can make use of for this input
 * size; 0 when a path without scratch will be taken anyway.  The reference
 * allocates a workspace in the same way for topk_softmax
 * (csrc/moe_topk_softmax_kernels.cu:486-492).
 */
int64_t sarathi_moe_align_workspace_bytes(int64_t numel, int num_experts);

/*
 * sarathi_moe_align_block_size for callers that cannot allocate device memory or bring a
 * workspace (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).
 * It has no counterpart in the reference.  Same arguments, results and error codes as
 * sarathi_moe_align_block_size without `workspace`; the scratch of the three-launch path (inputs
 * above 32 768 ids, or above 16 384 with more than 256 experts) is a fixed array of SARATHI_MOE_ALIGN_STATIC_SCRATCH_BYTES that lives in
 * the library's device image (every GPU the library runs on holds it until the process ends).
 * The call allocates and frees nothing.  Inputs for which
 * sarathi_moe_align_workspace_bytes(numel, num_experts) exceeds that size are refused with
 * SARATHI_ERR_SCRATCH_LIMIT (with 255 experts or fewer every numel fits; 1024 experts fit up to
 * 129 024 ids) and nothing is launched.  All calls on one GPU share the one array: calls that
 * overlap on the same GPU (different streams, or different host threads without ordering between
 * their launches) race on it; calls on one stream are safe.  The array's contents between calls
 * are irrelevant: every word a call reads it has written before.  This is the one entry point of
 * the library that keeps state (the per-device address of the array, looked up on the first call on
 * each device).  That lookup is host work: call the entry point once, eagerly, on every device
 * before capturing a call into a HIP graph (inputs of at most 32 768 ids never touch the array and
 * do not trigger the lookup, so use a larger one or rely on an earlier uncaptured call).
 */
#define SARATHI_MOE_ALIGN_STATIC_SCRATCH_BYTES (1 << 20)
int sarathi_moe_align_block_size_static(const void* topk_ids, int id_dtype, int64_t numel,
                                        int num_experts, int block_size,
                                        int32_t* sorted_token_ids, int64_t sorted_len,
                                        int32_t* expert_ids, int64_t expert_ids_len,
                                        int32_t* num_tokens_post_pad, int fill_pad,
                                        void* stream);

/*
 * Replaces grouped_topk(hidden_states, gating_output, topk, renormalize, num_expert_group,
 * topk_group), which the reference writes with tensor ops
 * (sarathi/model_executor/layers/fused_moe/fused_moe.py:377-408): softmax over the experts; the
 * experts form num_expert_group consecutive groups of equal size; the topk_group groups with the
 * largest member probability are kept and every other expert's probability is replaced by 0;
 * then the top-k of the result, optionally divided by their sum.  The reference's torch.topk
 * (sorted=False) leaves the output order and the choice among equal values unspecified; here
 * outputs are in descending order and equal values resolve to the lower index.
 * num_experts <= SARATHI_MOE_MAX_EXPERTS, num_expert_group <= 64 and a divisor of num_experts.
 */
int sarathi_grouped_topk(float* topk_weights, int32_t* topk_indices, const float* gating_output,
                         int64_t num_tokens, int num_experts, int topk, int num_expert_group,
                         int topk_group, int renormalize, void* stream);

/*
 * New entry: sarathi_topk_softmax followed by sarathi_moe_align_block_size (on the int32 ids it
 * just produced) in ONE launch, for the reference's per-layer sequence
 * fused_topk -> moe_align_block_size (sarathi/model_executor/layers/fused_moe/fused_moe.py:346-373
 * and :151-204).  Outputs are bit-identical to the two separate calls.  `counter` is one uint32
 * of device memory that is zero before the first call; the call leaves it zero again.  Calls
 * that share a counter must not overlap (use one counter per stream).  The single launch is taken
 * up to 1024 ids and a power-of-two expert count up to 16, where it is faster; with counter =
 * NULL or any other shape the two stand-alone kernels are launched instead.
 */
int sarathi_fused_topk_align(float* topk_weights, int32_t* topk_indices,
                             int32_t* token_expert_indices, const float* gating_output,
                             int64_t num_tokens, int num_experts, int topk, int renormalize,
                             int block_size, int32_t* sorted_token_ids, int64_t sorted_len,
                             int32_t* expert_ids, int64_t expert_ids_len,
                             int32_t* num_tokens_post_pad, int fill_pad, uint32_t* counter,
                             void* stream);

/*
 * Grouped expert GEMM that consumes moe_align_block_size's outputs; replaces the
 * Triton kernel launched by invoke_fused_moe_kernel
 * (sarathi/model_executor/layers/fused_moe/fused_moe.py:15-148, :207-260).
 * For every block of block_m consecutive slots of sorted_token_ids (one expert,
 * expert_ids[block]):  C[slot, :] = A[slot / top_k, :] @ B[expert]^T, fp32
 * accumulation, then the epilogue, rounded to `dtype`.  Epilogues:
 *   SARATHI_MOE_EPILOGUE_NONE           nothing (the reference's mul_routed_weight = False)
 *   SARATHI_MOE_EPILOGUE_ROUTED_WEIGHT  times topk_weights[slot] (mul_routed_weight = True)
 *   SARATHI_MOE_EPILOGUE_SILU_AND_MUL   (new) B holds gate rows [0, N/2) and up rows [N/2, N); C is
 *       [num_valid_tokens, N/2] = silu_and_mul of the [.., N] product, with the rounding points
 *       of the unfused sequence GEMM -> silu_and_mul (fused_moe.py:499-520), so results are
 *       bit-identical to it while the [.., N] intermediate never reaches memory.  N/2 must be a
 *       multiple of 4 (of 32 with packed weights).
 * A [tokens, K] with rows a_row_stride elements apart; A MUST hold at least
 * ceil(num_valid_tokens / top_k) rows (the kernel derives the extent of its reads from that
 * figure, not from the allocation) and top_k must be positive.  B
 * [E, N, K] K-contiguous with experts b_expert_stride elements apart, C
 * [num_valid_tokens, N] with rows c_row_stride apart (num_valid_tokens =
 * tokens * topk; slots holding a larger id are padding and skipped).
 * block_m must be the block_size moe_align_block_size ran with and one of 32,
 * 64, 128, 256; dtype bf16 or fp16; K a multiple of 64, N a multiple of 4.
 * dtype fp32 (the reference's fused_experts admits float32 tensors,
 * fused_moe.py:430) runs a plain float32 matrix-core kernel: row-major weights,
 * epilogue NONE or ROUTED_WEIGHT, block_m any multiple of 32, K, the strides and
 * N's pieces multiples of 4; the output is rounded through float16 before it is
 * stored, as the reference's kernel does with its compute_type for every dtype
 * but bfloat16 (fused_moe.py:142, 466).
 *
 * b_layout: SARATHI_MOE_B_ROW_MAJOR is the reference's [E, N, K] tensor.
 * SARATHI_MOE_B_PACKED is the same weights re-tiled once, offline, into the
 * order the matrix cores consume them: per expert ceil(N/32) row tiles, each
 * K/16 blocks of 1 KiB, a block holding for lane l = (n mod 32) + 32*((k mod 16)/8)
 * the 8 elements k mod 8 = 0..7 (rows beyond N zero); b_expert_stride then
 * counts ceil(N/32)*32*K elements.  Same results; within a few
 * per cent of the row-major path at every batch size.
 */
#define SARATHI_MOE_B_ROW_MAJOR 0
#define SARATHI_MOE_B_PACKED 1
#define SARATHI_MOE_EPILOGUE_NONE 0
#define SARATHI_MOE_EPILOGUE_ROUTED_WEIGHT 1
#define SARATHI_MOE_EPILOGUE_SILU_AND_MUL 2
int sarathi_moe_grouped_gemm(const void* a, const void* b, void* c, const float* topk_weights,
                             const int32_t* sorted_token_ids, const int32_t* expert_ids,
                             const int32_t* num_tokens_post_padded, int64_t num_valid_tokens,
                             int64_t sorted_len, int64_t n, int64_t k, int64_t a_row_stride,
                             int64_t b_expert_stride, int64_t c_row_stride, int block_m,
                             int top_k, int epilogue, int b_layout, int dtype, void* stream);

/*
 * Replaces the torch.sum(intermediate_cache3, dim=1, out=...) that ends fused_experts
 * (sarathi/model_executor/layers/fused_moe/fused_moe.py:539-543): out[t, :] = sum over j of
 * input[t, j, :] for the top_k expert outputs of token t, fp32 accumulation in ascending j, one
 * rounding to the tensor dtype.  input row (t, j) starts at t * in_token_stride + j * in_k_stride
 * elements, out row t at t * out_row_stride; rows are `hidden` contiguous elements.
 * dtype: SARATHI_DTYPE_F32 / F16 / BF16.
 */
int sarathi_moe_sum(void* out, const void* input, int64_t num_tokens, int64_t top_k,
                    int64_t hidden, int64_t in_token_stride, int64_t in_k_stride,
                    int64_t out_row_stride, int dtype, void* stream);

/*
 * Paged KV cache (NHD page layout: entry e of page p holds [num_kv_heads, head_size] elements and
 * starts page_stride*p + entry_stride*e elements after k_cache, resp. v_cache; the reference's
 * cache tensor [num_pages, 2, page_size, num_kv_heads, head_size],
 * sarathi/model_executor/attention/flashinfer_attention_wrapper.py:70-78, has k_cache = cache,
 * v_cache = cache + page_size*num_kv_heads*head_size, page_stride = 2*page_size*num_kv_heads*
 * head_size, entry_stride = num_kv_heads*head_size).
 *
 * The three calls below replace the flashinfer (flashinfer-python==0.4.1, requirements.txt:18)
 * functions the reference's attention wrapper calls.
 *
 * sarathi_get_seq_lens replaces get_seq_lens (flashinfer_attention_wrapper.py:213-217):
 *   seq_lens[i] = max(kv_indptr[i+1] - kv_indptr[i] - 1, 0) * page_size + kv_last_page_len[i].
 * sarathi_get_batch_indices_positions replaces get_batch_indices_positions
 * (flashinfer_attention_wrapper.py:220-226): for every request b and token i in
 * [append_indptr[b], append_indptr[b+1]): batch_indices[i] = b and positions[i] =
 * i + seq_lens[b] - append_indptr[b+1] (the request's last appended token is its last kv entry).
 * Tokens outside [append_indptr[0], append_indptr[num_seqs]) are left untouched.
 * sarathi_append_paged_kv_cache replaces append_paged_kv_cache(..., kv_layout="NHD")
 * (flashinfer_attention_wrapper.py:262-273): token i's key and value rows are copied to entry
 * positions[i] % page_size of page kv_indices[kv_indptr[batch_indices[i]] + positions[i] /
 * page_size].  Indices are not range-checked.
 *
 * sarathi_get_kv_slot_mapping (new) resolves that lookup once per batch:
 * slot_mapping[i] = page * page_size + entry.  The page table of a batch is the same for every
 * layer, so the append entry points accept the vector in place of the four index arrays
 * (slot_mapping != NULL: batch_indices, positions, kv_indices and kv_indptr are ignored and may be
 * NULL) and then need one index load per token instead of three dependent ones.  The mapping is
 * int32: num_pages * page_size must stay below 2^31.
 */
int sarathi_get_kv_slot_mapping(const int32_t* batch_indices, const int32_t* positions,
                                const int32_t* kv_indices, const int32_t* kv_indptr,
                                int32_t* slot_mapping, int64_t nnz, int page_size, void* stream);
int sarathi_get_seq_lens(const int32_t* kv_indptr, const int32_t* kv_last_page_len,
                         int32_t* seq_lens, int64_t num_seqs, int page_size, void* stream);
int sarathi_get_batch_indices_positions(const int32_t* append_indptr, const int32_t* seq_lens,
                                        int32_t* batch_indices, int32_t* positions,
                                        int64_t num_seqs, int64_t nnz, void* stream);
int sarathi_append_paged_kv_cache(const void* append_key, const void* append_value,
                                  const int32_t* batch_indices, const int32_t* positions,
                                  void* k_cache, void* v_cache, const int32_t* kv_indices,
                                  const int32_t* kv_indptr, const int32_t* slot_mapping,
                                  int64_t nnz, int num_kv_heads,
                                  int head_size, int page_size, int64_t key_stride,
                                  int64_t value_stride, int64_t page_stride, int64_t entry_stride,
                                  int dtype, void* stream);

/*
 * New entry: sarathi_rotary_embedding followed by sarathi_append_paged_kv_cache in one launch,
 * i.e. the reference's rotary call (sarathi/model_executor/models/llama.py:178) plus the cache
 * append of the attention wrapper (flashinfer_attention_wrapper.py:262-273).  query is rotated in
 * place for all num_tokens rows; the first num_append_tokens rows' rotated keys and their values
 * are written to the cache (the reference appends key[:num_total_tokens]).  key itself is
 * rotated in place only when write_key != 0 (attention reads keys from the cache, so the
 * in-place result is normally dead) or for rows at or above num_append_tokens.  Results in
 * query / key / cache are bit-identical to the two separate calls.
 */
int sarathi_rotary_embedding_append_paged_kv(
    const int64_t* positions, void* query, void* key, const void* value, const void* cos_sin_cache,
    const int32_t* batch_indices, const int32_t* append_positions, void* k_cache, void* v_cache,
    const int32_t* kv_indices, const int32_t* kv_indptr, const int32_t* slot_mapping,
    int64_t num_tokens, int64_t num_append_tokens, int num_heads, int num_kv_heads, int head_size,
    int rot_dim, int64_t query_stride, int64_t key_stride, int64_t value_stride, int page_size,
    int64_t page_stride, int64_t entry_stride, int is_neox, int write_key, int dtype,
    void* stream);

/*
 * No counterpart in the reference: spreads every expert's slots evenly over the blocks that
 * sarathi_moe_align_block_size gave it (fused_moe.py:151-204 fills them greedily, so an expert's
 * last block is often nearly empty; such blocks cost the grouped GEMM far more than their share
 * of the work, see csrc/moe_balance.hip).  sorted_in / expert_ids / num_tokens_post_pad are
 * moe_align_block_size's outputs for `block_size`, padding entries equal to `pad_value` (the
 * caller's numel).  sorted_out (another buffer of sorted_len entries) receives the same slots in
 * the same order with an expert's ceil(cnt / granule) tiles of `granule` slots dealt to its nb
 * blocks as evenly as they go (the first tiles % nb blocks take one tile more), padding elsewhere
 * and from num_tokens_post_pad on; expert_ids and num_tokens_post_pad stay valid for it.
 * rows_per_block = R > 1 deals the tiles over the expert's nb * R ranges of block_size / R slots
 * instead (each range filled from its own start), for a GEMM kernel whose waves split a block's
 * slots R ways: R = sarathi_moe_gemm_slot_rows(block_size, b_layout).  granule must divide
 * block_size / R.
 */
int sarathi_moe_balance_blocks(const int32_t* sorted_in, int32_t* sorted_out,
                               const int32_t* expert_ids, const int32_t* num_tokens_post_pad,
                               int64_t sorted_len, int num_experts, int block_size, int pad_value,
                               int granule, int rows_per_block, void* stream);

/*
 * No counterpart in the reference: riders for the grouped GEMM.  moe_align_block_size fills an
 * expert's blocks greedily (fused_moe.py:151-204), so an expert's last block is often nearly
 * empty, and a workgroup of the GEMM that works on such a block still pulls the expert's whole
 * weight tile through its compute unit.  sarathi_moe_plan_riders looks at moe_align_block_size's
 * outputs for block_m = 256 and writes one int32 per slot block into `riders`: the first slot of
 * a 32-slot tile of the same expert's last block that this block's workgroups multiply as well,
 * -1 for none, -2 for a last block all of whose tiles ride with others (the GEMM skips it).  A
 * last block rides when it holds at most as many 32-slot tiles as the expert has full blocks.
 * sarathi_moe_grouped_gemm_riders is sarathi_moe_grouped_gemm with that table: row-major weights,
 * block_m = 256, bfloat16 / float16 (anything else: SARATHI_ERR_UNSUPPORTED); same results bit
 * for bit (a slot's dot products do not depend on which workgroup forms them).  A launch so
 * small that the plain kernel takes 128-wide column blocks to fill the chip runs that kernel and
 * ignores the table.  The sorted ids must be in moe_align_block_size's greedy order (not rewritten
 * by sarathi_moe_balance_blocks).
 */
int sarathi_moe_plan_riders(const int32_t* sorted_token_ids, const int32_t* expert_ids,
                            const int32_t* num_tokens_post_padded, int64_t num_valid_tokens,
                            int64_t sorted_len, int block_m, int32_t* riders, int64_t riders_len,
                            void* stream);
int sarathi_moe_grouped_gemm_riders(const void* a, const void* b, void* c, const float* topk_weights,
                                    const int32_t* sorted_token_ids, const int32_t* expert_ids,
                                    const int32_t* num_tokens_post_padded, int64_t num_valid_tokens,
                                    int64_t sorted_len, int64_t n, int64_t k, int64_t a_row_stride,
                                    int64_t b_expert_stride, int64_t c_row_stride, int block_m,
                                    int top_k, int epilogue, int b_layout, int dtype,
                                    const int32_t* riders, void* stream);

/*
 * No counterpart in the reference: sarathi_moe_plan_riders and sarathi_moe_balance_blocks in one
 * launch, the choice made per expert (block_m = 256 only, SARATHI_ERR_UNSUPPORTED otherwise).  An
 * expert whose last block holds at most as many 32-slot tiles as the expert has full blocks keeps
 * moe_align_block_size's layout in `sorted_out` and gets riders; every other expert's slots are
 * spread evenly over the two 128-slot halves of each of its blocks (what
 * sarathi_moe_balance_blocks does with granule 32 and rows_per_block 2: a block costs the GEMM as
 * much as its fuller half) and its entries of `riders` are -1.  `sorted_out` (same length as
 * `sorted_in`, not the same memory) and `riders` (one int32 per slot block, at least
 * ceil(sorted_len / block_m)) then go to sarathi_moe_grouped_gemm_riders together with the
 * unchanged expert_ids and num_tokens_post_padded.  `pad_value` is the padding id
 * (num_valid_tokens); `sorted_in` must carry it in every unused slot of the live blocks
 * (sarathi_moe_align_block_size with fill_pad = 1).  Same GEMM results bit for bit.
 */
int sarathi_moe_plan_blocks(const int32_t* sorted_in, int32_t* sorted_out, const int32_t* expert_ids,
                            const int32_t* num_tokens_post_padded, int64_t sorted_len,
                            int num_experts, int block_m, int pad_value, int32_t* riders,
                            int64_t riders_len, void* stream);

/*
 * No counterpart in the reference: how many equal ranges of a slot block the waves of the
 * sarathi_moe_grouped_gemm kernel for (block_m, b_layout) split between them (1 or 2; each range
 * is swept by its own waves, 32 slots at a time, and ranges without a valid slot in a tile are
 * skipped per wave), or a negative SARATHI_ERR_* for an unsupported block_m / unknown layout.
 */
int sarathi_moe_gemm_slot_rows(int block_m, int b_layout);

/*
 * Measurement aid with no counterpart in the reference: a device-to-device copy of `bytes` bytes
 * (a multiple of 16, both pointers 16-byte aligned, below 4 GiB) launched the way this library's
 * streaming ops are -- one-wave workgroups that walk memory linearly, `kib_per_wave` 16-byte loads
 * per lane issued before the first of as many stores (1, 2, 4, 8, 12, 16, 18, 24, 36 or 48), the
 * same cache policies.  bench.py times it at each op's byte count and reports the fastest shape as
 * that launch size's ceiling.
 */
int sarathi_stream_copy(void* dst, const void* src, int64_t bytes, int kib_per_wave, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* SARATHI_OPS_H_ */
