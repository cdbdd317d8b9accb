// PyTorch-ROCm front end of the op library: a pybind11 module whose functions
// have the names and positional signatures of the reference's four extension
// modules (csrc/layernorm.cpp:9, csrc/activation.cpp:15-27, csrc/pos_encoding.cpp:11,
// csrc/moe.cpp:19-27), plus the entries the reference does not have: fused_add_rms_norm, the
// fused MoE routing variants, grouped_topk, the grouped expert GEMM and the paged KV-cache ops.
//
// This layer only (a) checks what the reference leaves unchecked: device, dtype,
// rank, inner contiguity; (b) makes the tensors' device current and looks up
// torch's current HIP stream for it; (c) forwards raw pointers, sizes and
// strides to the C ABI of include/sarathi_ops.h and turns a non-zero status
// into a RuntimeError.  It never copies or synchronises, and allocates only the scratch
// tensor that moe_align_block_size uses for inputs above 32 K ids and, once per (device, stream),
// the four-byte completion counter of fused_topk_align.
#include <c10/hip/HIPStream.h>
#include <hip/hip_runtime_api.h>
#include <torch/extension.h>

#include <map>
#include <mutex>
#include <utility>

#include "../../include/sarathi_ops.h"

namespace {

int dtype_code(const torch::Tensor& t, const char* op) {
  switch (t.scalar_type()) {
    case at::ScalarType::Float: return SARATHI_DTYPE_F32;
    case at::ScalarType::Half: return SARATHI_DTYPE_F16;
    case at::ScalarType::BFloat16: return SARATHI_DTYPE_BF16;
    default: TORCH_CHECK(false, op, ": expected a float32, float16 or bfloat16 tensor, got ",
                         t.scalar_type());
  }
  return -1;
}

int id_dtype_code(const torch::Tensor& t) {
  switch (t.scalar_type()) {
    case at::ScalarType::Byte: return SARATHI_IDTYPE_U8;
    case at::ScalarType::Char: return SARATHI_IDTYPE_I8;
    case at::ScalarType::Short: return SARATHI_IDTYPE_I16;
    case at::ScalarType::Int: return SARATHI_IDTYPE_I32;
    case at::ScalarType::Long: return SARATHI_IDTYPE_I64;
    default: TORCH_CHECK(false, "moe_align_block_size: topk_ids must be an integer tensor, got ",
                         t.scalar_type());
  }
  return -1;
}

void check_gpu(const torch::Tensor& t, const torch::Tensor& like, const char* op,
               const char* name) {
  TORCH_CHECK(t.is_cuda(), op, ": ", name, " must live on the GPU");
  TORCH_CHECK(t.device() == like.device(), op, ": ", name, " is on ", t.device(),
              " but the first tensor is on ", like.device());
}

// Makes `dev` the current HIP device for the scope and yields torch's current
// stream on it.
struct LaunchScope {
  int prev = -1;
  int dev;
  void* stream;
  explicit LaunchScope(const torch::Tensor& t) : dev(t.device().index()) {
    TORCH_CHECK(hipGetDevice(&prev) == hipSuccess, "hipGetDevice failed");
    if (prev != dev) TORCH_CHECK(hipSetDevice(dev) == hipSuccess, "hipSetDevice failed");
    stream = c10::hip::getCurrentHIPStream(static_cast<c10::DeviceIndex>(dev)).stream();
  }
  ~LaunchScope() {
    if (prev >= 0 && prev != dev) (void)hipSetDevice(prev);
  }
};

void raise_on(int status, const char* op) {
  TORCH_CHECK(status == SARATHI_OK, op, " failed: ", sarathi_ops_strerror(status), " (code ",
              status, ")");
}

// ---- layernorm_ops -----------------------------------------------------------

void rms_norm(torch::Tensor& out, torch::Tensor& input, torch::Tensor& weight, double epsilon) {
  const char* op = "rms_norm";
  check_gpu(input, input, op, "input");
  check_gpu(out, input, op, "out");
  check_gpu(weight, input, op, "weight");
  TORCH_CHECK(input.dim() == 2 && out.dim() == 2, op, ": input and out must be [num_tokens, hidden]");
  TORCH_CHECK(out.sizes() == input.sizes(), op, ": out and input shapes differ");
  TORCH_CHECK(out.scalar_type() == input.scalar_type() &&
                  weight.scalar_type() == input.scalar_type(),
              op, ": out, input and weight must share a dtype");
  TORCH_CHECK(weight.dim() == 1 && weight.size(0) == input.size(1) && weight.is_contiguous(), op,
              ": weight must be a contiguous [hidden] vector");
  TORCH_CHECK(input.stride(1) == 1 && out.stride(1) == 1, op, ": rows must be contiguous");
  LaunchScope scope(input);
  raise_on(sarathi_rms_norm(out.data_ptr(), input.data_ptr(), weight.data_ptr(), (float)epsilon,
                            input.size(0), input.size(1), input.stride(0), out.stride(0),
                            dtype_code(input, op), scope.stream),
           op);
}

void fused_add_rms_norm(torch::Tensor& input, torch::Tensor& residual, torch::Tensor& weight,
                        double epsilon) {
  const char* op = "fused_add_rms_norm";
  check_gpu(input, input, op, "input");
  check_gpu(residual, input, op, "residual");
  check_gpu(weight, input, op, "weight");
  TORCH_CHECK(input.dim() == 2, op, ": input must be [num_tokens, hidden]");
  TORCH_CHECK(residual.sizes() == input.sizes(), op, ": residual and input shapes differ");
  TORCH_CHECK(residual.scalar_type() == input.scalar_type() &&
                  weight.scalar_type() == input.scalar_type(),
              op, ": input, residual and weight must share a dtype");
  TORCH_CHECK(weight.dim() == 1 && weight.size(0) == input.size(1) && weight.is_contiguous(), op,
              ": weight must be a contiguous [hidden] vector");
  TORCH_CHECK(input.stride(1) == 1 && residual.stride(1) == 1, op, ": rows must be contiguous");
  TORCH_CHECK(input.numel() == 0 || input.data_ptr() != residual.data_ptr(), op,
              ": input and residual must not alias");
  LaunchScope scope(input);
  raise_on(sarathi_fused_add_rms_norm(input.data_ptr(), residual.data_ptr(), weight.data_ptr(),
                                      (float)epsilon, input.size(0), input.size(1),
                                      input.stride(0), residual.stride(0), dtype_code(input, op),
                                      scope.stream),
           op);
}

// ---- activation_ops ----------------------------------------------------------

void silu_and_mul(torch::Tensor& out, torch::Tensor& input) {
  const char* op = "silu_and_mul";
  check_gpu(input, input, op, "input");
  check_gpu(out, input, op, "out");
  TORCH_CHECK(input.dim() == 2 && out.dim() == 2, op, ": input [num_tokens, 2*d], out [num_tokens, d]");
  TORCH_CHECK(input.size(1) % 2 == 0 && out.size(1) * 2 == input.size(1) &&
                  out.size(0) == input.size(0),
              op, ": out must be [num_tokens, input.size(1) / 2]");
  TORCH_CHECK(out.scalar_type() == input.scalar_type(), op, ": out and input must share a dtype");
  TORCH_CHECK(input.stride(1) == 1 && out.stride(1) == 1, op, ": rows must be contiguous");
  LaunchScope scope(input);
  raise_on(sarathi_silu_and_mul(out.data_ptr(), input.data_ptr(), input.size(0), out.size(1),
                                input.stride(0), out.stride(0), dtype_code(input, op),
                                scope.stream),
           op);
}

template <bool FAST>
void gelu_impl(torch::Tensor& out, torch::Tensor& input) {
  const char* op = FAST ? "gelu_fast" : "gelu_new";
  check_gpu(input, input, op, "input");
  check_gpu(out, input, op, "out");
  TORCH_CHECK(input.dim() == 2 && out.sizes() == input.sizes(), op,
              ": input and out must both be [num_tokens, d]");
  TORCH_CHECK(out.scalar_type() == input.scalar_type(), op, ": out and input must share a dtype");
  TORCH_CHECK(input.is_contiguous() && out.is_contiguous(), op, ": tensors must be contiguous");
  LaunchScope scope(input);
  auto fn = FAST ? sarathi_gelu_fast : sarathi_gelu_new;
  raise_on(fn(out.data_ptr(), input.data_ptr(), input.size(0), input.size(1),
              dtype_code(input, op), scope.stream),
           op);
}
void gelu_new(torch::Tensor& out, torch::Tensor& input) { gelu_impl<false>(out, input); }
void gelu_fast(torch::Tensor& out, torch::Tensor& input) { gelu_impl<true>(out, input); }

// ---- pos_encoding_ops --------------------------------------------------------

void rotary_embedding(torch::Tensor& positions, torch::Tensor& query, torch::Tensor& key,
                      int64_t head_size, torch::Tensor& cos_sin_cache, bool is_neox) {
  const char* op = "rotary_embedding";
  check_gpu(query, query, op, "query");
  check_gpu(key, query, op, "key");
  check_gpu(positions, query, op, "positions");
  check_gpu(cos_sin_cache, query, op, "cos_sin_cache");
  TORCH_CHECK(positions.scalar_type() == at::ScalarType::Long && positions.dim() == 1 &&
                  positions.is_contiguous(),
              op, ": positions must be a contiguous int64 [num_tokens] tensor");
  TORCH_CHECK(query.dim() == 2 && key.dim() == 2, op, ": query and key must be 2-D");
  TORCH_CHECK(query.size(0) == positions.size(0) && key.size(0) == positions.size(0), op,
              ": query, key and positions disagree on num_tokens");
  TORCH_CHECK(key.scalar_type() == query.scalar_type() &&
                  cos_sin_cache.scalar_type() == query.scalar_type(),
              op, ": query, key and cos_sin_cache must share a dtype");
  TORCH_CHECK(head_size > 0 && query.size(1) % head_size == 0 && key.size(1) % head_size == 0, op,
              ": row widths must be multiples of head_size");
  TORCH_CHECK(cos_sin_cache.dim() == 2 && cos_sin_cache.is_contiguous(), op,
              ": cos_sin_cache must be a contiguous [max_position, rot_dim] tensor");
  TORCH_CHECK(query.stride(1) == 1 && key.stride(1) == 1, op, ": rows must be contiguous");
  const int64_t rot_dim = cos_sin_cache.size(1);
  TORCH_CHECK(rot_dim % 2 == 0 && rot_dim <= head_size, op, ": rot_dim must be even and <= head_size");
  LaunchScope scope(query);
  raise_on(sarathi_rotary_embedding(positions.data_ptr<int64_t>(), query.data_ptr(), key.data_ptr(),
                                    cos_sin_cache.data_ptr(), query.size(0),
                                    (int)(query.size(1) / head_size),
                                    (int)(key.size(1) / head_size), (int)head_size, (int)rot_dim,
                                    query.stride(0), key.stride(0), is_neox ? 1 : 0,
                                    dtype_code(query, op), scope.stream),
           op);
}

// ---- kv_cache_ops --------------------------------------------------------------

void check_i32(const torch::Tensor& t, const torch::Tensor& like, const char* op,
               const char* name) {
  check_gpu(t, like, op, name);
  TORCH_CHECK(t.scalar_type() == at::ScalarType::Int && t.dim() == 1 && t.is_contiguous(), op,
              ": ", name, " must be a contiguous int32 vector");
}

// k_cache / v_cache: [num_pages, page_size, num_kv_heads, head_size] views with the same strides
struct PagedGeom {
  int64_t page_size, heads, head_size, page_stride, entry_stride;
};
PagedGeom paged_geom(const torch::Tensor& k_cache, const torch::Tensor& v_cache, const char* op) {
  TORCH_CHECK(k_cache.dim() == 4 && v_cache.dim() == 4, op,
              ": k_cache and v_cache must be [num_pages, page_size, num_kv_heads, head_size]");
  TORCH_CHECK(k_cache.sizes() == v_cache.sizes() && k_cache.strides() == v_cache.strides() &&
                  k_cache.scalar_type() == v_cache.scalar_type(),
              op, ": k_cache and v_cache must agree in shape, strides and dtype");
  TORCH_CHECK(k_cache.stride(3) == 1 && k_cache.stride(2) == k_cache.size(3), op,
              ": the [num_kv_heads, head_size] part of a cache entry must be contiguous");
  return {k_cache.size(1), k_cache.size(2), k_cache.size(3), k_cache.stride(0), k_cache.stride(1)};
}

// rows of a [n, heads*head_size] or [n, heads, head_size] tensor: returns the row stride
int64_t token_rows(const torch::Tensor& t, int64_t width, int64_t head_size, const char* op,
                   const char* name) {
  TORCH_CHECK(t.dim() == 2 || t.dim() == 3, op, ": ", name, " must be 2-D or 3-D");
  if (t.dim() == 2) {
    TORCH_CHECK(t.size(1) == width && t.stride(1) == 1, op, ": ", name, " rows must be ", width,
                " contiguous elements");
  } else {
    TORCH_CHECK(t.size(1) * t.size(2) == width && t.size(2) == head_size && t.stride(2) == 1 &&
                    t.stride(1) == head_size,
                op, ": ", name, " must be [n, heads, ", head_size, "] with contiguous rows");
  }
  return t.stride(0);
}

void get_seq_lens(torch::Tensor& kv_indptr, torch::Tensor& kv_last_page_len,
                  torch::Tensor& seq_lens, int64_t page_size) {
  const char* op = "get_seq_lens";
  check_i32(kv_indptr, kv_indptr, op, "kv_indptr");
  check_i32(kv_last_page_len, kv_indptr, op, "kv_last_page_len");
  check_i32(seq_lens, kv_indptr, op, "seq_lens");
  const int64_t n = kv_last_page_len.numel();
  TORCH_CHECK(kv_indptr.numel() == n + 1 && seq_lens.numel() == n && page_size > 0, op,
              ": expected kv_indptr [n+1], kv_last_page_len [n], seq_lens [n]");
  LaunchScope scope(kv_indptr);
  raise_on(sarathi_get_seq_lens(kv_indptr.data_ptr<int32_t>(), kv_last_page_len.data_ptr<int32_t>(),
                                seq_lens.data_ptr<int32_t>(), n, (int)page_size, scope.stream),
           op);
}

void get_batch_indices_positions(torch::Tensor& append_indptr, torch::Tensor& seq_lens,
                                 torch::Tensor& batch_indices, torch::Tensor& positions) {
  const char* op = "get_batch_indices_positions";
  check_i32(append_indptr, append_indptr, op, "append_indptr");
  check_i32(seq_lens, append_indptr, op, "seq_lens");
  check_i32(batch_indices, append_indptr, op, "batch_indices");
  check_i32(positions, append_indptr, op, "positions");
  const int64_t n = seq_lens.numel();
  TORCH_CHECK(append_indptr.numel() == n + 1 && batch_indices.numel() == positions.numel(), op,
              ": expected append_indptr [n+1], seq_lens [n], batch_indices and positions [nnz]");
  LaunchScope scope(append_indptr);
  raise_on(sarathi_get_batch_indices_positions(
               append_indptr.data_ptr<int32_t>(), seq_lens.data_ptr<int32_t>(),
               batch_indices.data_ptr<int32_t>(), positions.data_ptr<int32_t>(), n,
               positions.numel(), scope.stream),
           op);
}

void get_kv_slot_mapping(torch::Tensor& batch_indices, torch::Tensor& positions,
                         torch::Tensor& kv_indices, torch::Tensor& kv_indptr,
                         torch::Tensor& slot_mapping, int64_t page_size) {
  const char* op = "get_kv_slot_mapping";
  check_i32(batch_indices, batch_indices, op, "batch_indices");
  check_i32(positions, batch_indices, op, "positions");
  check_i32(kv_indices, batch_indices, op, "kv_indices");
  check_i32(kv_indptr, batch_indices, op, "kv_indptr");
  check_i32(slot_mapping, batch_indices, op, "slot_mapping");
  const int64_t nnz = batch_indices.numel();
  TORCH_CHECK(positions.numel() == nnz && slot_mapping.numel() == nnz && page_size > 0, op,
              ": batch_indices, positions and slot_mapping must hold nnz entries");
  LaunchScope scope(batch_indices);
  raise_on(sarathi_get_kv_slot_mapping(batch_indices.data_ptr<int32_t>(),
                                       positions.data_ptr<int32_t>(),
                                       kv_indices.data_ptr<int32_t>(),
                                       kv_indptr.data_ptr<int32_t>(),
                                       slot_mapping.data_ptr<int32_t>(), nnz, (int)page_size,
                                       scope.stream),
           op);
}

void append_paged_kv_cache(torch::Tensor& append_key, torch::Tensor& append_value,
                           torch::Tensor& batch_indices, torch::Tensor& positions,
                           torch::Tensor& k_cache, torch::Tensor& v_cache,
                           torch::Tensor& kv_indices, torch::Tensor& kv_indptr,
                           c10::optional<torch::Tensor> slot_mapping) {
  const char* op = "append_paged_kv_cache";
  check_gpu(append_key, append_key, op, "append_key");
  check_gpu(append_value, append_key, op, "append_value");
  check_gpu(k_cache, append_key, op, "k_cache");
  check_gpu(v_cache, append_key, op, "v_cache");
  check_i32(batch_indices, append_key, op, "batch_indices");
  check_i32(positions, append_key, op, "positions");
  check_i32(kv_indices, append_key, op, "kv_indices");
  check_i32(kv_indptr, append_key, op, "kv_indptr");
  const PagedGeom g = paged_geom(k_cache, v_cache, op);
  TORCH_CHECK(append_key.scalar_type() == k_cache.scalar_type() &&
                  append_value.scalar_type() == k_cache.scalar_type(),
              op, ": keys, values and the cache must share a dtype");
  const int64_t width = g.heads * g.head_size;
  const int64_t ks = token_rows(append_key, width, g.head_size, op, "append_key");
  const int64_t vs = token_rows(append_value, width, g.head_size, op, "append_value");
  const int64_t nnz = append_key.size(0);
  TORCH_CHECK(append_value.size(0) == nnz && batch_indices.numel() == nnz &&
                  positions.numel() == nnz,
              op, ": append_key, append_value, batch_indices and positions disagree on nnz");
  const int32_t* slots = nullptr;
  if (slot_mapping.has_value()) {
    check_i32(*slot_mapping, append_key, op, "slot_mapping");
    TORCH_CHECK(slot_mapping->numel() == nnz, op, ": slot_mapping must hold nnz entries");
    slots = slot_mapping->data_ptr<int32_t>();
  }
  LaunchScope scope(append_key);
  raise_on(sarathi_append_paged_kv_cache(
               append_key.data_ptr(), append_value.data_ptr(), batch_indices.data_ptr<int32_t>(),
               positions.data_ptr<int32_t>(), k_cache.data_ptr(), v_cache.data_ptr(),
               kv_indices.data_ptr<int32_t>(), kv_indptr.data_ptr<int32_t>(), slots, nnz,
               (int)g.heads, (int)g.head_size, (int)g.page_size, nnz > 1 ? ks : width, nnz > 1 ? vs : width,
               g.page_stride, g.entry_stride, dtype_code(append_key, op), scope.stream),
           op);
}

void rotary_embedding_append_paged_kv(torch::Tensor& positions, torch::Tensor& query,
                                      torch::Tensor& key, torch::Tensor& value, int64_t head_size,
                                      torch::Tensor& cos_sin_cache, bool is_neox,
                                      torch::Tensor& batch_indices,
                                      torch::Tensor& append_positions, torch::Tensor& k_cache,
                                      torch::Tensor& v_cache, torch::Tensor& kv_indices,
                                      torch::Tensor& kv_indptr, int64_t num_append_tokens,
                                      bool write_key,
                                      c10::optional<torch::Tensor> slot_mapping) {
  const char* op = "rotary_embedding_append_paged_kv";
  check_gpu(query, query, op, "query");
  check_gpu(key, query, op, "key");
  check_gpu(value, query, op, "value");
  check_gpu(positions, query, op, "positions");
  check_gpu(cos_sin_cache, query, op, "cos_sin_cache");
  check_gpu(k_cache, query, op, "k_cache");
  check_gpu(v_cache, query, op, "v_cache");
  check_i32(batch_indices, query, op, "batch_indices");
  check_i32(append_positions, query, op, "append_positions");
  check_i32(kv_indices, query, op, "kv_indices");
  check_i32(kv_indptr, query, op, "kv_indptr");
  TORCH_CHECK(positions.scalar_type() == at::ScalarType::Long && positions.dim() == 1 &&
                  positions.is_contiguous(),
              op, ": positions must be a contiguous int64 [num_tokens] tensor");
  TORCH_CHECK(query.dim() == 2 && key.dim() == 2 && value.dim() == 2, op,
              ": query, key and value must be 2-D");
  const int64_t T = positions.size(0);
  TORCH_CHECK(query.size(0) == T && key.size(0) == T && value.size(0) == T, op,
              ": query, key, value and positions disagree on num_tokens");
  const PagedGeom g = paged_geom(k_cache, v_cache, op);
  TORCH_CHECK(key.scalar_type() == query.scalar_type() &&
                  value.scalar_type() == query.scalar_type() &&
                  cos_sin_cache.scalar_type() == query.scalar_type() &&
                  k_cache.scalar_type() == query.scalar_type(),
              op, ": query, key, value, cos_sin_cache and the cache must share a dtype");
  TORCH_CHECK(head_size == g.head_size && query.size(1) % head_size == 0 &&
                  key.size(1) == g.heads * head_size && value.size(1) == key.size(1),
              op, ": key / value rows must be num_kv_heads * head_size of the cache");
  TORCH_CHECK(cos_sin_cache.dim() == 2 && cos_sin_cache.is_contiguous(), op,
              ": cos_sin_cache must be a contiguous [max_position, rot_dim] tensor");
  TORCH_CHECK(query.stride(1) == 1 && key.stride(1) == 1 && value.stride(1) == 1, op,
              ": rows must be contiguous");
  const int64_t rot_dim = cos_sin_cache.size(1);
  TORCH_CHECK(rot_dim % 2 == 0 && rot_dim <= head_size, op,
              ": rot_dim must be even and <= head_size");
  TORCH_CHECK(num_append_tokens >= 0 && num_append_tokens <= T &&
                  batch_indices.numel() >= num_append_tokens &&
                  append_positions.numel() >= num_append_tokens,
              op, ": num_append_tokens must be within num_tokens and the index vectors");
  const int32_t* slots = nullptr;
  if (slot_mapping.has_value()) {
    check_i32(*slot_mapping, query, op, "slot_mapping");
    TORCH_CHECK(slot_mapping->numel() >= num_append_tokens, op,
                ": slot_mapping must hold num_append_tokens entries");
    slots = slot_mapping->data_ptr<int32_t>();
  }
  LaunchScope scope(query);
  raise_on(sarathi_rotary_embedding_append_paged_kv(
               positions.data_ptr<int64_t>(), query.data_ptr(), key.data_ptr(), value.data_ptr(),
               cos_sin_cache.data_ptr(), batch_indices.data_ptr<int32_t>(),
               append_positions.data_ptr<int32_t>(), k_cache.data_ptr(), v_cache.data_ptr(),
               kv_indices.data_ptr<int32_t>(), kv_indptr.data_ptr<int32_t>(), slots, T,
               num_append_tokens, (int)(query.size(1) / head_size), (int)g.heads, (int)head_size, (int)rot_dim,
               T > 1 ? query.stride(0) : query.size(1), T > 1 ? key.stride(0) : key.size(1),
               T > 1 ? value.stride(0) : value.size(1), (int)g.page_size, g.page_stride,
               g.entry_stride, is_neox ? 1 : 0, write_key ? 1 : 0, dtype_code(query, op),
               scope.stream),
           op);
}

// ---- moe_ops -----------------------------------------------------------------

void topk_softmax_impl(torch::Tensor& topk_weights, torch::Tensor& topk_indices,
                       torch::Tensor& token_expert_indices, torch::Tensor& gating_output,
                       bool renormalize, const char* op) {
  check_gpu(gating_output, gating_output, op, "gating_output");
  check_gpu(topk_weights, gating_output, op, "topk_weights");
  check_gpu(topk_indices, gating_output, op, "topk_indices");
  check_gpu(token_expert_indices, gating_output, op, "token_expert_indices");
  TORCH_CHECK(gating_output.scalar_type() == at::ScalarType::Float &&
                  topk_weights.scalar_type() == at::ScalarType::Float,
              op, ": gating_output and topk_weights must be float32");
  TORCH_CHECK(topk_indices.scalar_type() == at::ScalarType::Int &&
                  token_expert_indices.scalar_type() == at::ScalarType::Int,
              op, ": topk_indices and token_expert_indices must be int32");
  TORCH_CHECK(gating_output.dim() >= 1 && gating_output.is_contiguous() &&
                  topk_weights.is_contiguous() && topk_indices.is_contiguous() &&
                  token_expert_indices.is_contiguous(),
              op, ": tensors must be contiguous");
  const int64_t num_experts = gating_output.size(-1);
  TORCH_CHECK(num_experts > 0, op, ": gating_output has no experts");
  const int64_t num_tokens = gating_output.numel() / num_experts;
  const int64_t topk = topk_weights.size(-1);
  TORCH_CHECK(topk_weights.numel() == num_tokens * topk && topk_indices.numel() == num_tokens * topk &&
                  token_expert_indices.numel() == num_tokens * topk,
              op, ": outputs must be [num_tokens, topk]");
  LaunchScope scope(gating_output);
  raise_on(sarathi_topk_softmax(topk_weights.data_ptr<float>(), topk_indices.data_ptr<int32_t>(),
                                token_expert_indices.data_ptr<int32_t>(),
                                gating_output.data_ptr<float>(), num_tokens, (int)num_experts,
                                (int)topk, renormalize ? 1 : 0, scope.stream),
           op);
}

void topk_softmax(torch::Tensor& topk_weights, torch::Tensor& topk_indices,
                  torch::Tensor& token_expert_indices, torch::Tensor& gating_output) {
  topk_softmax_impl(topk_weights, topk_indices, token_expert_indices, gating_output, false,
                    "topk_softmax");
}

void topk_softmax_renorm(torch::Tensor& topk_weights, torch::Tensor& topk_indices,
                         torch::Tensor& token_expert_indices, torch::Tensor& gating_output) {
  topk_softmax_impl(topk_weights, topk_indices, token_expert_indices, gating_output, true,
                    "topk_softmax_renorm");
}

void moe_align_impl(torch::Tensor& topk_ids, int64_t num_experts, int64_t block_size,
                    torch::Tensor& sorted_token_ids, torch::Tensor& experts_ids,
                    torch::Tensor& num_tokens_post_pad, bool fill_pad, const char* op) {
  check_gpu(topk_ids, topk_ids, op, "topk_ids");
  check_gpu(sorted_token_ids, topk_ids, op, "sorted_token_ids");
  check_gpu(experts_ids, topk_ids, op, "experts_ids");
  check_gpu(num_tokens_post_pad, topk_ids, op, "num_tokens_post_pad");
  TORCH_CHECK(sorted_token_ids.scalar_type() == at::ScalarType::Int &&
                  experts_ids.scalar_type() == at::ScalarType::Int &&
                  num_tokens_post_pad.scalar_type() == at::ScalarType::Int,
              op, ": sorted_token_ids, experts_ids and num_tokens_post_pad must be int32");
  TORCH_CHECK(topk_ids.is_contiguous() && sorted_token_ids.is_contiguous() &&
                  experts_ids.is_contiguous() && num_tokens_post_pad.numel() >= 1,
              op, ": tensors must be contiguous");
  TORCH_CHECK(num_experts > 0 && num_experts <= INT32_MAX && block_size > 0 &&
                  block_size <= INT32_MAX,
              op, ": num_experts and block_size must be positive");
  LaunchScope scope(topk_ids);
  // Large inputs get a scratch tensor from torch's caching allocator (stream-ordered, so it may
  // be released as soon as the launches are queued), the way the reference's topk_softmax
  // obtains its workspace (csrc/moe_topk_softmax_kernels.cu:486-492).
  const int64_t ws_bytes = sarathi_moe_align_workspace_bytes(topk_ids.numel(), (int)num_experts);
  torch::Tensor workspace;
  if (ws_bytes > 0)
    workspace = torch::empty({ws_bytes / 4}, sorted_token_ids.options());
  raise_on(sarathi_moe_align_block_size(
               topk_ids.data_ptr(), id_dtype_code(topk_ids), topk_ids.numel(), (int)num_experts,
               (int)block_size, sorted_token_ids.data_ptr<int32_t>(), sorted_token_ids.numel(),
               experts_ids.data_ptr<int32_t>(), experts_ids.numel(),
               num_tokens_post_pad.data_ptr<int32_t>(), fill_pad ? 1 : 0,
               ws_bytes > 0 ? workspace.data_ptr() : nullptr, ws_bytes, scope.stream),
           op);
}

void moe_align_block_size(torch::Tensor topk_ids, int64_t num_experts, int64_t block_size,
                          torch::Tensor sorted_token_ids, torch::Tensor experts_ids,
                          torch::Tensor num_tokens_post_pad) {
  moe_align_impl(topk_ids, num_experts, block_size, sorted_token_ids, experts_ids,
                 num_tokens_post_pad, false, "moe_align_block_size");
}

void moe_align_block_size_filled(torch::Tensor topk_ids, int64_t num_experts, int64_t block_size,
                                 torch::Tensor sorted_token_ids, torch::Tensor experts_ids,
                                 torch::Tensor num_tokens_post_pad) {
  moe_align_impl(topk_ids, num_experts, block_size, sorted_token_ids, experts_ids,
                 num_tokens_post_pad, true, "moe_align_block_size_filled");
}

void grouped_topk(torch::Tensor& topk_weights, torch::Tensor& topk_indices,
                  torch::Tensor& gating_output, int64_t num_expert_group, int64_t topk_group,
                  bool renormalize) {
  const char* op = "grouped_topk";
  check_gpu(gating_output, gating_output, op, "gating_output");
  check_gpu(topk_weights, gating_output, op, "topk_weights");
  check_gpu(topk_indices, gating_output, op, "topk_indices");
  TORCH_CHECK(gating_output.scalar_type() == at::ScalarType::Float &&
                  topk_weights.scalar_type() == at::ScalarType::Float &&
                  topk_indices.scalar_type() == at::ScalarType::Int,
              op, ": gating_output / topk_weights must be float32, topk_indices int32");
  TORCH_CHECK(gating_output.dim() == 2 && gating_output.is_contiguous() &&
                  topk_weights.dim() == 2 && topk_weights.is_contiguous() &&
                  topk_indices.is_contiguous() && topk_weights.size(0) == gating_output.size(0) &&
                  topk_indices.numel() == topk_weights.numel(),
              op, ": expected gating_output [T, E], outputs [T, topk], all contiguous");
  LaunchScope scope(gating_output);
  raise_on(sarathi_grouped_topk(topk_weights.data_ptr<float>(), topk_indices.data_ptr<int32_t>(),
                                gating_output.data_ptr<float>(), gating_output.size(0),
                                (int)gating_output.size(1), (int)topk_weights.size(1),
                                (int)num_expert_group, (int)topk_group, renormalize ? 1 : 0,
                                scope.stream),
           op);
}

// One zeroed uint32 per (device, stream): the completion counter of the fused routing kernel.
// Allocated on first use and kept for the life of the process; the map is deliberately never
// destroyed, so no tensor is released after the runtime has shut down at process exit.
uint32_t* routing_counter(int dev, void* stream) {
  static std::mutex mu;
  static auto* counters = new std::map<std::pair<int, void*>, torch::Tensor>();
  std::lock_guard<std::mutex> lock(mu);
  auto key = std::make_pair(dev, stream);
  auto it = counters->find(key);
  if (it == counters->end()) {
    auto t = torch::zeros({1}, torch::TensorOptions().dtype(torch::kInt32).device(torch::kCUDA, dev));
    it = counters->emplace(key, t).first;
  }
  return reinterpret_cast<uint32_t*>(it->second.data_ptr<int32_t>());
}

// fused_topk + moe_align_block_size of fused_moe.py:346-373 / :151-204 in one launch
void fused_topk_align(torch::Tensor& topk_weights, torch::Tensor& topk_indices,
                      torch::Tensor& token_expert_indices, torch::Tensor& gating_output,
                      bool renormalize, int64_t block_size, torch::Tensor& sorted_token_ids,
                      torch::Tensor& experts_ids, torch::Tensor& num_tokens_post_pad,
                      bool fill_pad) {
  const char* op = "fused_topk_align";
  check_gpu(gating_output, gating_output, op, "gating_output");
  check_gpu(topk_weights, gating_output, op, "topk_weights");
  check_gpu(topk_indices, gating_output, op, "topk_indices");
  check_gpu(token_expert_indices, gating_output, op, "token_expert_indices");
  check_gpu(sorted_token_ids, gating_output, op, "sorted_token_ids");
  check_gpu(experts_ids, gating_output, op, "experts_ids");
  check_gpu(num_tokens_post_pad, gating_output, op, "num_tokens_post_pad");
  TORCH_CHECK(gating_output.scalar_type() == at::ScalarType::Float &&
                  topk_weights.scalar_type() == at::ScalarType::Float,
              op, ": gating_output and topk_weights must be float32");
  TORCH_CHECK(topk_indices.scalar_type() == at::ScalarType::Int &&
                  token_expert_indices.scalar_type() == at::ScalarType::Int &&
                  sorted_token_ids.scalar_type() == at::ScalarType::Int &&
                  experts_ids.scalar_type() == at::ScalarType::Int &&
                  num_tokens_post_pad.scalar_type() == at::ScalarType::Int,
              op, ": index tensors must be int32");
  TORCH_CHECK(gating_output.dim() == 2 && gating_output.is_contiguous() &&
                  topk_weights.is_contiguous() && topk_indices.is_contiguous() &&
                  token_expert_indices.is_contiguous() && sorted_token_ids.is_contiguous() &&
                  experts_ids.is_contiguous() && num_tokens_post_pad.numel() >= 1,
              op, ": tensors must be contiguous");
  const int64_t T = gating_output.size(0), E = gating_output.size(1);
  TORCH_CHECK(topk_weights.dim() == 2 && topk_weights.size(0) == T, op,
              ": topk_weights must be [num_tokens, topk]");
  const int64_t k = topk_weights.size(1);
  TORCH_CHECK(topk_indices.numel() == T * k && token_expert_indices.numel() == T * k, op,
              ": topk outputs must be [num_tokens, topk]");
  LaunchScope scope(gating_output);
  raise_on(sarathi_fused_topk_align(
               topk_weights.data_ptr<float>(), topk_indices.data_ptr<int32_t>(),
               token_expert_indices.data_ptr<int32_t>(), gating_output.data_ptr<float>(), T, (int)E,
               (int)k, renormalize ? 1 : 0, (int)block_size, sorted_token_ids.data_ptr<int32_t>(),
               sorted_token_ids.numel(), experts_ids.data_ptr<int32_t>(), experts_ids.numel(),
               num_tokens_post_pad.data_ptr<int32_t>(), fill_pad ? 1 : 0,
               routing_counter(scope.dev, scope.stream), scope.stream),
           op);
}

// torch.sum(input, dim=1, out=out) of fused_moe.py:539-543: input [tokens, top_k, hidden]
void moe_sum(torch::Tensor& input, torch::Tensor& out) {
  const char* op = "moe_sum";
  check_gpu(input, input, op, "input");
  check_gpu(out, input, op, "out");
  TORCH_CHECK(input.dim() == 3 && out.dim() == 2, op, ": input [tokens, top_k, hidden], out [tokens, hidden]");
  TORCH_CHECK(out.size(0) == input.size(0) && out.size(1) == input.size(2), op,
              ": out must be [input.size(0), input.size(2)]");
  TORCH_CHECK(out.scalar_type() == input.scalar_type(), op, ": out and input must share a dtype");
  TORCH_CHECK(input.size(1) >= 1, op, ": top_k must be at least 1");
  TORCH_CHECK((input.stride(2) == 1 || input.size(2) <= 1) && (out.stride(1) == 1 || out.size(1) <= 1),
              op, ": rows must be contiguous");
  LaunchScope scope(input);
  raise_on(sarathi_moe_sum(out.data_ptr(), input.data_ptr(), input.size(0), input.size(1),
                           input.size(2), input.stride(0), input.stride(1), out.stride(0),
                           dtype_code(input, op), scope.stream),
           op);
}

// A [tokens, K], B [E, N, K], C [tokens, topk, N] (or any tensor whose rows of N elements are
// addressed by slot = token * topk + j), as invoke_fused_moe_kernel passes them.  With
// b_packed, B is the re-tiled weight tensor [E, ceil(N/32), K/16, 2, 32, 8] and `n` its logical
// row count.
void moe_grouped_gemm(torch::Tensor& a, torch::Tensor& b, torch::Tensor& c,
                      torch::Tensor& topk_weights, torch::Tensor& sorted_token_ids,
                      torch::Tensor& expert_ids, torch::Tensor& num_tokens_post_padded,
                      int64_t num_valid_tokens, int64_t block_m, int64_t top_k,
                      bool mul_routed_weight, bool b_packed, int64_t n, bool silu_and_mul,
                      const c10::optional<torch::Tensor>& riders) {
  const char* op = "moe_grouped_gemm";
  check_gpu(a, a, op, "A");
  check_gpu(b, a, op, "B");
  check_gpu(c, a, op, "C");
  check_gpu(topk_weights, a, op, "topk_weights");
  check_gpu(sorted_token_ids, a, op, "sorted_token_ids");
  check_gpu(expert_ids, a, op, "expert_ids");
  check_gpu(num_tokens_post_padded, a, op, "num_tokens_post_padded");
  TORCH_CHECK(a.dim() == 2 && a.stride(1) == 1, op, ": A must be [tokens, K] with contiguous rows");
  const int64_t k = a.size(1);
  // the kernel gathers row slot / top_k of A for every slot below num_valid_tokens
  TORCH_CHECK(top_k > 0 && num_valid_tokens >= 0 && a.size(0) * top_k >= num_valid_tokens, op,
              ": A has ", a.size(0), " rows but num_valid_tokens = ", num_valid_tokens,
              " with top_k = ", top_k, " needs ceil(num_valid_tokens / top_k)");
  int64_t expert_stride;
  if (b_packed) {
    TORCH_CHECK(b.dim() == 6 && b.is_contiguous() && b.size(3) == 2 && b.size(4) == 32 &&
                    b.size(5) == 8 && b.size(2) * 16 == k && n > 0 && b.size(1) == (n + 31) / 32,
                op, ": packed B must be contiguous [E, ceil(N/32), K/16, 2, 32, 8]");
    expert_stride = b.stride(0);
  } else {
    TORCH_CHECK(b.dim() == 3 && b.size(2) == k && b.stride(2) == 1 && b.stride(1) == k, op,
                ": B must be [E, N, K] with contiguous matrices");
    n = b.size(1);
    expert_stride = b.stride(0);
  }
  TORCH_CHECK(a.scalar_type() == b.scalar_type() && c.scalar_type() == a.scalar_type(), op,
              ": A, B and C must share a dtype");
  TORCH_CHECK(a.scalar_type() == at::ScalarType::BFloat16 || a.scalar_type() == at::ScalarType::Half ||
                  a.scalar_type() == at::ScalarType::Float,
              op, ": only bfloat16, float16 and float32 are supported");
  TORCH_CHECK(a.scalar_type() != at::ScalarType::Float || (!b_packed && !silu_and_mul), op,
              ": float32 runs on row-major weights without the silu_and_mul epilogue");
  TORCH_CHECK(!(silu_and_mul && mul_routed_weight), op,
              ": silu_and_mul and mul_routed_weight are different epilogues; pick one");
  TORCH_CHECK(!silu_and_mul || n % 2 == 0, op, ": silu_and_mul needs an even N (gate rows, up rows)");
  const int64_t c_cols = silu_and_mul ? n / 2 : n;
  TORCH_CHECK(c.is_contiguous() && c.size(-1) == c_cols && c.numel() == num_valid_tokens * c_cols,
              op, ": C must be contiguous and hold num_valid_tokens rows of ", c_cols, " elements");
  TORCH_CHECK(topk_weights.scalar_type() == at::ScalarType::Float && topk_weights.is_contiguous() &&
                  topk_weights.numel() >= (mul_routed_weight ? num_valid_tokens : 0),
              op, ": topk_weights must be contiguous float32 [tokens, topk]");
  TORCH_CHECK(sorted_token_ids.scalar_type() == at::ScalarType::Int &&
                  expert_ids.scalar_type() == at::ScalarType::Int &&
                  num_tokens_post_padded.scalar_type() == at::ScalarType::Int &&
                  sorted_token_ids.is_contiguous() && expert_ids.is_contiguous(),
              op, ": routing tensors must be contiguous int32");
  TORCH_CHECK(block_m > 0 && expert_ids.numel() * block_m >= sorted_token_ids.numel(), op,
              ": expert_ids is too short for sorted_token_ids and block_m");
  const int epilogue = silu_and_mul ? SARATHI_MOE_EPILOGUE_SILU_AND_MUL
                       : mul_routed_weight ? SARATHI_MOE_EPILOGUE_ROUTED_WEIGHT
                                           : SARATHI_MOE_EPILOGUE_NONE;
  const int layout = b_packed ? SARATHI_MOE_B_PACKED : SARATHI_MOE_B_ROW_MAJOR;
  LaunchScope scope(a);
  if (riders.has_value()) {
    const torch::Tensor& r = *riders;
    check_gpu(r, a, op, "riders");
    TORCH_CHECK(r.scalar_type() == at::ScalarType::Int && r.is_contiguous() &&
                    r.numel() * block_m >= sorted_token_ids.numel(),
                op, ": riders must be contiguous int32 with one entry per slot block");
    raise_on(sarathi_moe_grouped_gemm_riders(
                 a.data_ptr(), b.data_ptr(), c.data_ptr(), topk_weights.data_ptr<float>(),
                 sorted_token_ids.data_ptr<int32_t>(), expert_ids.data_ptr<int32_t>(),
                 num_tokens_post_padded.data_ptr<int32_t>(), num_valid_tokens,
                 sorted_token_ids.numel(), n, k, a.stride(0), expert_stride, c_cols, (int)block_m,
                 (int)top_k, epilogue, layout, dtype_code(a, op), r.data_ptr<int32_t>(),
                 scope.stream),
             op);
    return;
  }
  raise_on(sarathi_moe_grouped_gemm(
               a.data_ptr(), b.data_ptr(), c.data_ptr(), topk_weights.data_ptr<float>(),
               sorted_token_ids.data_ptr<int32_t>(), expert_ids.data_ptr<int32_t>(),
               num_tokens_post_padded.data_ptr<int32_t>(), num_valid_tokens,
               sorted_token_ids.numel(), n, k, a.stride(0), expert_stride, c_cols, (int)block_m,
               (int)top_k, epilogue, layout, dtype_code(a, op), scope.stream),
           op);
}

// which 32-slot tiles of partly filled last blocks ride with which full blocks (input:
// moe_align_block_size's outputs, greedy fill)
void moe_plan_riders(torch::Tensor& sorted_token_ids, torch::Tensor& expert_ids,
                     torch::Tensor& num_tokens_post_padded, int64_t num_valid_tokens,
                     int64_t block_m, torch::Tensor& riders) {
  const char* op = "moe_plan_riders";
  check_gpu(sorted_token_ids, sorted_token_ids, op, "sorted_token_ids");
  check_gpu(expert_ids, sorted_token_ids, op, "expert_ids");
  check_gpu(num_tokens_post_padded, sorted_token_ids, op, "num_tokens_post_padded");
  check_gpu(riders, sorted_token_ids, op, "riders");
  TORCH_CHECK(sorted_token_ids.scalar_type() == at::ScalarType::Int &&
                  expert_ids.scalar_type() == at::ScalarType::Int &&
                  num_tokens_post_padded.scalar_type() == at::ScalarType::Int &&
                  riders.scalar_type() == at::ScalarType::Int,
              op, ": all tensors must be int32");
  TORCH_CHECK(sorted_token_ids.is_contiguous() && expert_ids.is_contiguous() && riders.is_contiguous() &&
                  num_tokens_post_padded.numel() >= 1,
              op, ": tensors must be contiguous");
  TORCH_CHECK(block_m > 0 && expert_ids.numel() * block_m >= sorted_token_ids.numel() &&
                  riders.numel() * block_m >= sorted_token_ids.numel(),
              op, ": expert_ids / riders are too short for sorted_token_ids and block_m");
  LaunchScope scope(sorted_token_ids);
  raise_on(sarathi_moe_plan_riders(sorted_token_ids.data_ptr<int32_t>(), expert_ids.data_ptr<int32_t>(),
                                   num_tokens_post_padded.data_ptr<int32_t>(), num_valid_tokens,
                                   sorted_token_ids.numel(), (int)block_m, riders.data_ptr<int32_t>(),
                                   riders.numel(), scope.stream),
           op);
}

// per expert: riders (greedy layout kept) or even fill of its blocks (input: moe_align_block_size's
// outputs)
void moe_plan_blocks(torch::Tensor& sorted_in, torch::Tensor& sorted_out, torch::Tensor& expert_ids,
                     torch::Tensor& num_tokens_post_pad, int64_t num_experts, int64_t block_m,
                     int64_t pad_value, torch::Tensor& riders) {
  const char* op = "moe_plan_blocks";
  check_gpu(sorted_in, sorted_in, op, "sorted_in");
  check_gpu(sorted_out, sorted_in, op, "sorted_out");
  check_gpu(expert_ids, sorted_in, op, "expert_ids");
  check_gpu(num_tokens_post_pad, sorted_in, op, "num_tokens_post_pad");
  check_gpu(riders, sorted_in, op, "riders");
  TORCH_CHECK(sorted_in.scalar_type() == at::ScalarType::Int && sorted_out.scalar_type() == at::ScalarType::Int &&
                  expert_ids.scalar_type() == at::ScalarType::Int &&
                  num_tokens_post_pad.scalar_type() == at::ScalarType::Int &&
                  riders.scalar_type() == at::ScalarType::Int,
              op, ": all tensors must be int32");
  TORCH_CHECK(sorted_in.is_contiguous() && sorted_out.is_contiguous() && expert_ids.is_contiguous() &&
                  riders.is_contiguous() && sorted_in.numel() == sorted_out.numel() &&
                  num_tokens_post_pad.numel() >= 1,
              op, ": tensors must be contiguous, sorted_in and sorted_out equally long");
  TORCH_CHECK(sorted_in.data_ptr() != sorted_out.data_ptr(), op, ": cannot run in place");
  TORCH_CHECK(block_m > 0 && num_experts > 0 &&
                  expert_ids.numel() * block_m >= sorted_in.numel() &&
                  riders.numel() * block_m >= sorted_in.numel(),
              op, ": expert_ids / riders are too short for sorted_in and block_m");
  LaunchScope scope(sorted_in);
  raise_on(sarathi_moe_plan_blocks(sorted_in.data_ptr<int32_t>(), sorted_out.data_ptr<int32_t>(),
                                   expert_ids.data_ptr<int32_t>(), num_tokens_post_pad.data_ptr<int32_t>(),
                                   sorted_in.numel(), (int)num_experts, (int)block_m, (int)pad_value,
                                   riders.data_ptr<int32_t>(), riders.numel(), scope.stream),
           op);
}

// even fill of every expert's slot blocks (input: moe_align_block_size's outputs)
void moe_balance_blocks(torch::Tensor& sorted_in, torch::Tensor& sorted_out, torch::Tensor& expert_ids,
                        torch::Tensor& num_tokens_post_pad, int64_t num_experts, int64_t block_size,
                        int64_t pad_value, int64_t granule, int64_t rows_per_block) {
  const char* op = "moe_balance_blocks";
  check_gpu(sorted_in, sorted_in, op, "sorted_in");
  check_gpu(sorted_out, sorted_in, op, "sorted_out");
  check_gpu(expert_ids, sorted_in, op, "expert_ids");
  check_gpu(num_tokens_post_pad, sorted_in, op, "num_tokens_post_pad");
  TORCH_CHECK(sorted_in.scalar_type() == at::ScalarType::Int && sorted_out.scalar_type() == at::ScalarType::Int &&
                  expert_ids.scalar_type() == at::ScalarType::Int &&
                  num_tokens_post_pad.scalar_type() == at::ScalarType::Int,
              op, ": all tensors must be int32");
  TORCH_CHECK(sorted_in.is_contiguous() && sorted_out.is_contiguous() && expert_ids.is_contiguous() &&
                  sorted_in.numel() == sorted_out.numel() && num_tokens_post_pad.numel() >= 1,
              op, ": sorted_in / sorted_out must be contiguous and equally long");
  TORCH_CHECK(sorted_in.data_ptr() != sorted_out.data_ptr(), op, ": cannot run in place");
  TORCH_CHECK(block_size > 0 && granule > 0 && num_experts > 0 && rows_per_block > 0 &&
                  block_size % rows_per_block == 0 && (block_size / rows_per_block) % granule == 0,
              op, ": bad block_size / granule / rows_per_block / num_experts");
  TORCH_CHECK(expert_ids.numel() * block_size >= sorted_in.numel() - (block_size - 1), op,
              ": expert_ids is too short for sorted_in");
  LaunchScope scope(sorted_in);
  raise_on(sarathi_moe_balance_blocks(sorted_in.data_ptr<int32_t>(), sorted_out.data_ptr<int32_t>(),
                                      expert_ids.data_ptr<int32_t>(),
                                      num_tokens_post_pad.data_ptr<int32_t>(), sorted_in.numel(),
                                      (int)num_experts, (int)block_size, (int)pad_value, (int)granule,
                                      (int)rows_per_block, scope.stream),
           op);
}

// plain copy in the launch shapes of the streaming ops (bench.py's ceiling)
void stream_copy(torch::Tensor& dst, torch::Tensor& src, int64_t kib_per_wave) {
  const char* op = "stream_copy";
  check_gpu(src, src, op, "src");
  check_gpu(dst, src, op, "dst");
  TORCH_CHECK(dst.is_contiguous() && src.is_contiguous(), op, ": tensors must be contiguous");
  TORCH_CHECK(dst.nbytes() == src.nbytes(), op, ": dst and src must hold the same number of bytes");
  LaunchScope scope(src);
  raise_on(sarathi_stream_copy(dst.data_ptr(), src.data_ptr(), (int64_t)src.nbytes(),
                               (int)kib_per_wave, scope.stream),
           op);
}

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  m.doc() = "gfx950 HIP implementation of Sarathi-Serve's csrc op library";
  m.def("abi_version", &sarathi_ops_abi_version);
  m.def("stream_copy", &stream_copy,
        "device-to-device copy in the launch shapes of the streaming ops (measurement aid)");
  // layernorm_ops
  m.def("rms_norm", &rms_norm, "out = rms_norm(input) * weight");
  m.def("fused_add_rms_norm", &fused_add_rms_norm,
        "residual += input; input = rms_norm(residual) * weight (both in place)");
  // activation_ops
  m.def("moe_sum", &moe_sum, "out[t] = sum over the top_k rows of input[t]");
  m.def("silu_and_mul", &silu_and_mul, "out = silu(input[:, :d]) * input[:, d:]");
  m.def("gelu_new", &gelu_new, "GPT-2 tanh GELU");
  m.def("gelu_fast", &gelu_fast, "approximate tanh GELU");
  // pos_encoding_ops
  m.def("rotary_embedding", &rotary_embedding,
        "in-place GPT-NeoX / GPT-J rotary embedding of query and key");
  // kv_cache_ops
  m.def("get_seq_lens", &get_seq_lens, "kv sequence lengths from the page table");
  m.def("get_batch_indices_positions", &get_batch_indices_positions,
        "request index and kv position of every appended token");
  m.def("get_kv_slot_mapping", &get_kv_slot_mapping,
        "page * page_size + entry of every appended token");
  m.def("append_paged_kv_cache", &append_paged_kv_cache,
        "copy key / value rows into their entries of a paged (NHD) KV cache",
        pybind11::arg("append_key"), pybind11::arg("append_value"), pybind11::arg("batch_indices"),
        pybind11::arg("positions"), pybind11::arg("k_cache"), pybind11::arg("v_cache"),
        pybind11::arg("kv_indices"), pybind11::arg("kv_indptr"),
        pybind11::arg("slot_mapping") = pybind11::none());
  m.def("rotary_embedding_append_paged_kv", &rotary_embedding_append_paged_kv,
        "rotary_embedding fused with append_paged_kv_cache", pybind11::arg("positions"),
        pybind11::arg("query"), pybind11::arg("key"), pybind11::arg("value"),
        pybind11::arg("head_size"), pybind11::arg("cos_sin_cache"), pybind11::arg("is_neox"),
        pybind11::arg("batch_indices"), pybind11::arg("append_positions"),
        pybind11::arg("k_cache"), pybind11::arg("v_cache"), pybind11::arg("kv_indices"),
        pybind11::arg("kv_indptr"), pybind11::arg("num_append_tokens"),
        pybind11::arg("write_key"), pybind11::arg("slot_mapping") = pybind11::none());
  // moe_ops
  m.def("topk_softmax", &topk_softmax, "softmax over experts + top-k (raw probabilities)");
  m.def("topk_softmax_renorm", &topk_softmax_renorm,
        "topk_softmax with the k weights of each token renormalised to sum to 1");
  m.def("moe_align_block_size", &moe_align_block_size,
        "stable sort of token ids by expert, runs padded to block_size");
  m.def("moe_align_block_size_filled", &moe_align_block_size_filled,
        "moe_align_block_size that also writes the padding value into unused slots");
  m.def("grouped_topk", &grouped_topk,
        "softmax, keep the best topk_group of num_expert_group expert groups, top-k of the rest");
  m.def("fused_topk_align", &fused_topk_align,
        "topk_softmax (+ optional renormalisation) and moe_align_block_size in one launch");
  m.def("moe_balance_blocks", &moe_balance_blocks,
        "spread every expert's slots evenly over its blocks (for the grouped GEMM)",
        pybind11::arg("sorted_in"), pybind11::arg("sorted_out"), pybind11::arg("expert_ids"),
        pybind11::arg("num_tokens_post_pad"), pybind11::arg("num_experts"), pybind11::arg("block_size"),
        pybind11::arg("pad_value"), pybind11::arg("granule"), pybind11::arg("rows_per_block") = 1);
  m.def("moe_gemm_slot_rows", [](int64_t block_m, bool b_packed) {
          const int r = sarathi_moe_gemm_slot_rows((int)block_m, b_packed ? SARATHI_MOE_B_PACKED
                                                                          : SARATHI_MOE_B_ROW_MAJOR);
          raise_on(r < 0 ? r : SARATHI_OK, "moe_gemm_slot_rows");
          return (int64_t)r;
        },
        "ranges of a slot block that separate waves of the grouped GEMM kernel sweep (1 or 2)");
  m.def("moe_grouped_gemm", &moe_grouped_gemm,
        "C[slot] = A[slot / top_k] @ B[expert(slot)]^T over moe_align_block_size's layout",
        pybind11::arg("a"), pybind11::arg("b"), pybind11::arg("c"), pybind11::arg("topk_weights"),
        pybind11::arg("sorted_token_ids"), pybind11::arg("expert_ids"),
        pybind11::arg("num_tokens_post_padded"), pybind11::arg("num_valid_tokens"),
        pybind11::arg("block_m"), pybind11::arg("top_k"), pybind11::arg("mul_routed_weight"),
        pybind11::arg("b_packed") = false, pybind11::arg("n") = 0,
        pybind11::arg("silu_and_mul") = false, pybind11::arg("riders") = pybind11::none());
  m.def("moe_plan_blocks", &moe_plan_blocks,
        "per expert: riders for its last block, or its slots spread evenly over its blocks",
        pybind11::arg("sorted_in"), pybind11::arg("sorted_out"), pybind11::arg("expert_ids"),
        pybind11::arg("num_tokens_post_pad"), pybind11::arg("num_experts"), pybind11::arg("block_m"),
        pybind11::arg("pad_value"), pybind11::arg("riders"));
  m.def("moe_plan_riders", &moe_plan_riders,
        "for moe_grouped_gemm(riders=...): tiles of partly filled last blocks that full blocks take along",
        pybind11::arg("sorted_token_ids"), pybind11::arg("expert_ids"),
        pybind11::arg("num_tokens_post_padded"), pybind11::arg("num_valid_tokens"),
        pybind11::arg("block_m"), pybind11::arg("riders"));
}
