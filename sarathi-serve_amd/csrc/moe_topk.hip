// topk_softmax (MoE gating) for gfx950.
//
// Replaces csrc/moe_topk_softmax_kernels.cu:50-503 of the reference.  Two
// kernels, neither needs a workspace:
//
//  * num_experts a power of two up to 256: a row of logits is shared by a
//    group of G lanes of a 64-lane wave (G = 1..32, so a wave holds 2..64
//    rows).  The column-to-lane assignment and the order in which the
//    exponentials are added (per lane in register order, then an xor butterfly
//    over the group) are those of the reference's fast path
//    (csrc/moe_topk_softmax_kernels.cu:236-303), so the softmax denominators
//    carry the same rounding.  Top-k is k rounds of "largest probability, lower
//    expert index on ties" (:311-346) with the winner blanked to -10000 (:376).
//
//  * any other num_experts up to 1024: one wave per row, lane l holds columns
//    l, l+64, ...; same selection rule.  This covers what the reference does
//    with two launches and a [tokens, experts] workspace (:50-166, :460-469).
//
// Output order is descending probability; token_expert_indices[t,j] = j*T + t.
// With renormalize != 0 the k weights of a row are divided by their sum
// (added in selection order), the step the reference's Python caller performs
// separately (sarathi/model_executor/layers/fused_moe/fused_moe.py:371-372).
#include "moe_topk_body.h"
#include "launch.h"

namespace sarathi_hip {

template <int E>
__global__ __launch_bounds__(kTopkBlock) void topk_softmax_pow2_kernel(
    float* __restrict__ weights, int32_t* __restrict__ indices, int32_t* __restrict__ source,
    const float* __restrict__ gating, int64_t num_tokens, int k, int renormalize) {
  topk_rows_pow2<E>(blockIdx.x, weights, indices, source, gating, num_tokens, k, renormalize);
}

template <int R>
__global__ __launch_bounds__(kTopkBlock) void topk_softmax_wave_kernel(
    float* __restrict__ weights, int32_t* __restrict__ indices, int32_t* __restrict__ source,
    const float* __restrict__ gating, int64_t num_tokens, int E, int k, int renormalize) {
  topk_row_wave<R>(blockIdx.x, weights, indices, source, gating, num_tokens, E, k, renormalize);
}

// grouped_topk (the routing of DeepSeek-V2 style models; the reference does it with tensor ops,
// sarathi/model_executor/layers/fused_moe/fused_moe.py:377-408): softmax over all experts, the
// experts form num_groups equal consecutive groups, the topk_group groups with the largest
// member score stay, every other expert's score becomes 0, then top-k of what is left.  One
// wave per row; equal scores resolve to the lower group / expert index; output in descending
// score order.
template <int R>
__global__ __launch_bounds__(kTopkBlock) void grouped_topk_wave_kernel(
    float* __restrict__ weights, int32_t* __restrict__ indices, const float* __restrict__ gating,
    int64_t num_tokens, int E, int k, int num_groups, int topk_group, int renormalize) {
  __shared__ float prob[SARATHI_MOE_MAX_EXPERTS];
  const int lane = threadIdx.x;
  const int64_t row = blockIdx.x;
  const float* rp = gating + row * E;
  constexpr float kLowest = -3.402823466e+38f;

  float v[R];
  float m = kLowest;
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int c = lane + 64 * r;
    v[r] = c < E ? rp[c] : kLowest;
    m = fmaxf(m, v[r]);
  }
  m = wave64_max(m);
  float sum = 0.f;
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int c = lane + 64 * r;
    v[r] = c < E ? expf(v[r] - m) : 0.f;
    sum += v[r];
  }
#pragma unroll
  for (int mask = 32; mask > 0; mask >>= 1) sum += __shfl_xor(sum, mask, 64);
  const float recip = 1.f / sum;
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int c = lane + 64 * r;
    v[r] = v[r] * recip;
    if (c < E) prob[c] = v[r];
  }
  __syncthreads();

  // lane g holds the best score of group g
  const int group_size = E / num_groups;
  float gmax = -1.f;
  if (lane < num_groups) {
    for (int i = 0; i < group_size; ++i) gmax = fmaxf(gmax, prob[lane * group_size + i]);
  }
  unsigned long long chosen = 0;
  for (int j = 0; j < topk_group; ++j) {
    float best = gmax;
    int bg = lane;
#pragma unroll
    for (int mask = 32; mask > 0; mask >>= 1) {
      float ov = __shfl_xor(best, mask, 64);
      int og = __shfl_xor(bg, mask, 64);
      if (beats(ov, og, best, bg)) { best = ov; bg = og; }
    }
    chosen |= 1ull << bg;
    if (lane == bg) gmax = -2.f;
  }
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int c = lane + 64 * r;
    if (c >= E) v[r] = -20000.f;  // padding never wins, not even after blanking
    else if (!((chosen >> (c / group_size)) & 1ull)) v[r] = 0.f;
  }

  float wsum = 0.f;
  for (int j = 0; j < k; ++j) {
    float best = v[0];
    int be = lane;
#pragma unroll
    for (int r = 1; r < R; ++r)
      if (v[r] > best) { best = v[r]; be = lane + 64 * r; }
#pragma unroll
    for (int mask = 32; mask > 0; mask >>= 1) {
      float ov = __shfl_xor(best, mask, 64);
      int oe = __shfl_xor(be, mask, 64);
      if (beats(ov, oe, best, be)) { best = ov; be = oe; }
    }
    if (lane == 0) {
      weights[row * k + j] = best;
      indices[row * k + j] = be;
    }
    wsum += best;
#pragma unroll
    for (int r = 0; r < R; ++r)
      if (lane == (be & 63) && r == (be >> 6)) v[r] = -10000.f;
  }
  if (renormalize && lane == 0) {
    for (int j = 0; j < k; ++j) weights[row * k + j] = weights[row * k + j] / wsum;
  }
}

template <int E>
static void launch_pow2(float* w, int32_t* idx, int32_t* src, const float* g, int64_t T, int k,
                        int renorm, hipStream_t st) {
  constexpr int rows = Pow2Layout<E>::ROWS_PER_WAVE;
  const int64_t blocks = (T + rows - 1) / rows;
  hipLaunchKernelGGL((topk_softmax_pow2_kernel<E>), dim3((unsigned)blocks), dim3(kTopkBlock), 0,
                     st, w, idx, src, g, T, k, renorm);
}

}  // namespace sarathi_hip

extern "C" int sarathi_topk_softmax(float* topk_weights, int32_t* topk_indices,
                                    int32_t* token_expert_indices, const float* gating_output,
                                    int64_t num_tokens, int num_experts, int topk,
                                    int renormalize, void* stream) {
  using namespace sarathi_hip;
  if (num_tokens > 0 && (!topk_weights || !topk_indices || !token_expert_indices || !gating_output))
    return SARATHI_ERR_INVALID_ARG;  // empty tensors have no data
  if (num_tokens < 0 || num_experts <= 0 || topk <= 0 || topk > num_experts)
    return SARATHI_ERR_INVALID_ARG;
  if (num_experts > SARATHI_MOE_MAX_EXPERTS) return SARATHI_ERR_UNSUPPORTED;
  // token_expert_indices holds j*T + t in int32
  if (num_tokens * (int64_t)topk > 0x7fffffffLL) return SARATHI_ERR_UNSUPPORTED;
  if (num_tokens == 0) return SARATHI_OK;
  hipStream_t st = (hipStream_t)stream;
  const int E = num_experts;
  const bool pow2 = (E & (E - 1)) == 0 && E <= 256 &&
                    (reinterpret_cast<uintptr_t>(gating_output) & (E < 4 ? E * 4 - 1 : 15)) == 0;
#define SK_P2(N)                                                                       \
  case N:                                                                              \
    launch_pow2<N>(topk_weights, topk_indices, token_expert_indices, gating_output,    \
                   num_tokens, topk, renormalize, st);                                 \
    return launch_status();
  if (pow2) {
    switch (E) {
      SK_P2(1) SK_P2(2) SK_P2(4) SK_P2(8) SK_P2(16) SK_P2(32) SK_P2(64) SK_P2(128) SK_P2(256)
      default: break;
    }
  }
#undef SK_P2
  const int R = (E + 63) / 64;
#define SK_WAVE(N)                                                                              \
  hipLaunchKernelGGL((topk_softmax_wave_kernel<N>), dim3((unsigned)num_tokens),                 \
                     dim3(kTopkBlock), 0, st, topk_weights, topk_indices, token_expert_indices, \
                     gating_output, num_tokens, E, topk, renormalize)
  if (R <= 1) SK_WAVE(1);
  else if (R <= 2) SK_WAVE(2);
  else if (R <= 4) SK_WAVE(4);
  else if (R <= 8) SK_WAVE(8);
  else SK_WAVE(16);
#undef SK_WAVE
  return launch_status();
}

extern "C" int sarathi_grouped_topk(float* topk_weights, int32_t* topk_indices,
                                    const float* gating_output, int64_t num_tokens,
                                    int num_experts, int topk, int num_expert_group,
                                    int topk_group, int renormalize, void* stream) {
  using namespace sarathi_hip;
  if (num_tokens > 0 && (!topk_weights || !topk_indices || !gating_output))
    return SARATHI_ERR_INVALID_ARG;
  if (num_tokens < 0 || num_experts <= 0 || topk <= 0 || topk > num_experts ||
      num_expert_group <= 0 || topk_group <= 0 || topk_group > num_expert_group ||
      num_experts % num_expert_group != 0)
    return SARATHI_ERR_INVALID_ARG;
  if (num_experts > SARATHI_MOE_MAX_EXPERTS || num_expert_group > 64)
    return SARATHI_ERR_UNSUPPORTED;
  if (num_tokens > 0x7fffffffLL) return SARATHI_ERR_UNSUPPORTED;
  if (num_tokens == 0) return SARATHI_OK;
  hipStream_t st = (hipStream_t)stream;
  const int R = (num_experts + 63) / 64;
#define SK_GROUPED(N)                                                                          \
  hipLaunchKernelGGL((grouped_topk_wave_kernel<N>), dim3((unsigned)num_tokens),                \
                     dim3(kTopkBlock), 0, st, topk_weights, topk_indices, gating_output,       \
                     num_tokens, num_experts, topk, num_expert_group, topk_group, renormalize)
  if (R <= 1) SK_GROUPED(1);
  else if (R <= 2) SK_GROUPED(2);
  else if (R <= 4) SK_GROUPED(4);
  else if (R <= 8) SK_GROUPED(8);
  else SK_GROUPED(16);
#undef SK_GROUPED
  return launch_status();
}
