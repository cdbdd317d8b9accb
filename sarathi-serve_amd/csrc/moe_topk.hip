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
#include "vec16.h"
#include "launch.h"

namespace sarathi_hip {

constexpr int kTopkBlock = 64;

SK_DEV bool beats(float v, int e, float best_v, int best_e) {
  return v > best_v || (v == best_v && e < best_e);
}

template <int E>
struct Pow2Layout {
  static constexpr int ELTS = E < 4 ? E : 4;                         // floats per load
  static constexpr int VECS = (E / (ELTS * 32)) > 1 ? (E / (ELTS * 32)) : 1;
  static constexpr int VPT = VECS * ELTS;                            // values per lane
  static constexpr int G = E / VPT;                                  // lanes per row
  static constexpr int COLS_PER_VEC = ELTS * G;
  static constexpr int ROWS_PER_WAVE = 64 / G;
};

template <int E>
__global__ __launch_bounds__(kTopkBlock) void topk_softmax_pow2_kernel(
    float* __restrict__ weights, int32_t* __restrict__ indices, int32_t* __restrict__ source,
    const float* __restrict__ gating, int64_t num_tokens, int k, int renormalize) {
  using L = Pow2Layout<E>;
  const int lane = threadIdx.x;
  const int g = lane % L::G;
  const int64_t row = (int64_t)blockIdx.x * L::ROWS_PER_WAVE + lane / L::G;
  // Lanes of rows past the end keep running on row 0's data so that the group
  // shuffles below always see live lanes; they just never store.
  const bool live = row < num_tokens;
  const float* rp = gating + (live ? row : 0) * E;

  float v[L::VPT];
#pragma unroll
  for (int l = 0; l < L::VECS; ++l) {
    const float* p = rp + l * L::COLS_PER_VEC + g * L::ELTS;
    if constexpr (L::ELTS == 4) {
      u32x4 q = *reinterpret_cast<const u32x4*>(p);
#pragma unroll
      for (int i = 0; i < 4; ++i) v[l * 4 + i] = as_f32(q[i]);
    } else if constexpr (L::ELTS == 2) {
      u32x2 q = *reinterpret_cast<const u32x2*>(p);
      v[0] = as_f32(q.x);
      v[1] = as_f32(q.y);
    } else {
      v[0] = p[0];
    }
  }

  float m = v[0];
#pragma unroll
  for (int i = 1; i < L::VPT; ++i) m = fmaxf(m, v[i]);
#pragma unroll
  for (int mask = L::G / 2; mask > 0; mask >>= 1) m = fmaxf(m, __shfl_xor(m, mask, 64));

  float sum = 0.f;
#pragma unroll
  for (int i = 0; i < L::VPT; ++i) {
    v[i] = expf(v[i] - m);
    sum += v[i];
  }
#pragma unroll
  for (int mask = L::G / 2; mask > 0; mask >>= 1) sum += __shfl_xor(sum, mask, 64);
  const float recip = 1.f / sum;
#pragma unroll
  for (int i = 0; i < L::VPT; ++i) v[i] = v[i] * recip;

  float wsum = 0.f;
  for (int j = 0; j < k; ++j) {
    float best = v[0];
    int be = g * L::ELTS;
#pragma unroll
    for (int i = 1; i < L::VPT; ++i) {
      const int col = (i / L::ELTS) * L::COLS_PER_VEC + g * L::ELTS + (i % L::ELTS);
      if (v[i] > best) { best = v[i]; be = col; }
    }
#pragma unroll
    for (int mask = L::G / 2; mask > 0; mask >>= 1) {
      float ov = __shfl_xor(best, mask, 64);
      int oe = __shfl_xor(be, mask, 64);
      if (beats(ov, oe, best, be)) { best = ov; be = oe; }
    }
    if (live && g == 0) {
      const int64_t o = row * k + j;
      weights[o] = best;
      indices[o] = be;
      source[o] = (int32_t)((int64_t)j * num_tokens + row);
    }
    wsum += best;
    // the lane that owns column `be` blanks it
    const int owner = (be / L::ELTS) % L::G;
    const int reg = (be / L::COLS_PER_VEC) * L::ELTS + be % L::ELTS;
#pragma unroll
    for (int i = 0; i < L::VPT; ++i)
      if (g == owner && i == reg) v[i] = -10000.f;
  }
  if (renormalize && live && g == 0) {
    for (int j = 0; j < k; ++j) weights[row * k + j] = weights[row * k + j] / wsum;
  }
}

// One wave per row, R = ceil(E / 64) values per lane.
template <int R>
__global__ __launch_bounds__(kTopkBlock) void topk_softmax_wave_kernel(
    float* __restrict__ weights, int32_t* __restrict__ indices, int32_t* __restrict__ source,
    const float* __restrict__ gating, int64_t num_tokens, int E, int k, int renormalize) {
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
    v[r] = c < E ? v[r] * recip : -20000.f;  // padding never wins, not even after blanking
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
      const int64_t o = row * k + j;
      weights[o] = best;
      indices[o] = be;
      source[o] = (int32_t)((int64_t)j * num_tokens + row);
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
  if (!topk_weights || !topk_indices || !token_expert_indices || !gating_output)
    return SARATHI_ERR_INVALID_ARG;
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
