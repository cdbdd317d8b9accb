// Device-side bodies of topk_softmax, shared by the stand-alone kernels (moe_topk.hip) and the
// fused routing kernel (moe_fused_routing.hip).  A body is executed by one whole wave.
#pragma once

#include "vec16.h"

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

// Stores an expert id.  PUBLISH: as a device-scope relaxed atomic, i.e. written through to the
// level of the memory system that every compute unit of the device reads coherently, for
// consumers in other workgroups of the same launch.
template <bool PUBLISH> SK_DEV void store_index(int32_t* p, int32_t v) {
  if constexpr (PUBLISH) __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  else *p = v;
}

// One wave: rows [block * ROWS_PER_WAVE, (block + 1) * ROWS_PER_WAVE).
template <int E, bool PUBLISH = false>
SK_DEV void topk_rows_pow2(int64_t block, float* __restrict__ weights, int32_t* indices,
                           int32_t* __restrict__ source, const float* __restrict__ gating,
                           int64_t num_tokens, int k, int renormalize) {
  using L = Pow2Layout<E>;
  const int lane = threadIdx.x & 63;
  const int g = lane % L::G;
  const int64_t row = block * L::ROWS_PER_WAVE + lane / L::G;
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
      store_index<PUBLISH>(&indices[o], be);
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
SK_DEV void topk_row_wave(int64_t row, float* __restrict__ weights, int32_t* indices,
                          int32_t* __restrict__ source, const float* __restrict__ gating,
                          int64_t num_tokens, int E, int k, int renormalize) {
  const int lane = threadIdx.x & 63;
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

}  // namespace sarathi_hip
