// topk_softmax and moe_align_block_size in one launch.
//
// The reference's MoE layer issues the two ops back to back for every layer
// (sarathi/model_executor/layers/fused_moe/fused_moe.py:363-372 and :192-203); both are latency
// bound, so a kernel boundary (drain, launch, ramp) is a large part of their cost.  Here
// workgroups of 16 waves compute the top-k of 16 row blocks each, exactly as the stand-alone
// kernel does, except that the expert ids are stored as device-scope atomics (written through to
// where every compute unit reads coherently); once every wave has waited for the
// acknowledgement of its stores (s_waitcnt vmcnt(0)) and met the others at a barrier, the workgroup
// bumps a counter in global memory, and the workgroup that sees the last count runs the
// single-workgroup sort, reading the ids of all workgroups with device-scope loads.  (A full
// device-scope fence on either side also works but costs several microseconds of cache
// write-back and invalidation, more than the launch it saves.)  No workgroup waits for another one: every
// wave reaches its exit whatever the others do.  The counter must be zero on entry and is zero
// again on exit; calls that share a counter must not overlap.
//
// The one launch pays only while the sort is small: its last workgroup sorts alone, on one compute
// unit, where the stand-alone moe_align_block_size spreads over several.  Measured on MI355X
// (8 experts, top-2, launches issued back to back): 32 ids 5.7 us against 6.8 us for the two
// launches, 1024 ids 6.7 against 6.7, 4096 ids 9.0 against 7.7, 8192 ids 12.5 against 8.9; with 64
// experts and top-6 it loses from 384 ids on.  So the entry point runs the fused kernel up to
// 1024 ids and 16 experts (a power of two) and the two stand-alone launches otherwise; results are
// identical either way.
#include "moe_align_body.h"
#include "moe_topk_body.h"
#include "launch.h"

namespace sarathi_hip {

constexpr int kFusedWaves = 16;
constexpr int64_t kFusedMaxIds = 1024;
constexpr int kFusedMaxExperts = 16;

template <int E>
__global__ __launch_bounds__(64 * kFusedWaves) void fused_topk_align_kernel(
    float* __restrict__ weights, int32_t* indices, int32_t* __restrict__ source,
    const float* __restrict__ gating, int64_t num_tokens, int k, int renormalize, int B, int nbits,
    int32_t* __restrict__ sorted, int64_t sorted_len, int32_t* __restrict__ expert_ids,
    int64_t expert_ids_len, int32_t* __restrict__ post_pad, int fill_pad, uint32_t* counter) {
  __shared__ int32_t cnt[kFusedWaves * 256];
  __shared__ int32_t tot[256];
  __shared__ int32_t cumsum[256 + 1];
  __shared__ int last;

  constexpr int rows = Pow2Layout<E>::ROWS_PER_WAVE;
  const int64_t row_blocks = (num_tokens + rows - 1) / rows;
  const int64_t block = (int64_t)blockIdx.x * kFusedWaves + (threadIdx.x >> 6);
  if (block < row_blocks)  // uniform over the wave
    topk_rows_pow2<E, true>(block, weights, indices, source, gating, num_tokens, k, renormalize);

  // Publication: the ids above are write-through (device-scope) stores, and their
  // acknowledgement, which vmcnt counts, comes back once they are where every compute unit reads
  // coherently.  Every wave waits for its own stores here; the barrier that follows then tells
  // thread 0 that all ids of this workgroup are visible before it bumps the counter.  (The
  // barrier alone does not: its workgroup-scope fence does not wait for global stores.)  The
  // textbook form -- plain stores, an agent-scope acquire-release fetch-add on the counter, plain
  // loads in the sorting workgroup -- is also correct and was measured: 5.4 / 6.0 / 6.7 / 7.3 us
  // at 16 / 64 / 256 / 512 tokens (8 experts, top-2) against 5.5 / 5.8 / 6.2 / 7.1 us for this
  // form; its release writes back and its acquire invalidates whole caches.
  wait_vmcnt<0>();
  __syncthreads();
  if (threadIdx.x == 0) {
    const uint32_t prev = atomicAdd(counter, 1u);
    const bool is_last = prev == gridDim.x - 1;
    if (is_last) atomicExch(counter, 0u);  // ready for the next call
    last = is_last;
  }
  __syncthreads();
  if (!last) return;
  align_single_workgroup<int32_t, true>(indices, num_tokens * k, E, B, nbits, sorted, sorted_len,
                                  expert_ids, expert_ids_len, post_pad, fill_pad, cnt, tot, cumsum);
}
template <int E>
static void launch_fused(float* w, int32_t* idx, int32_t* src, const float* g, int64_t T, int k,
                         int renorm, int B, int32_t* sorted, int64_t sorted_len,
                         int32_t* expert_ids, int64_t expert_ids_len, int32_t* post_pad,
                         int fill_pad, uint32_t* counter, hipStream_t st) {
  constexpr int rows = Pow2Layout<E>::ROWS_PER_WAVE;
  const int64_t row_blocks = (T + rows - 1) / rows;
  const int64_t grid = (row_blocks + kFusedWaves - 1) / kFusedWaves;
  int nbits = 0;
  while ((1 << nbits) < E) ++nbits;
  hipLaunchKernelGGL((fused_topk_align_kernel<E>), dim3((unsigned)grid), dim3(64 * kFusedWaves), 0,
                     st, w, idx, src, g, T, k, renorm, B, nbits, sorted, sorted_len, expert_ids,
                     expert_ids_len, post_pad, fill_pad, counter);
}

}  // namespace sarathi_hip

extern "C" int sarathi_fused_topk_align(float* topk_weights, int32_t* topk_indices,
                                        int32_t* token_expert_indices, const float* gating_output,
                                        int64_t num_tokens, int num_experts, int topk,
                                        int renormalize, int block_size,
                                        int32_t* sorted_token_ids, int64_t sorted_len,
                                        int32_t* expert_ids, int64_t expert_ids_len,
                                        int32_t* num_tokens_post_pad, int fill_pad,
                                        uint32_t* counter, void* stream) {
  using namespace sarathi_hip;
  if (!num_tokens_post_pad || (sorted_len > 0 && !sorted_token_ids) ||
      (expert_ids_len > 0 && !expert_ids))
    return SARATHI_ERR_INVALID_ARG;
  if (num_tokens > 0 && (!topk_weights || !topk_indices || !token_expert_indices || !gating_output))
    return SARATHI_ERR_INVALID_ARG;
  if (num_tokens < 0 || num_experts <= 0 || topk <= 0 || topk > num_experts || block_size <= 0 ||
      sorted_len < 0 || expert_ids_len < 0)
    return SARATHI_ERR_INVALID_ARG;
  if (num_experts > SARATHI_MOE_MAX_EXPERTS) return SARATHI_ERR_UNSUPPORTED;
  const int64_t numel = num_tokens * (int64_t)topk;
  if (numel > 0x7fffffffLL) return SARATHI_ERR_UNSUPPORTED;
  const int64_t nonempty_max = numel < num_experts ? numel : num_experts;
  const int64_t worst = numel + nonempty_max * ((int64_t)block_size - 1);
  if (worst > 0x7fffffffLL) return SARATHI_ERR_UNSUPPORTED;
  if (sorted_len < worst || expert_ids_len * (int64_t)block_size < worst)
    return SARATHI_ERR_INVALID_ARG;
  const int E = num_experts;
  const bool fusable = counter != nullptr && num_tokens > 0 && numel <= kFusedMaxIds &&
                       (E & (E - 1)) == 0 && E <= kFusedMaxExperts &&
                       (reinterpret_cast<uintptr_t>(gating_output) & (E < 4 ? E * 4 - 1 : 15)) == 0;
  if (!fusable) {
    // (zero tokens: topk_softmax is a no-op and the sort still writes num_tokens_post_pad = 0)
    int rc = sarathi_topk_softmax(topk_weights, topk_indices, token_expert_indices, gating_output,
                                  num_tokens, num_experts, topk, renormalize, stream);
    if (rc != SARATHI_OK) return rc;
    return sarathi_moe_align_block_size(topk_indices, SARATHI_IDTYPE_I32, numel, num_experts,
                                        block_size, sorted_token_ids, sorted_len, expert_ids,
                                        expert_ids_len, num_tokens_post_pad, fill_pad, nullptr, 0,
                                        stream);
  }
  hipStream_t st = (hipStream_t)stream;
#define SK_FUSED(N)                                                                             \
  case N:                                                                                       \
    launch_fused<N>(topk_weights, topk_indices, token_expert_indices, gating_output, num_tokens, \
                    topk, renormalize, block_size, sorted_token_ids, sorted_len, expert_ids,    \
                    expert_ids_len, num_tokens_post_pad, fill_pad, counter, st);                \
    return launch_status();
  switch (E) {
    SK_FUSED(1) SK_FUSED(2) SK_FUSED(4) SK_FUSED(8) SK_FUSED(16) SK_FUSED(32) SK_FUSED(64)
    SK_FUSED(128) SK_FUSED(256)
    default: return SARATHI_ERR_UNSUPPORTED;
  }
#undef SK_FUSED
}
