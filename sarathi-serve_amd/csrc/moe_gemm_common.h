// Pieces shared by the grouped expert GEMM kernels (moe_gemm.hip, moe_gemm_lds.hip).
#pragma once

#include <stdint.h>

#include "vec16.h"

namespace sarathi_hip {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));

constexpr int kGemmBN = 256;   // output columns per workgroup
constexpr int kGemmBK = 64;    // K elements per pipeline step
constexpr int kGemmWaveN = 64; // output columns per wave

enum : int { kEpiPlain = 0, kEpiMulWeight = 1, kEpiGatedSilu = 2 };

template <int DT> SK_DEV f32x16 mfma32(u32x4 a, u32x4 b, f32x16 c) {
  if constexpr (DT == kBF16)
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a),
                                                   __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  else
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a),
                                                  __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
}

// Position (0..7) of 16-byte chunk c inside row r of the token tile in LDS.  Rows are 128 bytes,
// i.e. exactly one pass over the 32 banks, so the bank group of an access is this position.
// An operand read has lane (row r, half g) fetch chunk 2s + g; the rotation below makes the
// positions distinct both over eight consecutive rows of one half and over four consecutive
// rows of both halves, whichever way the hardware groups the lanes of a 128-bit read.
SK_DEV int lds_slot(int r, int c) { return (c + 2 * (r & 3) + ((r >> 2) & 1)) & 7; }

// 16 bytes per lane from a buffer straight into LDS: lane l lands at lds_base + 16 l
// (lds_base is uniform over the wave).  Completion is tracked by the wave's vmcnt.
SK_DEV void dma_load16_to_lds(rsrc_t r, u32x4* lds_base, uint32_t byte_off) {
  __builtin_amdgcn_raw_ptr_buffer_load_lds(
      r, (__attribute__((address_space(3))) void*)lds_base, 16, byte_off, 0, 0, 0);
}

// Waits until at most N vector-memory operations of this wave are outstanding.
template <int N> SK_DEV void wait_vmcnt() { asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory"); }

struct MoeGemmArgs {
  const void* a;            // [tokens, K]
  const void* b;            // [E, N, K]
  void* c;                  // [tokens * top_k, N]
  const float* topk_weights;        // flat [tokens * top_k] or null
  const int32_t* sorted_token_ids;  // [em]
  const int32_t* expert_ids;        // [ceil(em / BM)]
  const int32_t* num_tokens_post_padded;
  uint32_t a_bytes;         // extent of A in bytes; a_bytes + 2*K stays below 4 GiB
  int64_t a_row_stride;     // elements
  int64_t b_expert_stride;  // elements
  int64_t c_row_stride;     // elements
  int32_t num_valid;        // tokens * top_k
  int32_t em;               // length of sorted_token_ids
  int32_t N, K;
  int32_t top_k;
  int32_t m_blocks, n_blocks;
};

}  // namespace sarathi_hip
