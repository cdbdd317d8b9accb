// Pieces shared by the grouped expert GEMM kernels (moe_gemm.hip, moe_gemm_wide.hip).
#pragma once

#include <stdint.h>

#include <type_traits>
#include "vec16.h"

namespace sarathi_hip {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));

constexpr int kGemmBN = 256;   // output columns per workgroup
constexpr int kGemmBK = 64;    // K elements per pipeline step
constexpr int kGemmWaveN = 64; // output columns per wave
// column blocks of an XCD in flight side by side (measured at 512..4096 tokens of the Mixtral
// layer: 2 and 4 within noise of each other, 1 and 8+ slower by 3-18 %)
constexpr int kGemmGroupN = 4;

enum : int { kEpiPlain = 0, kEpiMulWeight = 1, kEpiGatedSilu = 2 };

template <int DT> SK_DEV f32x16 mfma32(u32x4 a, u32x4 b, f32x16 c) {
  if constexpr (DT == kBF16)
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a),
                                                   __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  else
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a),
                                                  __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
}

// Rows of an operand tile in LDS are 128 bytes: eight 16-byte chunks, half a pass over the 64
// banks.  A 128-bit operand read is served sixteen lanes at a time (16 x 16 bytes = all 64 banks
// once); an MFMA operand read has those sixteen lanes fetch the same chunk of sixteen consecutive
// rows.  Even and odd rows already sit in different bank halves, so rotating the chunks of row r
// by (r >> 1) & 7 spreads the sixteen rows over all banks.  (Measured with
// SQ_LDS_BANK_CONFLICT: none with this rotation, every second LDS cycle with one that repeats
// after eight rows.)
SK_DEV int lds_rot(int r) { return (r >> 1) & 7; }
// Position (0..7) of chunk c inside row r, and the chunk that position p of row r holds.
SK_DEV int lds_slot(int r, int c) { return (c + lds_rot(r)) & 7; }
SK_DEV int lds_chunk_at(int r, int p) { return (p - lds_rot(r)) & 7; }

// 16 bytes per lane from a buffer straight into LDS: lane l lands at lds_base + 16 l
// (lds_base is uniform over the wave).  Completion is tracked by the wave's vmcnt.
SK_DEV void dma_load16_to_lds(rsrc_t r, u32x4* lds_base, uint32_t byte_off) {
  __builtin_amdgcn_raw_ptr_buffer_load_lds(
      r, (__attribute__((address_space(3))) void*)lds_base, 16, byte_off, 0, 0, 0);
}

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
  int32_t group_n;          // column blocks of one XCD that run side by side (see tile_of_block)
};

// Workgroup id -> (slot block, column block).  The hardware deals consecutive workgroup ids to
// the eight XCDs in turn, so id & 7 names the XCD (own L2) and column blocks are dealt to XCDs
// by pid_n & 7.  Within an XCD the tiles run in this order: group_n column blocks at a time, and
// inside such a group all slot blocks, the column blocks of the group innermost.  The compute
// units of an XCD therefore work at the same time on (resident workgroups / group_n) slot blocks
// x group_n column blocks: every token tile is pulled into that L2 once per group_n column blocks
// and every weight tile once per expert, instead of the whole activation matrix once per column
// block.
SK_DEV bool tile_of_block(const MoeGemmArgs& g, unsigned id, int& pid_m, int& pid_n) {
  const int xcd = id & 7u, t = id >> 3;
  const int n_local = (g.n_blocks + 7) >> 3;
  const int per_group = g.m_blocks * g.group_n;
  const int grp = t / per_group, rem = t - grp * per_group;
  const int g0 = grp * g.group_n;
  const int gsize = n_local - g0 < g.group_n ? n_local - g0 : g.group_n;
  pid_m = rem / gsize;
  pid_n = (g0 + rem - pid_m * gsize) * 8 + xcd;
  return pid_n < g.n_blocks;
}

// Calls f(std::integral_constant<int, n>) with n = min(live, L): lets a loop be compiled once per
// possible count of live tiles, each copy free of branches.
template <int L, typename F> SK_DEV void call_with_live(int live, F& f) {
  if constexpr (L == 0) {
    f(std::integral_constant<int, 0>{});
  } else {
    if (live >= L) f(std::integral_constant<int, L>{});
    else call_with_live<L - 1>(live, f);
  }
}

}  // namespace sarathi_hip
