// Grouped expert GEMM for MoE layers on gfx950 (MFMA).
//
// Counterpart of the reference's Triton `fused_moe_kernel`
// (sarathi/model_executor/layers/fused_moe/fused_moe.py:15-148): for every block of BM
// consecutive slots of sorted_token_ids (all routed to one expert, expert_ids[block]),
//   C[slot, :] = A[slot / top_k, :] @ B[expert]^T   (fp32 accumulation)
// optionally scaled by the slot's routing weight, rounded to the tensor dtype
// and stored at row `slot` of C.  A is [tokens, K], B is [E, N, K] (K
// contiguous), C is [tokens * top_k, N].  Padding slots (id >= num_valid) and
// blocks at or beyond num_tokens_post_padded produce nothing.
//
// Tiling: a workgroup of four waves owns BM slots x 256 output columns; wave w
// owns columns [64 w, 64 w + 64) for all BM slots, as 32x32 MFMA tiles
// (v_mfma_f32_32x32x16 bf16 / f16, 16 deep).  (BM = 256: eight waves, two rows
// of four, 128 slots per row.)  The MFMA "A" operand is fed with
// WEIGHT rows and the "B" operand with TOKEN rows, so a lane ends up holding
// four consecutive output columns of one token per accumulator quad and the
// epilogue writes 8-byte pieces of C rows.
//   weights  never shared between waves: each lane loads its 16-byte operand
//            pieces straight from global memory (buffer loads on the expert's
//            matrix, clipped at N rows) into the register slot that the MFMAs of
//            the current K-step have just consumed, i.e. one K-step (64) ahead
//            of their use, with no second register buffer.  Two layouts of B:
//              row-major [E, N, K] (the reference's): a wave's operand load
//                touches 32 rows x 32 bytes, which makes the texture-address
//                unit, not the MFMA pipe, the limit (~22-36 % of peak); only
//                32-slot blocks take this path, larger ones run the kernel of
//                moe_gemm_wide.hip;
//              packed    [E, N/32, K/16, 64 lanes, 8]: the 1 KiB a wave needs for
//                one 32x16 operand is contiguous in lane order, one fully
//                coalesced load (~1.3-1.9x faster in this kernel).  Weights are static, so
//                packing them once at load time is free.
//   tokens   shared by the four waves: gathered once per K-step into LDS by
//            buffer loads that write LDS directly (BM x 64 elements, 16-byte
//            chunks rotated by row so that the operand reads are bank-conflict
//            free), double buffered, one barrier per K-step.
// Epilogues: plain; times the slot's routing weight (the down projection); or gated SiLU (the
// gate/up projection followed by silu_and_mul, fused_moe.py:499-520): B then holds the gate rows
// [0, N/2) and the up rows [N/2, N), a wave takes 32 gate rows and the 32 matching up rows as
// its two weight tiles, so gate and up of an output element sit in the same lane, and
// C [slots, N/2] = T(T(silu(T(gate))) * T(up)) is written directly: bit-identical to the
// unfused pair of kernels, without the [slots, N] intermediate ever reaching memory.
// 32-slot tiles of a block that hold only padding are skipped.
// Workgroup ids are mapped so that the eight XCDs (id mod 8) each take their
// own column blocks, four of them side by side over all slot blocks: workgroups
// that run together on an XCD share token tiles and the experts' weight tiles
// in that XCD's L2 (tile_of_block).
#include "moe_gemm_common.h"
#include "launch.h"

namespace sarathi_hip {

// A workgroup is four waves side by side, each owning all BM slots x 64 output columns, for
// BM = 32, 64 and 128.  BM = 256 (packed weights only) is eight waves, two rows of four: each row
// owns 128 slots, the token tile in LDS serves all eight, and the second row's weight loads hit
// in the compute unit's L1 behind the first row's.
// At least two waves per SIMD: with 128 accumulator registers per lane (BM = 128) that caps the
// other registers at 128, which the main loop meets anyway; without the bound the epilogues
// that do arithmetic on the accumulators are allocated ~138 and the whole kernel drops to one
// wave per SIMD (measured: 15 % slower).
template <int DT, int BM, int EPI, bool PACKED>
__global__ __launch_bounds__(BM == 256 ? 512 : 256) __attribute__((amdgpu_waves_per_eu(2)))
void moe_gemm_kernel(MoeGemmArgs g) {
  constexpr bool MUL_WEIGHT = EPI == kEpiMulWeight;
  constexpr bool GATED = EPI == kEpiGatedSilu;
  constexpr int WR = BM == 256 ? 2 : 1;  // wave rows
  constexpr int THREADS = 256 * WR;
  constexpr int MT = BM / WR / 32;     // token tiles per wave
  constexpr int NT = kGemmWaveN / 32;  // weight tiles per wave
  constexpr int SUB = kGemmBK / 16;    // MFMA sub-steps per K-step
  constexpr int ROWS_PER_PASS = THREADS / 8;
  constexpr int A_LOADS = BM / ROWS_PER_PASS;  // 16-byte chunks each thread gathers per K-step
  __shared__ u32x4 tok_lds[2][BM * 8];  // [buffer][row * 8 + rotated chunk]

  // ---- which tile
  int pid_m, pid_n;
  if (!tile_of_block(g, blockIdx.x, pid_m, pid_n)) return;
  if (pid_m * BM >= *g.num_tokens_post_padded) return;
  const int expert = g.expert_ids[pid_m];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = (tid >> 6) & 3;  // wave column: output columns [64 wave, 64 wave + 64)
  const int row0 = (tid >> 8) * (BM / WR);  // wave row: first slot of this wave inside the block
  const int l32 = lane & 31, grp = lane >> 5;

  // ---- weights: buffer resource over the expert's matrix; rows >= N read as zero
  // first weight row (= output column) of this wave; gated: first GATE row, 32 per wave
  const int n_wave0 = GATED ? pid_n * (kGemmBN / 2) + wave * (kGemmWaveN / 2)
                            : pid_n * kGemmBN + wave * kGemmWaveN;
  const int half_n = g.N >> 1;  // gated: rows [half_n, N) are the up projection
  const int n_tiles = (g.N + 31) >> 5;
  const int64_t b_bytes = PACKED ? (int64_t)n_tiles * 32 * g.K * 2 : (int64_t)g.N * g.K * 2;
  const rsrc_t rb = make_rsrc(reinterpret_cast<const char*>(g.b) + (int64_t)expert * g.b_expert_stride * 2,
                              (uint32_t)b_bytes);
  uint32_t w_off[NT];  // byte offset of this lane's operand piece at k = 0
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
    // first weight row of tile nt; gated: tile 0 = gate rows, tile 1 = the matching up rows
    const int n_tile0 = GATED ? n_wave0 + nt * half_n : n_wave0 + nt * 32;
    const bool live = GATED ? n_wave0 < half_n : true;
    if constexpr (PACKED) {
      const int tile = n_tile0 >> 5;  // 32-row tile; its K/16 operand blocks of 1 KiB follow each other
      w_off[nt] = live && tile < n_tiles ? (uint32_t)tile * (uint32_t)g.K * 64u + lane * 16u
                                         : 0x80000000u;
    } else {
      const int n = n_tile0 + l32;
      const bool in_range = GATED ? n_wave0 + l32 < half_n : n < g.N;
      w_off[nt] = live && in_range ? (uint32_t)n * (uint32_t)g.K * 2u + grp * 16u : 0x80000000u;
    }
  }
  // operand piece of sub-step s (16 deep) of the K-step starting at k0
  auto load_weight = [&](int nt, int k0, int s) {
    return PACKED ? buf_load16<kCached>(rb, w_off[nt] + (uint32_t)((k0 >> 4) + s) * 1024u)
                  : buf_load16<kCached>(rb, w_off[nt] + (uint32_t)(k0 + s * 16) * 2u);
  };

  // ---- tokens: per K-step each thread moves one 16-byte chunk of rows (tid >> 3) +
  // ROWS_PER_PASS j from global memory straight into LDS (no register staging).
  // A is one buffer resource; padding slots get an offset at its end (every K offset added
  // later keeps them beyond it without wrapping), so their loads deposit zeros without a branch.
  const rsrc_t ra = make_rsrc(g.a, g.a_bytes);
  const int a_chunk = tid & 7;
  uint32_t a_off[A_LOADS];
#pragma unroll
  for (int j = 0; j < A_LOADS; ++j) {
    const int r = (tid >> 3) + ROWS_PER_PASS * j;
    const int slot_index = pid_m * BM + r;
    const int sid = slot_index < g.em ? g.sorted_token_ids[slot_index] : g.num_valid;
    a_off[j] = sid < g.num_valid
                   ? (uint32_t)(sid / g.top_k) * (uint32_t)(g.a_row_stride * 2) +
                         (uint32_t)lds_chunk_at(r, a_chunk) * 16u
                   : g.a_bytes;
  }
  // LDS DMA: lane l of a wave deposits its 16 bytes at (wave-uniform base) + 16 l, i.e. at
  // position l & 7 of row base_row + l / 8; the lane therefore fetches the chunk that the rotated
  // layout keeps at that position (the inverse of lds_slot, folded into a_off above).
  auto gather_to_lds = [&](int k0, int buf) {
#pragma unroll
    for (int j = 0; j < A_LOADS; ++j) {
      const int base_row = (tid >> 6) * 8 + ROWS_PER_PASS * j;
      dma_load16_to_lds(ra, &tok_lds[buf][base_row * 8], a_off[j] + (uint32_t)k0 * 2u);
    }
  };
  f32x16 acc[NT][MT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[nt][mt][i] = 0.f;

  // Note: the workgroups that share a weight tile (the slot blocks of one expert, side by side
  // on one XCD) deliberately walk K in lockstep from 0.  Rotating their starting offsets was
  // measured and is ~1.8x slower: the tile then has to stay in the 4 MB L2 for the whole loop
  // instead of for one step.
  const int steps = g.K / kGemmBK;
  int kstep = 0;
  u32x4 w[NT][SUB];
  gather_to_lds(kstep * kGemmBK, 0);
#pragma unroll
  for (int nt = 0; nt < NT; ++nt)
#pragma unroll
    for (int s = 0; s < SUB; ++s) w[nt][s] = load_weight(nt, kstep * kGemmBK, s);
  __syncthreads();

  // (Meeting the other waves one sub-step earlier, so that the next K-step's first operand read
  // is already in flight under this K-step's last MFMAs, was measured and is 1-4 % slower.)
  // The loop body is branch-free so that the scheduler can keep loads, LDS reads and MFMAs
  // interleaved: the last step simply loads the wrapped-around "next" K-step again (issued,
  // never used), and the token operands of sub-step s + 1 are read from LDS before the MFMAs
  // of sub-step s are issued.
  // Padding sits at the end of an expert's run of slots, so the last block of every expert has
  // 32-slot tiles without a single valid slot (half a block per expert on average).  mt_live is
  // one past the last tile of this block that holds a valid slot; the loop is compiled once per
  // possible value, each copy branch-free and without the LDS reads and MFMAs of the tiles
  // beyond it.
  int mt_live = 0;
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int slot_index = pid_m * BM + row0 + mt * 32 + l32;
    const int sid = slot_index < g.em ? g.sorted_token_ids[slot_index] : g.num_valid;
    if (__ballot(sid < g.num_valid) != 0ull) mt_live = mt + 1;
  }
  auto k_loop = [&](auto live_tag) {
    constexpr int LIVE = decltype(live_tag)::value;  // tiles 0 .. LIVE - 1 are computed
    auto read_live_tokens = [&](int buf, int s, u32x4 (&tokv)[MT]) {
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        if (mt >= LIVE) continue;
        const int r = row0 + mt * 32 + l32;
        tokv[mt] = tok_lds[buf][r * 8 + lds_slot(r, 2 * s + grp)];
      }
    };
    for (int step = 0; step < steps; ++step) {
      const int cur = step & 1;
      kstep = kstep + 1 < steps ? kstep + 1 : 0;
      const int k_next = kstep * kGemmBK;
      gather_to_lds(k_next, cur ^ 1);
      u32x4 tokv[2][MT];
      read_live_tokens(cur, 0, tokv[0]);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int s = 0; s < SUB; ++s) {
        if (s + 1 < SUB) read_live_tokens(cur, s + 1, tokv[(s + 1) & 1]);
        __builtin_amdgcn_sched_barrier(0);  // LDS reads of s + 1 are in flight under the MFMAs of s
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
#pragma unroll
          for (int mt = 0; mt < MT; ++mt) {
            if (mt >= LIVE) continue;
            acc[nt][mt] = mfma32<DT>(w[nt][s], tokv[s & 1][mt], acc[nt][mt]);
          }
          w[nt][s] = load_weight(nt, k_next, s);  // the slot is free again: refill it
        }
        // keep this sub-step's loads here (a full K-step ahead of their use) and the LDS reads
        // of the next sub-step ahead of its MFMAs
        __builtin_amdgcn_sched_barrier(0);
      }
      // the DMA of this step is older than the NT * SUB weight loads issued since.  A wave
      // without live tiles (eight-wave variant: a wave row that is all padding) has no use for
      // its weight loads, so the compiler drops them: it must wait for everything, or its share
      // of the token gather could still be in flight when the others pass the barrier.
      wait_vmcnt<LIVE == 0 ? 0 : NT * SUB>();
      lds_barrier();
    }
  };
  call_with_live<MT>(mt_live, k_loop);

  // ---- epilogue: lane holds, per accumulator quad, 4 consecutive columns of one token
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int slot_index = pid_m * BM + row0 + mt * 32 + l32;
    const int sid = slot_index < g.em ? g.sorted_token_ids[slot_index] : g.num_valid;
    if (sid >= g.num_valid) continue;
    float scale = 1.f;
    if constexpr (MUL_WEIGHT) scale = g.topk_weights[sid];
    char* crow = reinterpret_cast<char*>(g.c) + (int64_t)sid * g.c_row_stride * 2;
    if constexpr (GATED) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int n = n_wave0 + q * 8 + grp * 4;
        float v[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const float x = rnd<DT>(acc[0][mt][q * 4 + e]), y = rnd<DT>(acc[1][mt][q * 4 + e]);
          v[e] = rnd<DT>(silu_f32(x)) * y;
        }
        if (n + 3 < half_n) {
          u32x2 out = {pack2<DT>(v[0], v[1]), pack2<DT>(v[2], v[3])};
          *reinterpret_cast<u32x2*>(crow + (int64_t)n * 2) = out;
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (n + e < half_n) store_elem<DT>(crow, n + e, v[e]);
        }
      }
    } else {
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int n = n_wave0 + nt * 32 + q * 8 + grp * 4;
          float v0 = acc[nt][mt][q * 4 + 0], v1 = acc[nt][mt][q * 4 + 1];
          float v2 = acc[nt][mt][q * 4 + 2], v3 = acc[nt][mt][q * 4 + 3];
          if constexpr (MUL_WEIGHT) { v0 *= scale; v1 *= scale; v2 *= scale; v3 *= scale; }
          if (n + 3 < g.N) {
            u32x2 out = {pack2<DT>(v0, v1), pack2<DT>(v2, v3)};
            *reinterpret_cast<u32x2*>(crow + (int64_t)n * 2) = out;
          } else {
            const float v[4] = {v0, v1, v2, v3};
#pragma unroll
            for (int e = 0; e < 4; ++e)
              if (n + e < g.N) store_elem<DT>(crow, n + e, v[e]);
          }
        }
      }
    }
  }
}

template <int DT, int BM>
static int launch_moe_gemm(const MoeGemmArgs& g, int epilogue, bool packed, hipStream_t st) {
  const int64_t groups = (g.n_blocks + 7) / 8;
  const int64_t blocks = groups * g.m_blocks * 8;
  if (blocks > 0x7fffffffLL) return SARATHI_ERR_UNSUPPORTED;
  const dim3 grid((unsigned)blocks), block(BM == 256 ? 512 : 256);
#define SK_LAUNCH(EP, PK) \
  hipLaunchKernelGGL((moe_gemm_kernel<DT, BM, EP, PK>), grid, block, 0, st, g)
  if constexpr (BM == 256) {  // eight waves: packed weights only
    if (epilogue == kEpiMulWeight) SK_LAUNCH(kEpiMulWeight, true);
    else if (epilogue == kEpiGatedSilu) SK_LAUNCH(kEpiGatedSilu, true);
    else SK_LAUNCH(kEpiPlain, true);
  } else
  if (epilogue == kEpiMulWeight) {
    if (packed) SK_LAUNCH(kEpiMulWeight, true); else SK_LAUNCH(kEpiMulWeight, false);
  } else if (epilogue == kEpiGatedSilu) {
    if (packed) SK_LAUNCH(kEpiGatedSilu, true); else SK_LAUNCH(kEpiGatedSilu, false);
  } else {
    if (packed) SK_LAUNCH(kEpiPlain, true); else SK_LAUNCH(kEpiPlain, false);
  }
#undef SK_LAUNCH
  return launch_status();
}

// moe_gemm_wide.hip: row-major weights at 64-, 128- and 256-slot blocks, four waves
int launch_moe_gemm_wide(MoeGemmArgs g, int64_t out_cols, int block_m, int epilogue, int dtype,
                         hipStream_t st);
bool moe_gemm_wide_takes_narrow_blocks(int64_t out_cols, int m_blocks, int block_m, int epilogue);
// moe_gemm_rider.hip: row-major weights at 256-slot blocks, with riders
int launch_moe_gemm_rider(MoeGemmArgs g, int64_t out_cols, int epilogue, int dtype,
                         const int32_t* ride, hipStream_t st);
// moe_gemm_f32.hip: float32 tensors
int launch_moe_gemm_f32(const void* a, const void* b, void* c, const float* topk_weights,
                        const int32_t* sorted_token_ids, const int32_t* expert_ids,
                        const int32_t* num_tokens_post_padded, int64_t num_valid_tokens,
                        int64_t sorted_len, int64_t n, int64_t k, int64_t a_row_stride,
                        int64_t b_expert_stride, int64_t c_row_stride, int block_m, int top_k,
                        int epilogue, int b_layout, hipStream_t st);

}  // namespace sarathi_hip

// Ranges of a slot block that separate waves sweep: the four-wave kernel for row-major weights has
// two wave rows at every block size, the kernel of this file only in its eight-wave form.
extern "C" int sarathi_moe_gemm_slot_rows(int block_m, int b_layout) {
  if (b_layout != SARATHI_MOE_B_ROW_MAJOR && b_layout != SARATHI_MOE_B_PACKED)
    return SARATHI_ERR_INVALID_ARG;
  if (block_m != 32 && block_m != 64 && block_m != 128 && block_m != 256)
    return SARATHI_ERR_UNSUPPORTED;
  if (b_layout == SARATHI_MOE_B_ROW_MAJOR) return block_m >= 64 ? 2 : 1;
  return block_m == 256 ? 2 : 1;
}

namespace sarathi_hip {
static int grouped_gemm(const void* a, const void* b, void* c, const float* topk_weights,
                        const int32_t* sorted_token_ids, const int32_t* expert_ids,
                        const int32_t* num_tokens_post_padded, int64_t num_valid_tokens,
                        int64_t sorted_len, int64_t n, int64_t k, int64_t a_row_stride,
                        int64_t b_expert_stride, int64_t c_row_stride, int block_m, int top_k,
                        int epilogue, int b_layout, int dtype, const int32_t* ride, void* stream) {
  if (!a || !b || !c || !sorted_token_ids || !expert_ids || !num_tokens_post_padded)
    return SARATHI_ERR_INVALID_ARG;
  if (epilogue != SARATHI_MOE_EPILOGUE_NONE && epilogue != SARATHI_MOE_EPILOGUE_ROUTED_WEIGHT &&
      epilogue != SARATHI_MOE_EPILOGUE_SILU_AND_MUL)
    return SARATHI_ERR_INVALID_ARG;
  if (epilogue == SARATHI_MOE_EPILOGUE_ROUTED_WEIGHT && !topk_weights)
    return SARATHI_ERR_INVALID_ARG;
  const bool gated = epilogue == SARATHI_MOE_EPILOGUE_SILU_AND_MUL;
  if (gated && (n & 1)) return SARATHI_ERR_INVALID_ARG;
  const int64_t c_cols = gated ? n / 2 : n;  // width of C
  if (num_valid_tokens < 0 || sorted_len < 0 || n <= 0 || k <= 0 || top_k <= 0 ||
      a_row_stride < k || c_row_stride < c_cols || b_expert_stride < n * k ||
      (b_layout != SARATHI_MOE_B_ROW_MAJOR && b_layout != SARATHI_MOE_B_PACKED))
    return SARATHI_ERR_INVALID_ARG;
  const bool packed = b_layout == SARATHI_MOE_B_PACKED;
  if (packed && b_expert_stride < (n + 31) / 32 * 32 * k) return SARATHI_ERR_INVALID_ARG;
  // riders exist in one kernel only: row-major 16-bit weights at 256-slot blocks
  if (ride && (packed || block_m != 256 || (dtype != kBF16 && dtype != kF16)))
    return SARATHI_ERR_UNSUPPORTED;
  if (dtype == kF32)
    return launch_moe_gemm_f32(a, b, c, topk_weights, sorted_token_ids, expert_ids,
                               num_tokens_post_padded, num_valid_tokens, sorted_len, n, k,
                               a_row_stride, b_expert_stride, c_row_stride, block_m, top_k,
                               epilogue, b_layout, (hipStream_t)stream);
  if (block_m != 32 && block_m != 64 && block_m != 128 && block_m != 256)
    return SARATHI_ERR_UNSUPPORTED;
  if (dtype != kBF16 && dtype != kF16) return SARATHI_ERR_UNSUPPORTED;
  // 16-byte operand pieces and whole K-steps; one buffer resource per expert matrix
  if (k % kGemmBK != 0 || a_row_stride % 8 != 0 || b_expert_stride % 8 != 0 || n % 4 != 0 ||
      c_row_stride % 4 != 0 || !aligned16(a) || !aligned16(b) || (reinterpret_cast<uintptr_t>(c) & 7u))
    return SARATHI_ERR_UNSUPPORTED;
  // gated: output pieces of 4 columns; packed tiles of 32 rows must not straddle gate and up
  if (gated && (c_cols % 4 != 0 || (packed && c_cols % 32 != 0))) return SARATHI_ERR_UNSUPPORTED;
  if ((n + 31) / 32 * 32 * k * 2 >= 0x80000000LL || num_valid_tokens > 0x7fffffffLL || sorted_len > 0x7fffffffLL)
    return SARATHI_ERR_UNSUPPORTED;
  // A is addressed through one buffer resource with 32-bit offsets
  const int64_t a_rows = (num_valid_tokens + top_k - 1) / top_k;
  const int64_t a_extent = ((a_rows > 0 ? a_rows - 1 : 0) * a_row_stride + k) * 2;
  if (a_extent + 2 * k >= 0x100000000LL) return SARATHI_ERR_UNSUPPORTED;
  if (sorted_len == 0 || num_valid_tokens == 0) return SARATHI_OK;
  MoeGemmArgs g;
  g.a = a; g.b = b; g.c = c;
  g.topk_weights = topk_weights;
  g.sorted_token_ids = sorted_token_ids;
  g.expert_ids = expert_ids;
  g.num_tokens_post_padded = num_tokens_post_padded;
  g.a_bytes = (uint32_t)a_extent;
  g.a_row_stride = a_row_stride;
  g.b_expert_stride = b_expert_stride;
  g.c_row_stride = c_row_stride;
  g.num_valid = (int32_t)num_valid_tokens;
  g.em = (int32_t)sorted_len;
  g.N = (int32_t)n; g.K = (int32_t)k;
  g.top_k = top_k;
  g.m_blocks = (int32_t)((sorted_len + block_m - 1) / block_m);
  g.n_blocks = gated ? (int32_t)((c_cols + kGemmBN / 2 - 1) / (kGemmBN / 2))
                     : (int32_t)((n + kGemmBN - 1) / kGemmBN);
  g.group_n = kGemmGroupN;
  hipStream_t st = (hipStream_t)stream;
  const int mw = epilogue;
  // row-major weights run the four-wave kernel of moe_gemm_wide.hip from 64-slot blocks on (32-slot
  // wave tiles for decode-size batches, 128 x 128 wave tiles at 256-slot blocks)
  // riders are an optimisation (the plain kernels compute every block themselves): a launch so
  // small that the plain kernel would take 128-wide column blocks to fill the chip keeps those
  if (ride && !moe_gemm_wide_takes_narrow_blocks(c_cols, g.m_blocks, block_m, mw))
    return launch_moe_gemm_rider(g, c_cols, mw, dtype, ride, st);
  if (!packed && block_m >= 64) return launch_moe_gemm_wide(g, c_cols, block_m, mw, dtype, st);
#define SK_GEMM(DT)                                                       \
  switch (block_m) {                                                      \
    case 32: return launch_moe_gemm<DT, 32>(g, mw, packed, st);           \
    case 64: return launch_moe_gemm<DT, 64>(g, mw, packed, st);           \
    case 256: return launch_moe_gemm<DT, 256>(g, mw, packed, st);         \
    default: return launch_moe_gemm<DT, 128>(g, mw, packed, st);          \
  }
  if (dtype == kBF16) { SK_GEMM(kBF16) } else { SK_GEMM(kF16) }
#undef SK_GEMM
}
}  // namespace sarathi_hip

extern "C" int sarathi_moe_grouped_gemm(const void* a, const void* b, void* c,
                                        const float* topk_weights,
                                        const int32_t* sorted_token_ids,
                                        const int32_t* expert_ids,
                                        const int32_t* num_tokens_post_padded,
                                        int64_t num_valid_tokens, int64_t sorted_len, int64_t n,
                                        int64_t k, int64_t a_row_stride, int64_t b_expert_stride,
                                        int64_t c_row_stride, int block_m, int top_k,
                                        int epilogue, int b_layout, int dtype,
                                        void* stream) {
  return sarathi_hip::grouped_gemm(a, b, c, topk_weights, sorted_token_ids, expert_ids,
                                   num_tokens_post_padded, num_valid_tokens, sorted_len, n, k,
                                   a_row_stride, b_expert_stride, c_row_stride, block_m, top_k,
                                   epilogue, b_layout, dtype, nullptr, stream);
}

extern "C" int sarathi_moe_grouped_gemm_riders(
    const void* a, const void* b, void* c, const float* topk_weights,
    const int32_t* sorted_token_ids, const int32_t* expert_ids,
    const int32_t* num_tokens_post_padded, int64_t num_valid_tokens, int64_t sorted_len, int64_t n,
    int64_t k, int64_t a_row_stride, int64_t b_expert_stride, int64_t c_row_stride, int block_m,
    int top_k, int epilogue, int b_layout, int dtype, const int32_t* riders, void* stream) {
  if (!riders) return SARATHI_ERR_INVALID_ARG;
  return sarathi_hip::grouped_gemm(a, b, c, topk_weights, sorted_token_ids, expert_ids,
                                   num_tokens_post_padded, num_valid_tokens, sorted_len, n, k,
                                   a_row_stride, b_expert_stride, c_row_stride, block_m, top_k,
                                   epilogue, b_layout, dtype, riders, stream);
}
