// Grouped expert GEMM for row-major ([E, N, K]) expert weights, both operands through LDS, at
// 128-slot blocks (64- and 256-slot blocks run the four-wave kernel of moe_gemm_wide.hip).
//
// Same computation and argument block as moe_gemm.hip.  That kernel feeds the weights from global
// memory straight into registers, wave by wave: with the packed layout every such load is one
// contiguous KiB, but with row-major weights a lane's 16 bytes come from 32 different rows, 8 KB
// or more apart, and the vector-memory front end becomes the limit.  Here a workgroup of EIGHT
// waves owns BM slots x 256 output columns: two wave rows of BM / 2 slots share each weight
// tile, and four wave columns share each token tile, both through LDS, so a compute unit loads
// 48 KB per 64-deep K-step for 4.2 MFLOP at BM = 128.  Every wave holds a (BM / 2) x 64
// accumulator tile (64 registers at BM = 128).
//
// Data movement: every global -> LDS transfer is a buffer load that writes LDS directly (no
// register staging), issued one K-step ahead into the other half of a double buffer; one barrier
// per K-step.
//   tokens   BM rows x 128 bytes per K-step, 16-byte chunks rotated by row (bank-conflict-free
//            operand reads), exactly as in moe_gemm.hip.
//   weights  a strip's 64 rows x 128 bytes are fetched as whole 128-byte row segments (eight
//            lanes per row: fully coalesced) into the same rotated row layout as the tokens;
//            32 KiB per K-step.
// LDS: 2 x (BM x 128 bytes of tokens + 32 KiB of weights), 96 KiB at BM = 128, requested as dynamic
// shared memory.
#include <atomic>
#include "moe_gemm_common.h"
#include "launch.h"

namespace sarathi_hip {

constexpr int kLdsWaves = 8;          // 2 wave rows x 4 wave columns
constexpr int kLdsWgtUnits = 256 * 8;  // 16-byte units of a weight buffer (256 rows x 128 bytes)
// dynamic shared memory of a workgroup with BM slots: tokens + weights, double buffered
constexpr int lds_bytes(int BM) { return 2 * (BM * 8 + kLdsWgtUnits) * 16; }

// BM = 128 is the block size in use (the kernel body is generic in BM = 64, 128, 256).
template <int DT, int BM, int EPI>
__global__ __launch_bounds__(64 * kLdsWaves) __attribute__((amdgpu_waves_per_eu(2)))
void moe_gemm_lds_kernel(MoeGemmArgs g) {
  constexpr bool MUL_WEIGHT = EPI == kEpiMulWeight;
  constexpr bool GATED = EPI == kEpiGatedSilu;
  constexpr int BN = 256;
  constexpr int MT = BM / 64, NT = 2, SUB = kGemmBK / 16;  // a wave row holds BM / 2 slots
  constexpr int TOK_UNITS = BM * 8;
  constexpr int TOK_PASSES = BM / 64;  // 512 threads move 64 rows of 128 bytes per pass
  extern __shared__ u32x4 lds[];
  u32x4* const tok = lds;                  // [2][BM rows][8 units]
  u32x4* const wgt = lds + 2 * TOK_UNITS;  // [2][256 rows][8 units]

  // ---- which tile (same id -> tile map as the register kernel)
  int pid_m, pid_n;
  if (!tile_of_block(g, blockIdx.x, pid_m, pid_n)) return;
  if (pid_m * BM >= *g.num_tokens_post_padded) return;
  const int expert = g.expert_ids[pid_m];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wn = wave & 3;          // wave column: weight strip of 64 rows
  const int row0 = (wave >> 2) * (BM / 2);  // wave row: first slot of this wave inside the block
  const int l32 = lane & 31, grp = lane >> 5;
  const int half_n = g.N >> 1;      // gated: weight rows [half_n, N) are the up projection

  // first weight row of strip `strip`, tile `nt` of this workgroup (gated: tile 0 holds 32 gate
  // rows, tile 1 the matching up rows), or -1 when the strip lies beyond the matrix
  auto tile_row0 = [&](int strip, int nt) {
    if constexpr (GATED) {
      const int gate0 = pid_n * (BN / 2) + strip * 32;
      return gate0 < half_n ? gate0 + nt * half_n : -1;
    } else {
      const int n0 = pid_n * BN + strip * 64 + nt * 32;
      return n0 < g.N ? n0 : -1;
    }
  };

  // ---- weights: four DMA instructions per wave and K-step
  const int64_t b_bytes = (int64_t)g.N * g.K * 2;
  const rsrc_t rb = make_rsrc(
      reinterpret_cast<const char*>(g.b) + (int64_t)expert * g.b_expert_stride * 2, (uint32_t)b_bytes);
  uint32_t w_off[4];  // global byte offset at k = 0 of the piece this lane moves
  int w_unit[4];      // LDS unit (wave-uniform) at which the instruction's 64 lanes start
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int q = wave * 4 + i;  // 0..31
    // instruction q covers rows [8 (q & 7), +8) of strip q >> 3; lane = (row, position)
    const int strip = q >> 3, rr = (q & 7) * 8 + (lane >> 3);  // row inside the strip, 0..63
    const int r0 = tile_row0(strip, rr >> 5);
    const int n = r0 + (rr & 31);
    const bool in_range = r0 >= 0 && (GATED ? (r0 - (rr >> 5) * half_n) + (rr & 31) < half_n
                                            : n < g.N);
    const int R = strip * 64 + rr;  // row inside the workgroup's weight tile
    const int chunk = lds_chunk_at(R, lane & 7);
    w_off[i] = in_range ? (uint32_t)n * (uint32_t)g.K * 2u + (uint32_t)chunk * 16u : 0x80000000u;
    w_unit[i] = (strip * 64 + (q & 7) * 8) * 8;
  }
  auto dma_weights = [&](int k0, int buf) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
      dma_load16_to_lds(rb, wgt + buf * kLdsWgtUnits + w_unit[i], w_off[i] + (uint32_t)k0 * 2u);
  };

  // ---- tokens: one DMA instruction per wave, pass and K-step (64 rows per pass)
  const rsrc_t ra = make_rsrc(g.a, g.a_bytes);
  uint32_t a_off[TOK_PASSES];
#pragma unroll
  for (int j = 0; j < TOK_PASSES; ++j) {
    const int r = (tid >> 3) + 64 * j;
    const int slot_index = pid_m * BM + r;
    const int sid = slot_index < g.em ? g.sorted_token_ids[slot_index] : g.num_valid;
    const int chunk = lds_chunk_at(r, tid & 7);
    a_off[j] = sid < g.num_valid
                   ? (uint32_t)(sid / g.top_k) * (uint32_t)(g.a_row_stride * 2) + (uint32_t)chunk * 16u
                   : g.a_bytes;
  }
  auto dma_tokens = [&](int k0, int buf) {
#pragma unroll
    for (int j = 0; j < TOK_PASSES; ++j)
      dma_load16_to_lds(ra, tok + buf * TOK_UNITS + (wave * 8 + 64 * j) * 8,
                        a_off[j] + (uint32_t)k0 * 2u);
  };

  f32x16 acc[NT][MT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[nt][mt][i] = 0.f;

  const int steps = g.K / kGemmBK;
  auto wrap = [&](int k) { return k < steps ? k : k - steps; };  // k < 2 * steps
  dma_tokens(0, 0);
  dma_weights(0, 0);
  wait_vmcnt<0>();
  lds_barrier();
  int kstep = wrap(1);  // the K-step whose transfers are in flight
  dma_tokens(kstep * kGemmBK, 1);
  dma_weights(kstep * kGemmBK, 1);
  // Padding sits at the end of an expert's run of slots, so the last block of every expert has
  // 32-slot tiles without a single valid slot.  mt_live is one past the last tile of this wave's
  // rows that holds a valid slot; the loop is compiled once per possible value, each copy
  // branch-free and without the token reads and MFMAs of the tiles beyond it (a wave without any
  // live tile only moves data and meets the others at the barriers).
  int mt_live = 0;
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int slot_index = pid_m * BM + row0 + mt * 32 + l32;
    const int sid = slot_index < g.em ? g.sorted_token_ids[slot_index] : g.num_valid;
    if (__ballot(sid < g.num_valid) != 0ull) mt_live = mt + 1;
  }

  // Branch-free loop: the last two steps fetch wrapped-around K-steps again (never used).
  // The barrier of a step sits before its LAST sub-step, whose operands are already in registers:
  // once every wave is past it, the other buffer has landed and nobody reads this one any more,
  // so the transfers two K-steps ahead start into this buffer and the first operands of the next
  // step are read while the matrix cores still work on this step's last sub-step.
  auto k_loop = [&](auto live_tag) {
    constexpr int LIVE = decltype(live_tag)::value;  // tiles 0 .. LIVE - 1 are computed
    auto read_operands = [&](int buf, int s, u32x4 (&tv)[MT], u32x4 (&wv)[NT]) {
      const u32x4* tb = tok + buf * TOK_UNITS;
      const u32x4* wb = wgt + buf * kLdsWgtUnits;
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        if (mt >= LIVE) continue;
        const int r = row0 + mt * 32 + l32;
        tv[mt] = tb[r * 8 + lds_slot(r, 2 * s + grp)];
      }
      if (LIVE == 0) return;
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) {
        const int R = wn * 64 + nt * 32 + l32;
        wv[nt] = wb[R * 8 + lds_slot(R, 2 * s + grp)];
      }
    };
    u32x4 tv[2][MT], wv[2][NT];
    read_operands(0, 0, tv[0], wv[0]);
    for (int step = 0; step < steps; ++step) {
      const int cur = step & 1;
#pragma unroll
      for (int s = 0; s < SUB; ++s) {
        if (s + 1 < SUB) {
          read_operands(cur, s + 1, tv[(s + 1) & 1], wv[(s + 1) & 1]);
        } else {
          wait_vmcnt<0>();  // the next step's transfers (issued a whole K-step ago) have landed
          lds_barrier();
          kstep = wrap(kstep + 1);
          dma_tokens(kstep * kGemmBK, cur);
          dma_weights(kstep * kGemmBK, cur);
          read_operands(cur ^ 1, 0, tv[0], wv[0]);
        }
        __builtin_amdgcn_sched_barrier(0);  // the reads are in flight under the MFMAs of s
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
          for (int mt = 0; mt < MT; ++mt) {
            if (mt >= LIVE) continue;
            acc[nt][mt] = mfma32<DT>(wv[s & 1][nt], tv[s & 1][mt], acc[nt][mt]);
          }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  };
  call_with_live<MT>(mt_live, k_loop);
  wait_vmcnt<0>();  // nothing may still be writing LDS when the workgroup ends

  // ---- epilogue: lane holds, per accumulator quad, 4 consecutive columns of one token
  const int n_wave0 = GATED ? pid_n * (BN / 2) + wn * 32 : pid_n * BN + wn * 64;
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
          float v[4];
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            v[e] = acc[nt][mt][q * 4 + e];
            if constexpr (MUL_WEIGHT) v[e] *= scale;
          }
          if (n + 3 < g.N) {
            u32x2 out = {pack2<DT>(v[0], v[1]), pack2<DT>(v[2], v[3])};
            *reinterpret_cast<u32x2*>(crow + (int64_t)n * 2) = out;
          } else {
#pragma unroll
            for (int e = 0; e < 4; ++e)
              if (n + e < g.N) store_elem<DT>(crow, n + e, v[e]);
          }
        }
      }
    }
  }
}

template <int DT, int BM, int EPI>
static int launch_one(const MoeGemmArgs& g, dim3 grid, hipStream_t st) {
  auto kernel = moe_gemm_lds_kernel<DT, BM, EPI>;
  constexpr int bytes = lds_bytes(BM);
  // more LDS than the default per-workgroup limit: opt in once per kernel and device
  static std::atomic<bool> raised[64] = {};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return SARATHI_ERR_LAUNCH;
  if (!raised[dev].load(std::memory_order_acquire)) {  // racing first calls both set it: harmless
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                            hipFuncAttributeMaxDynamicSharedMemorySize, bytes) != hipSuccess)
      return SARATHI_ERR_LAUNCH;
    raised[dev].store(true, std::memory_order_release);
  }
  hipLaunchKernelGGL(kernel, grid, dim3(64 * kLdsWaves), bytes, st, g);
  return launch_status();
}

template <int DT, int BM>
static int launch_epilogue(const MoeGemmArgs& g, dim3 grid, int epilogue, hipStream_t st) {
  switch (epilogue) {
    case kEpiMulWeight: return launch_one<DT, BM, kEpiMulWeight>(g, grid, st);
    case kEpiGatedSilu: return launch_one<DT, BM, kEpiGatedSilu>(g, grid, st);
    default: return launch_one<DT, BM, kEpiPlain>(g, grid, st);
  }
}

// Entry used by sarathi_moe_grouped_gemm; block_m is 128.  `g` is complete except
// for n_blocks, which depends on the epilogue.
int launch_moe_gemm_lds(MoeGemmArgs g, int64_t out_cols, int block_m, int epilogue, int dtype,
                        hipStream_t st) {
  const int64_t cols_per_block = epilogue == kEpiGatedSilu ? 128 : 256;
  g.n_blocks = (int32_t)((out_cols + cols_per_block - 1) / cols_per_block);
  const int64_t blocks = (int64_t)((g.n_blocks + 7) / 8) * g.m_blocks * 8;
  if (blocks > 0x7fffffffLL) return SARATHI_ERR_UNSUPPORTED;
  const dim3 grid((unsigned)blocks);
#define SK_PICK(DT) return launch_epilogue<DT, 128>(g, grid, epilogue, st);
  (void)block_m;
  if (dtype == kBF16) { SK_PICK(kBF16) } else { SK_PICK(kF16) }
#undef SK_PICK
}

}  // namespace sarathi_hip
