// Grouped expert GEMM for row-major ([E, N, K]) expert weights: four waves, one per SIMD at
// 256-slot blocks, each owning a 128 x 128 accumulator tile (smaller tiles at 64- and 128-slot
// blocks).
//
// Same computation and argument block as moe_gemm.hip.  That kernel feeds the weights from global
// memory straight into registers, wave by wave: with the packed layout every such load is one
// contiguous KiB, but with row-major weights a lane's 16 bytes come from 32 different rows, 8 KB
// or more apart.  Here both operands are shared through LDS and fetched as whole 128-byte row
// segments (eight lanes per row).  An earlier kernel moved them global -> LDS with buffer loads
// that write LDS directly, eight waves per workgroup; such a transfer can only be issued once
// every wave has finished reading the buffer it overwrites, so all 64 of a K-step's transfers
// left in one burst behind the barrier, the vector-memory front end backed up, and the MFMAs
// queued behind them waited (removing the transfers from that loop: +28 %; feeding them
// cache-resident data instead: only +9 %).  Here the operands pass through registers: a thread's
// 16 global loads of K-step i + 2 are spread over K-step i, stay in registers for one K-step, and
// are stored to LDS during K-step i + 1 (see the loop): loads and LDS stores trickle out between
// the MFMAs instead of piling up behind a barrier.  That takes 64 registers on top of 256
// accumulators and 64 of operand fragments, hence one wave per SIMD with the full 512-entry
// register file, and a 128 x 128 wave tile, which also needs a third fewer LDS bytes per flop
// than 128 x 64.
//
// LDS: two buffers of (BM token rows + BN weight rows) x 128 bytes, the 16-byte chunks of a row
// rotated as in moe_gemm.hip (bank-conflict-free operand reads); 128 KiB at BM = BN = 256,
// requested as dynamic shared memory.
#include <atomic>
#include "moe_gemm_common.h"
#include "launch.h"

namespace sarathi_hip {

// dynamic shared memory: BM token rows + BN weight rows of 128 bytes, double buffered
constexpr int wide_lds_bytes(int BM, int BN) { return 2 * (BM * 8 + BN * 8) * 16; }

// BN = 256 is the shape described above.  BN = 128 (wave tiles of 128 x 64) exists for launches
// that would otherwise have too few workgroups to keep every compute unit streaming weights:
// the down projection of a decode-size batch is 8 experts x 16 column blocks of 256.
// BM = 64 (wave tiles of 32 slots x BN / 2 columns, 64 or 32 accumulator registers, 48-80 KiB of
// LDS) is the same loop for decode-size batches: two or three workgroups share a compute unit, so
// that more weight bytes are in flight while nearly all the time goes into streaming them.
// BM = 128 (64-slot wave tiles) completes the set of block sizes.
template <int DT, int EPI, int BN, int BM>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, BM == 256 ? 1 : BM == 128 ? 2 : 4)))
void moe_gemm_wide_kernel(MoeGemmArgs g) {
  constexpr bool MUL_WEIGHT = EPI == kEpiMulWeight;
  constexpr bool GATED = EPI == kEpiGatedSilu;
  constexpr int MT = BM / 64, NT = BN / 64, SUB = kGemmBK / 16;
  constexpr int WCR = BN / 2;      // weight rows of a wave column
  constexpr int ROWS = 8;          // rows of an operand a thread moves per K-step, at most
  constexpr int T_ROWS = BM / 32;  // token rows a thread moves per K-step
  constexpr int W_ROWS = BN / 32;  // weight rows a thread moves per K-step
  constexpr int kTokUnits = BM * 8, kWgtUnits = BN * 8;
  extern __shared__ u32x4 lds[];
  u32x4* const tok = lds;                  // [2][BM rows][8 units]
  u32x4* const wgt = lds + 2 * kTokUnits;  // [2][BN rows][8 units]

  int pid_m, pid_n;
  if (!tile_of_block(g, blockIdx.x, pid_m, pid_n)) return;
  if (pid_m * BM >= *g.num_tokens_post_padded) return;
  const int expert = g.expert_ids[pid_m];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wc = wave & 1;                 // wave column: BN / 2 weight rows
  const int row0 = (wave >> 1) * (BM / 2);  // wave row: first slot of this wave inside the block
  const int l32 = lane & 31, grp = lane >> 5;
  const int half_n = g.N >> 1;  // gated: weight rows [half_n, N) are the up projection

  // Row R of the workgroup's weight tile -> row of the expert's matrix, or -1 beyond it.  Gated:
  // the first half of a wave column's tiles are gate rows and the second half the matching up
  // rows, so gate and up of an output element end up in the same lane.
  auto weight_row = [&](int R) {
    if constexpr (GATED) {
      const int in_col = R % WCR;  // row inside the wave column
      const int gate = pid_n * (BN / 2) + (R / WCR) * (WCR / 2) + in_col % (WCR / 2);
      return gate < half_n ? gate + (in_col / (WCR / 2)) * half_n : -1;
    } else {
      const int n = pid_n * BN + R;
      return n < g.N ? n : -1;
    }
  };

  // ---- global -> register -> LDS: thread t moves position t & 7 of rows (t >> 3) + 32 j
  const rsrc_t ra = make_rsrc(g.a, g.a_bytes);
  const rsrc_t rb = make_rsrc(reinterpret_cast<const char*>(g.b) + (int64_t)expert * g.b_expert_stride * 2,
                              (uint32_t)((int64_t)g.N * g.K * 2));
  const int pos = tid & 7;
  uint32_t a_off[T_ROWS], w_off[W_ROWS];
#pragma unroll
  for (int j = 0; j < ROWS; ++j) {
    const int r = (tid >> 3) + 32 * j;
    const uint32_t chunk = (uint32_t)lds_chunk_at(r, pos) * 16u;
    if (j < T_ROWS) {
      const int slot_index = pid_m * BM + r;
      const int sid = slot_index < g.em ? g.sorted_token_ids[slot_index] : g.num_valid;
      // a padding slot reads beyond the end of A, i.e. zeros, whatever K offset is added
      a_off[j] = sid < g.num_valid ? (uint32_t)(sid / g.top_k) * (uint32_t)(g.a_row_stride * 2) + chunk
                                   : g.a_bytes;
    }
    if (j < W_ROWS) {
      const int n = weight_row(r);
      w_off[j] = n >= 0 ? (uint32_t)n * (uint32_t)g.K * 2u + chunk : 0x80000000u;
    }
  }
  // one K-step of operands on its way from global memory to LDS; row j of both operands (as
  // far as each has a row j) moves together
  u32x4 st_tok[T_ROWS], st_wgt[W_ROWS];
  auto load_rows = [&](int k0, int j0, int j1) {
#pragma unroll
    for (int j = j0; j < j1; ++j) {
      if (j < T_ROWS) st_tok[j] = buf_load16<kCached>(ra, a_off[j] + (uint32_t)k0 * 2u);
      if (j < W_ROWS) st_wgt[j] = buf_load16<kCached>(rb, w_off[j] + (uint32_t)k0 * 2u);
    }
  };
  auto store_rows = [&](int buf, int j0, int j1) {
#pragma unroll
    for (int j = j0; j < j1; ++j) {
      const int unit = ((tid >> 3) + 32 * j) * 8 + pos;
      if (j < T_ROWS) tok[buf * kTokUnits + unit] = st_tok[j];
      if (j < W_ROWS) wgt[buf * kWgtUnits + unit] = st_wgt[j];
    }
  };

  f32x16 acc[NT][MT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[nt][mt][i] = 0.f;

  // tiles of 32 slots without a valid slot are skipped (see moe_gemm.hip)
  int mt_live = 0;
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int slot_index = pid_m * BM + row0 + mt * 32 + l32;
    const int sid = slot_index < g.em ? g.sorted_token_ids[slot_index] : g.num_valid;
    if (__ballot(sid < g.num_valid) != 0ull) mt_live = mt + 1;
  }

  const int steps = g.K / kGemmBK;
  auto wrap = [&](int k) { return k < steps ? k : k - steps; };  // k < 2 * steps
  // K-step j is read from LDS buffer j & 1
  load_rows(0, 0, ROWS);
  store_rows(0, 0, ROWS);
  load_rows(wrap(1) * kGemmBK, 0, ROWS);
  lds_barrier();

  // During K-step i (LDS buffer i & 1 is read), row by row of a thread's share:
  //   sub-steps 0..2  store the registers, which hold K-step i + 1 since they were loaded during
  //                   K-step i - 1, to the other LDS buffer, which nobody reads since the last
  //                   barrier, and load K-step i + 2 into them (the last loads in sub-step 3);
  //   before sub-step 3  barrier: the stores above are visible and every wave has read all it
  //                   needs of this buffer (sub-step 3's operands are in registers already), so
  //                   the first operands of K-step i + 1 are read under sub-step 3's MFMAs.
  // Branch-free: the last two K-steps load and store wrapped-around data that is never used.
  auto k_loop = [&](auto live_tag) {
    constexpr int LIVE = decltype(live_tag)::value;  // token tiles 0 .. LIVE - 1 are computed
    auto read_operands = [&](int buf, int s, u32x4 (&tv)[MT], u32x4 (&wv)[NT]) {
      const u32x4* tb = tok + buf * kTokUnits;
      const u32x4* wb = wgt + buf * kWgtUnits;
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        if (mt >= LIVE) continue;
        const int r = row0 + mt * 32 + l32;
        tv[mt] = tb[r * 8 + lds_slot(r, 2 * s + grp)];
      }
      if (LIVE == 0) return;
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) {
        const int R = wc * WCR + nt * 32 + l32;
        wv[nt] = wb[R * 8 + lds_slot(R, 2 * s + grp)];
      }
    };
    u32x4 tv[2][MT], wv[2][NT];
    read_operands(0, 0, tv[0], wv[0]);
    auto sub_step = [&](auto s_tag, int cur, int k_load) {
      constexpr int s = decltype(s_tag)::value;
      constexpr int ST0 = s * 3, ST1 = s * 3 + 3 < ROWS ? s * 3 + 3 : ROWS;  // rows stored here
      if constexpr (s + 1 < SUB) {
        read_operands(cur, s + 1, tv[(s + 1) & 1], wv[(s + 1) & 1]);
        store_rows(cur ^ 1, ST0, ST1);
      } else {
        lds_barrier();
        read_operands(cur ^ 1, 0, tv[0], wv[0]);
      }
      // rows 0-1, 2-3, 4-5, 6-7: each after its store (rows 0-2, 3-5, 6-7).  (Loading every row
      // right after its store, for a full K-step between load and store, crowds the first two
      // sub-steps with memory instructions and measured 2.5 % slower.)
      load_rows(k_load, s * 2, s * 2 + 2);
      if constexpr (LIVE == 0) __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
          if (mt >= LIVE) continue;
          acc[nt][mt] = mfma32<DT>(wv[s & 1][nt], tv[s & 1][mt], acc[nt][mt]);
        }
      if constexpr (LIVE == MT && BN == 256 && BM == 256) {
        // One wave per SIMD: nothing else runs while this wave issues memory instructions, so
        // they go out one at a time in the shadow of the MFMAs (each MFMA keeps the matrix
        // core busy for 32 cycles): 8 LDS reads, the LDS stores, then the global loads.  (Measured
        // against: the compiler's own order, 7 % slower; stores and loads ahead of the reads,
        // 4 % slower; reads two per MFMA, equal.)
        constexpr int kMfma = 0x008, kVmemRead = 0x020, kDsRead = 0x100, kDsWrite = 0x200;
        constexpr int WRITES = s + 1 < SUB ? 2 * (ST1 - ST0) : 0;
#pragma unroll
        for (int i = 0; i < MT + NT; ++i) {
          __builtin_amdgcn_sched_group_barrier(kMfma, 1, 0);
          __builtin_amdgcn_sched_group_barrier(kDsRead, 1, 0);
        }
#pragma unroll
        for (int i = 0; i < WRITES; ++i) {
          __builtin_amdgcn_sched_group_barrier(kMfma, 1, 0);
          __builtin_amdgcn_sched_group_barrier(kDsWrite, 1, 0);
        }
        // the four global loads over the MFMAs that are left (2, 2, 4, 8)
        constexpr int LEFT = MT * NT - (MT + NT) - WRITES;
        constexpr int PER = LEFT >= 4 ? 1 : 2;
#pragma unroll
        for (int i = 0; i < 4 / PER; ++i) {
          __builtin_amdgcn_sched_group_barrier(kMfma, 1, 0);
          __builtin_amdgcn_sched_group_barrier(kVmemRead, PER, 0);
        }
      } else if constexpr (LIVE > 0) {
        // partly filled blocks, narrow column blocks: the same idea with fewer MFMAs to hide
        // behind (several memory instructions per MFMA)
        constexpr int kMfma = 0x008, kMemory = 0x020 | 0x100 | 0x200;
        constexpr auto rows_in = [](int j0, int j1, int n) {  // rows j0 <= j < j1 that are below n
          return (j1 < n ? j1 : n) - (j0 < n ? j0 : n);
        };
        constexpr int STORES = s + 1 < SUB ? rows_in(ST0, ST1, T_ROWS) + rows_in(ST0, ST1, W_ROWS) : 0;
        constexpr int LOADS = rows_in(s * 2, s * 2 + 2, T_ROWS) + rows_in(s * 2, s * 2 + 2, W_ROWS);
        constexpr int OPS = LIVE + NT + STORES + LOADS;
        constexpr int PER = (OPS + NT * LIVE - 1) / (NT * LIVE);
#pragma unroll
        for (int i = 0; i < NT * LIVE; ++i) {
          __builtin_amdgcn_sched_group_barrier(kMfma, 1, 0);
          __builtin_amdgcn_sched_group_barrier(kMemory, PER, 0);
        }
      }
      __builtin_amdgcn_sched_barrier(0);
    };
    for (int step = 0; step < steps; ++step) {
      const int cur = step & 1;
      const int k_load = wrap(wrap(step + 1) + 1) * kGemmBK;  // K-step step + 2
      sub_step(std::integral_constant<int, 0>{}, cur, k_load);
      sub_step(std::integral_constant<int, 1>{}, cur, k_load);
      sub_step(std::integral_constant<int, 2>{}, cur, k_load);
      sub_step(std::integral_constant<int, 3>{}, cur, k_load);
    }
  };
  call_with_live<MT>(mt_live, k_loop);

  // ---- epilogue: lane holds, per accumulator quad, 4 consecutive columns of one token
  const int n_wave0 = GATED ? pid_n * (BN / 2) + wc * (WCR / 2) : pid_n * BN + wc * WCR;
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int slot_index = pid_m * BM + row0 + mt * 32 + l32;
    const int sid = slot_index < g.em ? g.sorted_token_ids[slot_index] : g.num_valid;
    if (sid >= g.num_valid) continue;
    float scale = 1.f;
    if constexpr (MUL_WEIGHT) scale = g.topk_weights[sid];
    char* crow = reinterpret_cast<char*>(g.c) + (int64_t)sid * g.c_row_stride * 2;
    constexpr int OUT_TILES = GATED ? NT / 2 : NT;
#pragma unroll
    for (int nt = 0; nt < OUT_TILES; ++nt) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int n = n_wave0 + nt * 32 + q * 8 + grp * 4;
        const int n_end = GATED ? half_n : g.N;
        float v[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          if constexpr (GATED) {
            const float x = rnd<DT>(acc[nt][mt][q * 4 + e]), y = rnd<DT>(acc[nt + NT / 2][mt][q * 4 + e]);
            v[e] = rnd<DT>(silu_f32(x)) * y;
          } else {
            v[e] = acc[nt][mt][q * 4 + e];
            if constexpr (MUL_WEIGHT) v[e] *= scale;
          }
        }
        if (n + 3 < n_end) {
          u32x2 out = {pack2<DT>(v[0], v[1]), pack2<DT>(v[2], v[3])};
          *reinterpret_cast<u32x2*>(crow + (int64_t)n * 2) = out;
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (n + e < n_end) store_elem<DT>(crow, n + e, v[e]);
        }
      }
    }
  }
}

template <int DT, int EPI, int BN, int BM>
static int launch_wide(const MoeGemmArgs& g, dim3 grid, hipStream_t st) {
  auto kernel = moe_gemm_wide_kernel<DT, EPI, BN, BM>;
  constexpr int bytes = wide_lds_bytes(BM, BN);
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
  hipLaunchKernelGGL(kernel, grid, dim3(256), bytes, st, g);
  return launch_status();
}

template <int DT, int BN, int BM>
static int launch_wide_epilogue(MoeGemmArgs g, int64_t out_cols, int epilogue, hipStream_t st) {
  const int64_t cols_per_block = epilogue == kEpiGatedSilu ? BN / 2 : BN;
  g.n_blocks = (int32_t)((out_cols + cols_per_block - 1) / cols_per_block);
  const int64_t blocks = (int64_t)((g.n_blocks + 7) / 8) * g.m_blocks * 8;
  if (blocks > 0x7fffffffLL) return SARATHI_ERR_UNSUPPORTED;
  const dim3 grid((unsigned)blocks);
  switch (epilogue) {
    case kEpiMulWeight: return launch_wide<DT, kEpiMulWeight, BN, BM>(g, grid, st);
    case kEpiGatedSilu: return launch_wide<DT, kEpiGatedSilu, BN, BM>(g, grid, st);
    default: return launch_wide<DT, kEpiPlain, BN, BM>(g, grid, st);
  }
}

// Entry used by sarathi_moe_grouped_gemm for row-major weights at 64-, 128- and 256-slot blocks.  `g`
// is complete except for n_blocks, which depends on the epilogue and the column-block width.
// Column blocks of 256 unless that leaves compute units short of workgroups.  Measured on the
// Mixtral projections: at 256-slot blocks (one workgroup per compute unit) 128-wide blocks are
// 1-12 % faster while the wide launch has fewer than 256 workgroups and 20 % slower from there
// on; at 64-slot blocks (two to three per compute unit) they are faster up to 896 workgroups
// (16-64 tokens: gate/up projection 0.333 -> 0.326 ms, down projection 0.205 -> 0.178 ms) and
// slower at 1792 (256 tokens).
bool moe_gemm_wide_takes_narrow_blocks(int64_t out_cols, int m_blocks, int block_m, int epilogue) {
  const int64_t cols_wide = epilogue == kEpiGatedSilu ? 128 : 256;
  const int64_t wide_blocks = (out_cols + cols_wide - 1) / cols_wide * m_blocks;
  return block_m != 128 && wide_blocks < (block_m == 256 ? 256 : 1024);
}

int launch_moe_gemm_wide(MoeGemmArgs g, int64_t out_cols, int block_m, int epilogue, int dtype,
                         hipStream_t st) {
  const bool narrow = moe_gemm_wide_takes_narrow_blocks(out_cols, g.m_blocks, block_m, epilogue);
#define SK_PICK(DT)                                                                               \
  if (block_m == 256)                                                                             \
    return narrow ? launch_wide_epilogue<DT, 128, 256>(g, out_cols, epilogue, st)                 \
                  : launch_wide_epilogue<DT, 256, 256>(g, out_cols, epilogue, st);                \
  if (block_m == 128)                                                                             \
    return launch_wide_epilogue<DT, 256, 128>(g, out_cols, epilogue, st);                         \
  return narrow ? launch_wide_epilogue<DT, 128, 64>(g, out_cols, epilogue, st)                    \
                : launch_wide_epilogue<DT, 256, 64>(g, out_cols, epilogue, st);
  if (dtype == kBF16) { SK_PICK(kBF16) } else { SK_PICK(kF16) }
#undef SK_PICK
}

}  // namespace sarathi_hip
