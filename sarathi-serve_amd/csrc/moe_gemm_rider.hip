// Grouped expert GEMM for row-major ([E, N, K]) expert weights at 256-slot blocks in which a
// workgroup can take along ("ride") one 32-slot tile of another block of the same expert.
//
// Same computation, argument block, tile order, LDS layout and wave tiling as moe_gemm_wide.hip at
// BM = BN = 256 (four waves, one per SIMD, each a 128 x 128 accumulator tile; two LDS buffers of
// one 64-element K-step each).  A workgroup's time is mostly the fixed cost of pulling its expert's
// 256-row weight tile through the compute unit: about 64 us for a block with a handful of slots
// against 113 us for a full one (Mixtral gate/up shape).  An expert's last block is such a block
// whenever its load is a little above a multiple of 256, which costs 8 % of a 4096-token Mixtral
// layer and 25 % of a 1024-token one.  Here the workgroups of the expert's full blocks each
// multiply one 32-slot tile of that last block with the weight fragments they read anyway, and the
// last block gets no workgroups at all.  The plan (which block takes which tile) is a table with
// one entry per block, made on the device from the sorted slots (moe_plan_riders_kernel).
//
// Two paths through the K-loop:
//   without a rider   tokens and weights move global -> registers -> LDS exactly as in
//                     moe_gemm_wide.hip (64 staging registers per lane);
//   with a rider      the rider tile's two accumulators (32 registers) take the place of the token
//                     staging registers, and tokens and rider rows move by buffer loads that write
//                     LDS directly (1 KiB per instruction: eight rows of 128 bytes, lane l the
//                     chunk that the rotated layout keeps at position l & 7 of row l >> 3).
// Results have the same bits as moe_gemm_wide.hip's: every output element is the same chain of
// MFMAs over K in the same order, whichever workgroup computes it.
#include <atomic>
#include "moe_gemm_common.h"
#include "launch.h"

namespace sarathi_hip {

constexpr int kRideBM = 256, kRideBN = 256;
constexpr int kRiderRows = 32;
// 16-byte units of one LDS buffer: token rows, weight rows, rider rows, 8 units (128 bytes) each
constexpr int kRideTokUnits = kRideBM * 8, kRideWgtUnits = kRideBN * 8, kRideRiderUnits = kRiderRows * 8;
constexpr int kRideBufUnits = kRideTokUnits + kRideWgtUnits + kRideRiderUnits;
constexpr int kRideLdsBytes = 2 * kRideBufUnits * 16;

// The rider's two accumulator tiles do not fit beside the 256 accumulator registers of the main
// tile and live in ordinary vector registers.  Written through the builtin, the register allocator
// answers a 17th and 18th accumulator by moving accumulators between the two register files around
// every MFMA of the loop (hundreds of copies per K-step); an instruction whose accumulator operand
// can only be a vector register keeps the rider's tiles where they are and the others untouched.
// The s_nop covers the wait states between a vector instruction that wrote an operand (the
// fragment select) and the matrix instruction that reads it, which the compiler does not insert
// for an instruction it cannot see.
template <int DT> SK_DEV void mfma32_in_vgprs(u32x4 a, u32x4 b, f32x16& c) {
  if constexpr (DT == kBF16)
    asm volatile("s_nop 1\n\tv_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(c) : "v"(a), "v"(b));
  else
    asm volatile("s_nop 1\n\tv_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+v"(c) : "v"(a), "v"(b));
}

// `ride` holds one entry per slot block: the first slot of a 32-slot tile that this block's
// workgroups multiply as well (a tile of the same expert's last block), -1 for none, or -2 for a
// block whose tiles are all taken along by others, which its own workgroups skip.
template <int DT, int EPI>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1)))
void moe_gemm_rider_kernel(MoeGemmArgs g, const int32_t* __restrict__ ride) {
  constexpr bool MUL_WEIGHT = EPI == kEpiMulWeight;
  constexpr bool GATED = EPI == kEpiGatedSilu;
  constexpr int BM = kRideBM, BN = kRideBN;
  constexpr int MT = 4, NT = 4, SUB = kGemmBK / 16;
  constexpr int WCR = BN / 2;      // weight rows of a wave column
  constexpr int W_ROWS = BN / 32;  // weight rows a thread moves per K-step
  extern __shared__ u32x4 lds[];

  int pid_m, pid_n;
  if (!tile_of_block(g, blockIdx.x, pid_m, pid_n)) return;
  if (pid_m * BM >= *g.num_tokens_post_padded) return;
  const int ride_slot0 = ride[pid_m];
  if (ride_slot0 == -2) return;
  const bool riding = ride_slot0 >= 0;
  const int expert = g.expert_ids[pid_m];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // scalar: LDS bases of the transfers
  const int wc = wave & 1;                  // wave column: BN / 2 weight rows
  const int wr = wave >> 1;                 // wave row
  const int row0 = wr * (BM / 2);           // first slot of this wave inside the block
  const int l32 = lane & 31, grp = lane >> 5;
  const int half_n = g.N >> 1;  // gated: weight rows [half_n, N) are the up projection

  auto weight_row = [&](int R) {  // as in moe_gemm_wide.hip
    if constexpr (GATED) {
      const int in_col = R % WCR;
      const int gate = pid_n * (BN / 2) + (R / WCR) * (WCR / 2) + in_col % (WCR / 2);
      return gate < half_n ? gate + (in_col / (WCR / 2)) * half_n : -1;
    } else {
      const int n = pid_n * BN + R;
      return n < g.N ? n : -1;
    }
  };

  const rsrc_t ra = make_rsrc(g.a, g.a_bytes);
  const rsrc_t rb = make_rsrc(reinterpret_cast<const char*>(g.b) + (int64_t)expert * g.b_expert_stride * 2,
                              (uint32_t)((int64_t)g.N * g.K * 2));
  // ---- tokens.  A workgroup without a rider moves them like the weights, global -> register ->
  // LDS, exactly as moe_gemm_wide.hip does.  A workgroup with a rider has no registers for that
  // (its rider accumulators take their place): it moves tokens and rider rows by transfers of
  // 1 KiB that write LDS directly, eight rows of 128 bytes each; wave w moves token rows
  // [64 w, 64 w + 64) with eight of them and rider rows [8 w, 8 w + 8) with a ninth, lane l the
  // chunk that the rotated layout keeps at position l & 7 of row l >> 3.
  auto token_offset = [&](int slot_index, int r_in_tile, int position) {
    const int sid = slot_index < g.em ? g.sorted_token_ids[slot_index] : g.num_valid;
    const uint32_t chunk = (uint32_t)lds_chunk_at(r_in_tile, position) * 16u;
    // a padding slot reads beyond the end of A, i.e. zeros, whatever K offset is added
    return sid < g.num_valid ? (uint32_t)(sid / g.top_k) * (uint32_t)(g.a_row_stride * 2) + chunk
                             : g.a_bytes;
  };
  // ---- weights: global -> register -> LDS as in moe_gemm_wide.hip: thread t moves position
  // t & 7 of rows (t >> 3) + 32 j
  const int pos = tid & 7;
  uint32_t w_off[W_ROWS];
#pragma unroll
  for (int j = 0; j < W_ROWS; ++j) {
    const int r = (tid >> 3) + 32 * j;
    const int n = weight_row(r);
    w_off[j] = n >= 0 ? (uint32_t)n * (uint32_t)g.K * 2u + (uint32_t)lds_chunk_at(r, pos) * 16u
                      : 0x80000000u;
  }
  u32x4 st_wgt[W_ROWS];
  auto load_rows = [&](int k0, int j0, int j1) {
#pragma unroll
    for (int j = j0; j < j1; ++j) st_wgt[j] = buf_load16<kCached>(rb, w_off[j] + (uint32_t)k0 * 2u);
  };
  auto store_rows = [&](int buf, int j0, int j1) {
#pragma unroll
    for (int j = j0; j < j1; ++j)
      lds[buf * kRideBufUnits + kRideTokUnits + ((tid >> 3) + 32 * j) * 8 + pos] = st_wgt[j];
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

  // The loop is compiled once per count of live token tiles and, for full blocks, once more with a
  // rider: each copy free of branches.  K-step i is read from LDS buffer i & 1.
  //   weights   (and, without a rider, tokens) sub-steps 0..2 store the registers (K-step i + 1,
  //             loaded during K-step i - 1) to the other buffer and load K-step i + 2 into them
  //             (the last loads in sub-step 3);
  //   barrier   before sub-step 3, whose operands are in registers by then: the stores and, with a
  //             rider, the token transfers of K-step i + 1 are visible, nobody reads buffer i & 1
  //             any more;
  //   with a rider  sub-step 3 issues the token transfers of K-step i + 2 into buffer i & 1.
  //             Before the next barrier they must have landed: six weight loads (sub-steps 0..2)
  //             are issued after them, so at most six vector-memory operations may still be
  //             outstanding there.
  auto k_loop_of = [&](auto live_tag, auto riding_tag, f32x16 (&racc)[2]) {
    constexpr int LIVE = decltype(live_tag)::value;  // token tiles 0 .. LIVE - 1 are computed
    constexpr bool RIDING = decltype(riding_tag)::value;
    constexpr int kTok = 9;  // RIDING: token transfers of a K-step, per wave
    uint32_t a_off[8], r_off = 0;
    u32x4 st_tok[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      if constexpr (RIDING) {
        const int r = wave * 64 + i * 8 + (lane >> 3);
        a_off[i] = token_offset(pid_m * BM + r, r, lane & 7);
      } else {
        const int r = (tid >> 3) + 32 * i;
        a_off[i] = token_offset(pid_m * BM + r, r, pos);
      }
    }
    if constexpr (RIDING) {
      const int r = wave * 8 + (lane >> 3);
      r_off = token_offset(ride_slot0 + r, r, lane & 7);
    }
    auto issue_tokens = [&](int k0, int buf) {  // RIDING
      u32x4* base = lds + buf * kRideBufUnits;
#pragma unroll
      for (int i = 0; i < 8; ++i)
        dma_load16_to_lds(ra, base + (wave * 64 + i * 8) * 8, a_off[i] + (uint32_t)k0 * 2u);
      dma_load16_to_lds(ra, base + kRideTokUnits + kRideWgtUnits + wave * 64, r_off + (uint32_t)k0 * 2u);
    };
    auto load_tokens = [&](int k0, int j0, int j1) {  // not RIDING
#pragma unroll
      for (int j = j0; j < j1; ++j) st_tok[j] = buf_load16<kCached>(ra, a_off[j] + (uint32_t)k0 * 2u);
    };
    auto store_tokens = [&](int buf, int j0, int j1) {
#pragma unroll
      for (int j = j0; j < j1; ++j)
        lds[buf * kRideBufUnits + ((tid >> 3) + 32 * j) * 8 + pos] = st_tok[j];
    };
    if constexpr (RIDING) {
      issue_tokens(0, 0);
      load_rows(0, 0, W_ROWS);
      store_rows(0, 0, W_ROWS);
      load_rows(wrap(1) * kGemmBK, 0, W_ROWS);
      issue_tokens(wrap(1) * kGemmBK, 1);
      wait_vmcnt<W_ROWS + kTok>();  // the tokens of K-step 0 (and the weights stored above)
    } else {
      load_tokens(0, 0, 8);
      load_rows(0, 0, W_ROWS);
      store_tokens(0, 0, 8);
      store_rows(0, 0, W_ROWS);
      load_tokens(wrap(1) * kGemmBK, 0, 8);
      load_rows(wrap(1) * kGemmBK, 0, W_ROWS);
    }
    lds_barrier();

    auto read_operands = [&](int buf, int s, u32x4 (&tv)[MT], u32x4 (&wv)[NT], u32x4& rv) {
      const u32x4* tb = lds + buf * kRideBufUnits;
      const u32x4* wb = tb + kRideTokUnits;
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        if (mt >= LIVE) continue;
        const int r = row0 + mt * 32 + l32;
        tv[mt] = tb[r * 8 + lds_slot(r, 2 * s + grp)];
      }
      if constexpr (RIDING)
        rv = tb[kRideTokUnits + kRideWgtUnits + l32 * 8 + lds_slot(l32, 2 * s + grp)];
      if (LIVE == 0) return;
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) {
        const int R = wc * WCR + nt * 32 + l32;
        wv[nt] = wb[R * 8 + lds_slot(R, 2 * s + grp)];
      }
    };
    u32x4 tv[2][MT], wv[2][NT], rv[2];
    read_operands(0, 0, tv[0], wv[0], rv[0]);
    auto sub_step = [&](auto s_tag, int cur, int k_load) {
      constexpr int s = decltype(s_tag)::value;
      constexpr int ST0 = s * 3, ST1 = s * 3 + 3 < W_ROWS ? s * 3 + 3 : W_ROWS;  // rows stored here
      if constexpr (s + 1 < SUB) {
        read_operands(cur, s + 1, tv[(s + 1) & 1], wv[(s + 1) & 1], rv[(s + 1) & 1]);
        if constexpr (!RIDING) store_tokens(cur ^ 1, ST0, ST1);
        store_rows(cur ^ 1, ST0, ST1);
      } else {
        if constexpr (RIDING) wait_vmcnt<6>();
        lds_barrier();
        read_operands(cur ^ 1, 0, tv[0], wv[0], rv[0]);
        if constexpr (RIDING) issue_tokens(k_load, cur);
      }
      if constexpr (!RIDING) load_tokens(k_load, s * 2, s * 2 + 2);
      load_rows(k_load, s * 2, s * 2 + 2);
      if constexpr (LIVE == 0) __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
          if (mt >= LIVE) continue;
          acc[nt][mt] = mfma32<DT>(wv[s & 1][nt], tv[s & 1][mt], acc[nt][mt]);
        }
      if constexpr (RIDING) {
        // which two weight fragments: uniform over the wave, picked without a branch
        const u32x4 wa = wr ? wv[s & 1][GATED ? 1 : 2] : wv[s & 1][0];
        const u32x4 wb = wr ? wv[s & 1][NT - 1] : wv[s & 1][GATED ? NT / 2 : 1];
        mfma32_in_vgprs<DT>(wa, rv[s & 1], racc[0]);
        mfma32_in_vgprs<DT>(wb, rv[s & 1], racc[1]);
      }
      if constexpr (LIVE == MT) {
        // One wave per SIMD: nothing else runs while this wave issues memory instructions, so
        // they go out one at a time in the shadow of the MFMAs: the LDS reads, the LDS stores, then
        // the global loads and transfers.
        constexpr int kMfma = 0x008, kVmem = 0x010, kDsRead = 0x100, kDsWrite = 0x200;
        constexpr int READS = MT + NT + (RIDING ? 1 : 0);
        constexpr int WRITES = (s + 1 < SUB ? ST1 - ST0 : 0) * (RIDING ? 1 : 2);
        constexpr int VMEM = RIDING ? 2 + (s + 1 < SUB ? 0 : kTok) : 4;
#pragma unroll
        for (int i = 0; i < READS; ++i) {
          __builtin_amdgcn_sched_group_barrier(kMfma, 1, 0);
          __builtin_amdgcn_sched_group_barrier(kDsRead, 1, 0);
        }
#pragma unroll
        for (int i = 0; i < WRITES; ++i) {
          __builtin_amdgcn_sched_group_barrier(kMfma, 1, 0);
          __builtin_amdgcn_sched_group_barrier(kDsWrite, 1, 0);
        }
        constexpr int LEFT = MT * NT - READS - WRITES;
        constexpr int PER = (VMEM + LEFT - 1) / LEFT;
#pragma unroll
        for (int i = 0; i < LEFT; ++i) {
          __builtin_amdgcn_sched_group_barrier(kMfma, 1, 0);
          __builtin_amdgcn_sched_group_barrier(kVmem, PER, 0);
        }
      } else if constexpr (LIVE > 0) {
        // partly filled blocks (never with a rider): the same idea with fewer MFMAs to hide behind
        // (several memory instructions per MFMA)
        constexpr int kMfma = 0x008, kMemory = 0x020 | 0x100 | 0x200;
        constexpr auto rows_in = [](int j0, int j1, int n) {  // rows j0 <= j < j1 that are below n
          return (j1 < n ? j1 : n) - (j0 < n ? j0 : n);
        };
        constexpr int STORES = s + 1 < SUB ? 2 * rows_in(ST0, ST1, W_ROWS) : 0;
        constexpr int LOADS = 2 * rows_in(s * 2, s * 2 + 2, W_ROWS);
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
    // the transfers issued past the last K-step must have landed before this workgroup's LDS can
    // be handed to the next one
    wait_vmcnt<0>();
  };
  auto k_loop = [&](auto live_tag) {
    f32x16 unused[2];
    k_loop_of(live_tag, std::false_type{}, unused);
  };

  // ---- epilogue pieces: lane holds, per accumulator quad, 4 consecutive columns of one token
  const int n_wave0 = GATED ? pid_n * (BN / 2) + wc * (WCR / 2) : pid_n * BN + wc * WCR;
  const int n_end = GATED ? half_n : g.N;
  auto store_quad = [&](char* crow, int n, const float (&v)[4]) {
    if (n + 3 < n_end) {
      u32x2 out = {pack2<DT>(v[0], v[1]), pack2<DT>(v[2], v[3])};
      *reinterpret_cast<u32x2*>(crow + (int64_t)n * 2) = out;
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (n + e < n_end) store_elem<DT>(crow, n + e, v[e]);
    }
  };
  if (riding) {  // riders go with full blocks
    // the rider tile: 32 slots x the 64 columns of two of this wave's weight tiles (gated: a gate
    // tile and its up tile)
    f32x16 racc[2];
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int i = 0; i < 16; ++i) racc[t][i] = 0.f;
    k_loop_of(std::integral_constant<int, MT>{}, std::true_type{}, racc);
    // wait states between the last matrix instruction and the first read of its result, which the
    // compiler does not insert for an instruction it cannot see
    asm volatile("s_nop 7\n\ts_nop 7\n\ts_nop 7" ::: "memory");
    const int slot_index = ride_slot0 + l32;
    const int sid = slot_index < g.em ? g.sorted_token_ids[slot_index] : g.num_valid;
    if (sid < g.num_valid) {
      float scale = 1.f;
      if constexpr (MUL_WEIGHT) scale = g.topk_weights[sid];
      char* crow = reinterpret_cast<char*>(g.c) + (int64_t)sid * g.c_row_stride * 2;
      const int rnt0 = GATED ? wr : 2 * wr, rnt1 = GATED ? wr + NT / 2 : 2 * wr + 1;
      constexpr int OUT_TILES = GATED ? 1 : 2;
#pragma unroll
      for (int t = 0; t < OUT_TILES; ++t) {
        const int nt = t == 0 ? rnt0 : rnt1;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int n = n_wave0 + nt * 32 + q * 8 + grp * 4;
          float v[4];
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            if constexpr (GATED) {
              const float x = rnd<DT>(racc[0][q * 4 + e]), y = rnd<DT>(racc[1][q * 4 + e]);
              v[e] = rnd<DT>(silu_f32(x)) * y;
            } else {
              v[e] = racc[t][q * 4 + e];
              if constexpr (MUL_WEIGHT) v[e] *= scale;
            }
          }
          store_quad(crow, n, v);
        }
      }
    }
  } else {
    call_with_live<MT>(mt_live, k_loop);
  }

  // ---- epilogue of the block's own tiles
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
        store_quad(crow, n, v);
      }
    }
  }
}

template <int DT, int EPI>
static int launch_rider(const MoeGemmArgs& g, const int32_t* ride, dim3 grid, hipStream_t st) {
  auto kernel = moe_gemm_rider_kernel<DT, EPI>;
  // more LDS than the default per-workgroup limit: opt in once per kernel and device
  static std::atomic<bool> raised[64] = {};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return SARATHI_ERR_LAUNCH;
  if (!raised[dev].load(std::memory_order_acquire)) {  // racing first calls both set it: harmless
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                            hipFuncAttributeMaxDynamicSharedMemorySize, kRideLdsBytes) != hipSuccess)
      return SARATHI_ERR_LAUNCH;
    raised[dev].store(true, std::memory_order_release);
  }
  hipLaunchKernelGGL(kernel, grid, dim3(256), kRideLdsBytes, st, g, ride);
  return launch_status();
}

template <int DT>
static int launch_rider_epilogue(MoeGemmArgs g, int64_t out_cols, int epilogue, const int32_t* ride,
                                 hipStream_t st) {
  const int64_t cols_per_block = epilogue == kEpiGatedSilu ? kRideBN / 2 : kRideBN;
  g.n_blocks = (int32_t)((out_cols + cols_per_block - 1) / cols_per_block);
  const int64_t blocks = (int64_t)((g.n_blocks + 7) / 8) * g.m_blocks * 8;
  if (blocks > 0x7fffffffLL) return SARATHI_ERR_UNSUPPORTED;
  const dim3 grid((unsigned)blocks);
  switch (epilogue) {
    case kEpiMulWeight: return launch_rider<DT, kEpiMulWeight>(g, ride, grid, st);
    case kEpiGatedSilu: return launch_rider<DT, kEpiGatedSilu>(g, ride, grid, st);
    default: return launch_rider<DT, kEpiPlain>(g, ride, grid, st);
  }
}

// Which tiles ride where.  moe_align_block_size fills an expert's blocks greedily, so only an
// expert's last block can be partly filled, from its start.  If that block holds t 32-slot tiles
// and the expert has at least t full blocks before it, tile j of the last block rides with the
// expert's j-th block and the last block itself is skipped.  One thread per block.
__global__ __launch_bounds__(256) void moe_plan_riders_kernel(
    const int32_t* __restrict__ sorted_token_ids, const int32_t* __restrict__ expert_ids,
    const int32_t* __restrict__ post_pad, int32_t num_valid, int32_t em, int32_t m_blocks,
    int32_t block_m, int32_t* __restrict__ ride) {
  const int b = blockIdx.x * 256 + threadIdx.x;
  if (b >= m_blocks) return;
  int end = *post_pad;
  if (end > em) end = em;
  const int live_blocks = end / block_m;
  int out = -1;
  if (b < live_blocks) {
    const int e = expert_ids[b];
    int b0 = b, last = b;
    while (b0 > 0 && expert_ids[b0 - 1] == e) --b0;
    while (last + 1 < live_blocks && expert_ids[last + 1] == e) ++last;
    // valid slots of the last block: its first entry that is padding (binary search: real ids
    // first, then padding)
    const int32_t* blk = sorted_token_ids + (int64_t)last * block_m;
    int lo = 0, hi = block_m;
    while (lo < hi) {
      const int mid = (lo + hi) >> 1;
      if (blk[mid] < num_valid) lo = mid + 1; else hi = mid;
    }
    const int tiles = (lo + 31) >> 5;
    if (last > b0 && tiles <= last - b0) {
      if (b == last) out = -2;
      else if (b - b0 < tiles) out = last * block_m + 32 * (b - b0);
    }
  }
  ride[b] = out;
}

// Row-major 16-bit weights, 256-slot blocks, with the riders table of sarathi_moe_plan_riders.
int launch_moe_gemm_rider(MoeGemmArgs g, int64_t out_cols, int epilogue, int dtype,
                         const int32_t* ride, hipStream_t st) {
  if (!ride) return SARATHI_ERR_INVALID_ARG;
  if (dtype == kBF16) return launch_rider_epilogue<kBF16>(g, out_cols, epilogue, ride, st);
  return launch_rider_epilogue<kF16>(g, out_cols, epilogue, ride, st);
}

}  // namespace sarathi_hip

extern "C" int sarathi_moe_plan_riders(const int32_t* sorted_token_ids, const int32_t* expert_ids,
                                       const int32_t* num_tokens_post_padded,
                                       int64_t num_valid_tokens, int64_t sorted_len, int block_m,
                                       int32_t* riders, int64_t riders_len, void* stream) {
  using namespace sarathi_hip;
  if (num_valid_tokens < 0 || sorted_len < 0 || block_m <= 0 || riders_len < 0)
    return SARATHI_ERR_INVALID_ARG;
  if (block_m != kRideBM) return SARATHI_ERR_UNSUPPORTED;
  const int64_t m_blocks = (sorted_len + block_m - 1) / block_m;
  if (riders_len < m_blocks) return SARATHI_ERR_INVALID_ARG;
  if (m_blocks == 0) return SARATHI_OK;
  if (!sorted_token_ids || !expert_ids || !num_tokens_post_padded || !riders)
    return SARATHI_ERR_INVALID_ARG;
  if (num_valid_tokens > 0x7fffffffLL || sorted_len > 0x7fffffffLL) return SARATHI_ERR_UNSUPPORTED;
  hipLaunchKernelGGL(moe_plan_riders_kernel, dim3((unsigned)((m_blocks + 255) / 256)), dim3(256), 0,
                     (hipStream_t)stream, sorted_token_ids, expert_ids, num_tokens_post_padded,
                     (int32_t)num_valid_tokens, (int32_t)sorted_len, (int32_t)m_blocks,
                     (int32_t)block_m, riders);
  return launch_status();
}
