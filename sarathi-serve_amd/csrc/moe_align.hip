// moe_align_block_size for gfx950: stable counting sort of token->expert ids
// with every expert's run padded to a multiple of block_size.
//
// Replaces csrc/moe_align_block_size_kernels.cu:23-135 of the reference, which
// runs ONE block of num_experts threads, each walking its shard serially
// through shared-memory read-modify-writes.  Here one workgroup of W waves
// (W = 16, or 8 above 512 experts) does the same sort with every lane busy:
//
//   1. count   wave w owns a contiguous, ascending chunk of the flat ids and
//              reads it 64 ids at a time, coalesced (up to 8 tiles are loaded
//              ahead, and a chunk of at most 8 tiles simply stays in registers
//              for pass 3).  Inside a 64-id tile the lanes that hold the same
//              expert find each other with a bit-serial ballot match (log2(E)
//              ballots), which gives every lane its rank among equal ids and
//              the group's size; the first lane of each group adds the size to
//              cnt[e][w] in LDS.
//   2. scan    per expert, an exclusive scan of cnt[e][.] over the waves done by
//              W adjacent lanes with shuffles, then a wave-level prefix scan of
//              the padded totals -> cumsum[].
//   3. scatter every wave walks its chunk again: slot = cumsum[e] + cnt[e][w]
//              + rank-in-tile, and the group leader bumps cnt[e][w].  Chunks
//              are ascending and tiles are visited in order, so the order
//              inside an expert is ascending token index, exactly the
//              reference's (stable) order.
//   4. expert_ids by binary search of cumsum, and (fill_pad) the padding slots
//              set to numel, the caller-side `fill_` of
//              sarathi/model_executor/layers/fused_moe/fused_moe.py:195.
//
// Each LDS counter has a single writer wave, there is no global scratch and no
// inter-workgroup traffic, so the result is deterministic and bit-exact.
//
// That single workgroup (moe_align_kernel) takes inputs of up to 256 ids, more than 256 experts,
// and id arrays that are not 16-byte aligned.  The other paths of this file, all with the same
// results:
//   moe_align_few_experts_kernel   up to 32 experts, 257..32768 ids: one launch of independent
//                                  four-wave workgroups with packed register counters
//                                  (8192 ids of 8 experts: 5.2 us)
//   moe_align_lds_hist_kernel      33..256 experts, same scheme with LDS histograms
//                                  (12288 ids of 64 experts: 7.4 us)
//   count -> scan -> scatter       above 32768 ids (16384 with more than 256 experts): three
//                                  launches over the whole GPU with a caller workspace, or with the
//                                  file-scope array of sarathi_moe_align_block_size_static
#include <atomic>

#include "moe_align_body.h"
#include "launch.h"

namespace sarathi_hip {

template <typename IdT>
__global__ __launch_bounds__(1024) void moe_align_kernel(
    const IdT* __restrict__ ids, int64_t numel, int E, int B, int nbits,
    int32_t* __restrict__ sorted, int64_t sorted_len, int32_t* __restrict__ expert_ids,
    int64_t expert_ids_len, int32_t* __restrict__ post_pad, int fill_pad) {
  __shared__ int32_t cnt[kAlignCntInts];
  __shared__ int32_t tot[kAlignMaxExperts];
  __shared__ int32_t cumsum[kAlignMaxExperts + 1];
  align_single_workgroup<IdT>(ids, numel, E, B, nbits, sorted, sorted_len, expert_ids,
                              expert_ids_len, post_pad, fill_pad, cnt, tot, cumsum);
}

// ---------------------------------------------------------------------------
// Few experts (E <= 32), up to 32 768 ids: ONE launch of several workgroups that never talk to
// each other.  A single workgroup is bound by one compute unit's instruction issue (8192 ids,
// 8 experts: 8.5 us, and twice that with half the waves); here every workgroup reads ALL ids
// (they sit in L2, 32 KiB) and derives by itself the two things it needs: the per-expert totals
// (-> cumsum) and the per-expert count of everything before its own tiles.  Counting is one
// shift-and-add per id into byte-wide fields of a 64-bit register per lane (8 experts per
// register), folded over the wave and the workgroup's four waves at the end.  A wave then
// scatters its own one or two tiles with one ballot per expert.  The results do not depend on
// how many workgroups run, and nothing is exchanged through global memory, so the sort is
// deterministic and bit-exact.  8192 ids, 8 experts on MI355X: 8.5 us as one workgroup, 6.2 us
// in this form with 64-bit counters and shuffle scans, 5.2 us with 32-bit counters, DPP folds and
// the expert prefix in scalar registers (the shipped form).  expert_ids and the padding slots are
// written in slices, one per workgroup.
// ---------------------------------------------------------------------------
constexpr int kFewMaxExperts = 32;
// Largest input of the one-launch kernels below.  Every workgroup reads all ids, so the work
// grows with the square of the input; measured against the three-launch path on MI355X: 24 576
// ids of 64 experts 11.5 vs 18.8 us, 32 768 ids of 8 experts 11.8 vs 12.9 us, 49 152 ids of 64
// experts 20.2 vs 20.9 us.  (A byte-wide counter of the few-experts kernel sees at most
// 32768 / 256 = 128 ids.)
constexpr int64_t kOneLaunchMaxIds = 32768;
constexpr int kFewWaves = 4;
// The few-experts kernel counts in byte-wide fields per lane and folds them over the wave in
// 16-bit fields: a lane sees at most kOneLaunchMaxIds / (64 * kFewWaves) ids (plus one load's worth
// of rounding), a wave 64 times that.  Raising the id limit or lowering the wave count past these
// bounds would wrap a counter silently.
static_assert(kOneLaunchMaxIds / (64 * kFewWaves) + 4 <= 255,
              "per-lane byte counters of moe_align_few_experts_kernel would overflow");
static_assert(kOneLaunchMaxIds / kFewWaves + 4 * 64 <= 65535,
              "16-bit wave totals of moe_align_few_experts_kernel would overflow");
constexpr int kFewCountBatch = 8;   // 16-byte loads in flight per lane while counting

// Adds `v` over the 64 lanes of a wave; the total is valid in LANE 63 only.  Four DPP folds make
// every row of 16 lanes uniform, two row broadcasts carry the row totals up to the last row.  Six
// VALU instructions and no scalar round trip (six ds_bpermute shuffles cost ten times as much).
template <int CTRL, int ROW_MASK> SK_DEV uint32_t dpp_add_u32(uint32_t x) {
  return x + (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, CTRL, ROW_MASK, 0xf, false);
}
SK_DEV uint32_t wave64_sum_to_lane63(uint32_t v) {
  v = dpp_add_u32<0xB1, 0xf>(v);   // quad_perm [1,0,3,2]
  v = dpp_add_u32<0x4E, 0xf>(v);   // quad_perm [2,3,0,1]
  v = dpp_add_u32<0x141, 0xf>(v);  // row_half_mirror
  v = dpp_add_u32<0x140, 0xf>(v);  // row_mirror
  v = dpp_add_u32<0x142, 0xa>(v);  // row_bcast:15 into rows 1 and 3
  v = dpp_add_u32<0x143, 0xc>(v);  // row_bcast:31 into rows 2 and 3
  return v;
}

// ACCS = ceil(E / 4) packed counters per lane (four byte-wide fields each)
template <typename IdT, int ACCS>
__global__ __launch_bounds__(64 * kFewWaves) void moe_align_few_experts_kernel(
    const IdT* __restrict__ ids, int64_t numel, int E, int B, int32_t* __restrict__ sorted,
    int64_t sorted_len, int32_t* __restrict__ expert_ids, int64_t expert_ids_len,
    int32_t* __restrict__ post_pad, int fill_pad) {
  constexpr int EMAX = ACCS * 4;
  // per wave: totals and before-counts as 16-bit fields, two experts per dword
  __shared__ uint32_t red[kFewWaves][2][ACCS * 2];   // [wave][all / before][packed halves]
  __shared__ int32_t own[kFewWaves][EMAX];           // ids of expert e in wave w's own tile
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // uniform, and the compiler knows it
  const int tiles_total = (int)((numel + 63) >> 6);
  const int wg_first = (int)blockIdx.x * kFewWaves;  // first own tile of the workgroup
  const int my_tile = wg_first + wave;               // the wave's own tile

  // ---- own tile: its ids stay in a register for the scatter
  const rsrc_t rid = id_rsrc(ids, 0, numel);  // at most 32768 ids
  int mine;
  {
    const int64_t i = ((int64_t)my_tile << 6) + lane;
    const IdT raw = buf_load_id<IdT>(rid, (uint32_t)(i * (int64_t)sizeof(IdT)));
    mine = i < numel ? checked_expert(raw, E) : -1;
  }

  // ---- count all ids: wave v of every workgroup takes the v-th quarter of them, each lane
  // kPer consecutive ids per load (16 bytes of int32 ids), so a step covers 64 * kPer ids.  Steps
  // are visited in ascending order and the workgroup's own tiles start on a step boundary (256
  // ids), so the count of everything before them is the running count at the moment the walk
  // reaches that boundary.
  // The vector loads see the array rounded up to whole 16-byte granules: a load that straddles
  // the exact end would be dropped as a whole by the range check, valid ids included.  `ids` is
  // 16-byte aligned here, so the granule that holds the last id lies inside the same page; what
  // is read beyond the last id is discarded by position.
  const rsrc_t rid16 = make_rsrc(ids, (uint32_t)((numel * (int64_t)sizeof(IdT) + 15) & ~15ll));
  constexpr int kPer = sizeof(IdT) == 8 ? 2 : 4;
  constexpr int kStepIds = 64 * kPer;
  const int steps_total = (int)((numel + kStepIds - 1) / kStepIds);
  const int own_step = wg_first * 64 / kStepIds;  // first step of the workgroup's own tiles
  const int quarter = (steps_total + kFewWaves - 1) / kFewWaves;
  const int q_lo = wave * quarter;
  const int q_hi = q_lo + quarter < steps_total ? q_lo + quarter : steps_total;
  uint32_t all[ACCS], before[ACCS];
#pragma unroll
  for (int a = 0; a < ACCS; ++a) all[a] = before[a] = 0u;
  for (int t0 = q_lo; t0 < q_hi; t0 += kFewCountBatch) {
    int e[kFewCountBatch][kPer];
#pragma unroll
    for (int u = 0; u < kFewCountBatch; ++u) {
      const int64_t i0 = ((int64_t)(t0 + u) * 64 + lane) * kPer;  // first id of the lane
      const uint32_t off = (uint32_t)(i0 * (int64_t)sizeof(IdT));
      IdT raw[kPer];
      if constexpr (sizeof(IdT) >= 4) {
        const u32x4 v = buf_load16<kCached>(rid16, off);
        if constexpr (sizeof(IdT) == 4) {
          raw[0] = (IdT)v.x; raw[1] = (IdT)v.y; raw[2] = (IdT)v.z; raw[3] = (IdT)v.w;
        } else {
          raw[0] = (IdT)(((uint64_t)v.y << 32) | v.x);
          raw[1] = (IdT)(((uint64_t)v.w << 32) | v.z);
        }
      } else if constexpr (sizeof(IdT) == 2) {
        const u32x2 v = buf_load8<kCached>(rid16, off);
        raw[0] = (IdT)(v.x & 0xffffu); raw[1] = (IdT)(v.x >> 16);
        raw[2] = (IdT)(v.y & 0xffffu); raw[3] = (IdT)(v.y >> 16);
      } else {
        const uint32_t v = (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(rid16, off, 0, 0);
        raw[0] = (IdT)(v & 0xffu); raw[1] = (IdT)((v >> 8) & 0xffu);
        raw[2] = (IdT)((v >> 16) & 0xffu); raw[3] = (IdT)(v >> 24);
      }
#pragma unroll
      for (int j = 0; j < kPer; ++j)
        e[u][j] = (t0 + u < q_hi && i0 + j < numel) ? checked_expert(raw[j], E) : -1;
    }
    __builtin_amdgcn_sched_barrier(0);  // the whole batch is in flight before the first use
#pragma unroll
    for (int u = 0; u < kFewCountBatch; ++u) {
      const bool snapshot = t0 + u == own_step;  // uniform
#pragma unroll
      for (int a = 0; a < ACCS; ++a) before[a] = snapshot ? all[a] : before[a];
#pragma unroll
      for (int j = 0; j < kPer; ++j) {
        const uint32_t one = 1u << ((e[u][j] & 3) * 8);
#pragma unroll
        for (int a = 0; a < ACCS; ++a)
          all[a] += (e[u][j] >> 2) == a ? one : 0u;  // -1 >> 2 matches no accumulator
      }
    }
  }
  if (own_step >= q_hi) {  // the whole quarter lies before the workgroup's tiles (uniform)
#pragma unroll
    for (int a = 0; a < ACCS; ++a) before[a] = all[a];
  }
  // a lane has seen at most 32768 / 4 / 64 = 128 ids, so a byte field holds at most 128; widen
  // the fields to 16 bits (even and odd experts apart) and add over the wave: at most 8192 per field
#pragma unroll
  for (int a = 0; a < ACCS; ++a) {
#pragma unroll
    for (int which = 0; which < 2; ++which) {
      const uint32_t v = which ? before[a] : all[a];
      const uint32_t r0 = wave64_sum_to_lane63(v & 0x00ff00ffu);         // experts 4a+0 (low), 4a+2 (high)
      const uint32_t r1 = wave64_sum_to_lane63((v >> 8) & 0x00ff00ffu);  // experts 4a+1, 4a+3
      if (lane == 63) {
        red[wave][which][a * 2 + 0] = r0;
        red[wave][which][a * 2 + 1] = r1;
      }
    }
  }
  // ---- ids per expert in the wave's own tile
  {
    int c = 0;
#pragma unroll
    for (int x = 0; x < EMAX; ++x) {
      const int n = __popcll(__ballot(mine == x));
      c = lane == x ? n : c;
    }
    if (lane < EMAX) own[wave][lane] = c;
  }
  __syncthreads();

  // ---- every wave on its own: totals, cumsum, first slot of its own ids of every expert.
  // Lane x < E gathers expert x's figures; the prefix over the experts runs in scalar registers,
  // which is also where the scatter below wants the result.
  int tot = 0, bef = 0, padded = 0;
  {
    const int x = lane < E ? lane : 0;
    const int word = (x >> 2) * 2 + (x & 1), shift = ((x >> 1) & 1) * 16;
    uint32_t ra[kFewWaves], rb[kFewWaves];
    int ro[kFewWaves];
#pragma unroll
    for (int w = 0; w < kFewWaves; ++w) {  // all reads first, one wait
      ra[w] = red[w][0][word];
      rb[w] = red[w][1][word];
      ro[w] = own[w][x];
    }
#pragma unroll
    for (int w = 0; w < kFewWaves; ++w) {
      tot += (ra[w] >> shift) & 0xffff;
      bef += (rb[w] >> shift) & 0xffff;
      bef += w < wave ? ro[w] : 0;
    }
    if (lane >= E) tot = bef = 0;
    padded = (tot + B - 1) / B * B;
  }
  // scalars: cum[x] = first slot of expert x, first[x] = first slot of this wave's ids of it
  int first[EMAX], cum[EMAX + 1], count[EMAX];
  cum[0] = 0;
#pragma unroll
  for (int x = 0; x < EMAX; ++x) {
    first[x] = cum[x] + __builtin_amdgcn_readlane(bef, x);
    count[x] = __builtin_amdgcn_readlane(tot, x);
    cum[x + 1] = cum[x] + __builtin_amdgcn_readlane(padded, x);
  }
  const int total = cum[EMAX];
  if (blockIdx.x == 0 && tid == 0) *post_pad = total;

  // ---- scatter the own tile: one ballot per expert gives every member its rank
  {
    int slot = -1;
#pragma unroll
    for (int x = 0; x < EMAX; ++x) {
      const unsigned long long m = __ballot(mine == x);
      const int rank = __builtin_amdgcn_mbcnt_hi((unsigned)(m >> 32),
                                                 __builtin_amdgcn_mbcnt_lo((unsigned)m, 0));
      slot = mine == x ? first[x] + rank : slot;
    }
    if (slot >= 0 && slot < sorted_len) sorted[slot] = (int32_t)(((int64_t)my_tile << 6) + lane);
  }

  // ---- expert id of every block and the padding slots, in slices over all threads of the grid;
  // the prefix is in scalar registers, so no table look-up: the expert of a block is the number
  // of experts whose run ends at or before the block's first slot
  const int64_t gtid = (int64_t)blockIdx.x * blockDim.x + tid;
  const int64_t gthreads = (int64_t)gridDim.x * blockDim.x;
  const int nblk = total / B;
  for (int64_t b = gtid; b < nblk; b += gthreads) {
    if (b < expert_ids_len) {
      const int pos = (int)b * B;
      int x = 0;
#pragma unroll
      for (int y = 1; y < EMAX; ++y) x += pos >= cum[y] ? 1 : 0;  // cum[y] = total for y > E
      expert_ids[b] = x;
    }
  }
  if (fill_pad) {
    const int32_t pad = (int32_t)numel;
    for (int64_t j = gtid; j < B; j += gthreads) {  // an expert's run ends with < B padding slots
#pragma unroll
      for (int x = 0; x < EMAX; ++x) {
        const int64_t slot = (int64_t)cum[x] + count[x] + j;
        if (slot < cum[x + 1]) sorted[slot] = pad;
      }
    }
    for (int64_t i = (int64_t)total + gtid; i < sorted_len; i += gthreads) sorted[i] = pad;
  }
}

// ---------------------------------------------------------------------------
// 33 .. 256 experts, up to 32 768 ids: the same independent-workgroups scheme with the counters
// in LDS.  Every wave keeps a histogram row of its quarter of the ids (one LDS atomic per id;
// with this many experts the lanes of a wave rarely collide), copies it at the moment its walk
// reaches the workgroup's own tiles (= the count of everything before them), and ranks the ids
// of its own tile with the bit-serial ballot match.  After ONE barrier every wave combines the
// four rows by itself.  (One workgroup of 16 waves needs 20 us for 12 288 ids of 64 experts.)
// ---------------------------------------------------------------------------
constexpr int kHistMaxExperts = 256;

template <typename IdT>
__global__ __launch_bounds__(64 * kFewWaves) void moe_align_lds_hist_kernel(
    const IdT* __restrict__ ids, int64_t numel, int E, int B, int nbits,
    int32_t* __restrict__ sorted, int64_t sorted_len, int32_t* __restrict__ expert_ids,
    int64_t expert_ids_len, int32_t* __restrict__ post_pad, int fill_pad) {
  __shared__ int32_t hist[kFewWaves][kHistMaxExperts];    // ids of expert x in wave w's quarter
  __shared__ int32_t bef[kFewWaves][kHistMaxExperts];     // ... of those, before the own tiles
  __shared__ int32_t own[kFewWaves][kHistMaxExperts];     // ids of expert x in wave w's own tile
  __shared__ int32_t firsts[kFewWaves][kHistMaxExperts];  // per wave: first slot of its ids of x
  __shared__ int32_t cums[kFewWaves][kHistMaxExperts + 1];
  __shared__ int32_t tots[kFewWaves][kHistMaxExperts];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wg_first = (int)blockIdx.x * kFewWaves;
  const int my_tile = wg_first + wave;
  for (int x = lane; x < E; x += 64) hist[wave][x] = bef[wave][x] = own[wave][x] = 0;  // own rows

  const rsrc_t rid = id_rsrc(ids, 0, numel);
  int mine;
  {
    const int64_t i = ((int64_t)my_tile << 6) + lane;
    const IdT raw = buf_load_id<IdT>(rid, (uint32_t)(i * (int64_t)sizeof(IdT)));
    mine = i < numel ? checked_expert(raw, E) : -1;
  }

  // ---- count: a step is 64 ids here (the own tiles start on a step boundary)
  const int tiles_total = (int)((numel + 63) >> 6);
  const int quarter = (tiles_total + kFewWaves - 1) / kFewWaves;
  const int q_lo = wave * quarter;
  const int q_hi = q_lo + quarter < tiles_total ? q_lo + quarter : tiles_total;
  for (int t0 = q_lo; t0 < q_hi; t0 += kAlignBatch) {
    int e[kAlignBatch];
#pragma unroll
    for (int u = 0; u < kAlignBatch; ++u) {
      const int64_t i = ((int64_t)(t0 + u) << 6) + lane;
      const IdT raw = buf_load_id<IdT>(rid, (uint32_t)(i * (int64_t)sizeof(IdT)));
      e[u] = (t0 + u < q_hi && i < numel) ? checked_expert(raw, E) : -1;
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int u = 0; u < kAlignBatch; ++u) {
      if (t0 + u == wg_first) {  // uniform: LDS operations of a wave complete in order
        for (int x = lane; x < E; x += 64) bef[wave][x] = hist[wave][x];
      }
      if (e[u] >= 0) atomicAdd(&hist[wave][e[u]], 1);
    }
  }
  if (wg_first >= q_hi) {
    for (int x = lane; x < E; x += 64) bef[wave][x] = hist[wave][x];
  }
  // ---- own tile: rank among equal ids and the group's size
  const TileMatch m = match_expert(mine, mine >= 0, nbits);
  if (mine >= 0 && m.rank == 0) own[wave][mine] = m.count;
  __syncthreads();

  // ---- every wave on its own: totals, padded prefix, first slot of its ids of every expert
  int carry = 0;
  for (int base = 0; base < E; base += 64) {
    const int x = base + lane;
    int tot = 0, b = 0;
    if (x < E) {
#pragma unroll
      for (int w = 0; w < kFewWaves; ++w) {
        tot += hist[w][x];
        b += bef[w][x] + (w < wave ? own[w][x] : 0);
      }
    }
    const int padded = x < E ? (tot + B - 1) / B * B : 0;
    int incl = padded;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
      const int y = __shfl_up(incl, off, 64);
      if (lane >= off) incl += y;
    }
    if (x < E) {
      cums[wave][x] = carry + incl - padded;
      tots[wave][x] = tot;
      firsts[wave][x] = carry + incl - padded + b;
    }
    carry += __shfl(incl, 63, 64);
  }
  const int total = carry;
  if (lane == 0) cums[wave][E] = total;
  if (blockIdx.x == 0 && tid == 0) *post_pad = total;

  // ---- scatter the own tile (the wave reads back its own LDS rows: in order, no barrier)
  if (mine >= 0) {
    const int64_t slot = (int64_t)firsts[wave][mine] + m.rank;
    if (slot < sorted_len) sorted[slot] = (int32_t)(((int64_t)my_tile << 6) + lane);
  }

  // ---- expert id of every block and the padding slots, in slices over all threads of the grid
  const int32_t* cs = cums[wave];
  const int64_t gtid = (int64_t)blockIdx.x * blockDim.x + tid;
  const int64_t gthreads = (int64_t)gridDim.x * blockDim.x;
  const int nblk = total / B;
  for (int64_t b = gtid; b < nblk; b += gthreads) {
    if (b < expert_ids_len) {
      const int pos = (int)b * B;
      int lo = 0, hi = E;  // invariant: cumsum[lo] <= pos < cumsum[hi]
      while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (cs[mid] <= pos) lo = mid; else hi = mid;
      }
      expert_ids[b] = lo;
    }
  }
  if (fill_pad) {
    const int32_t pad = (int32_t)numel;
    for (int64_t i = gtid; i < (int64_t)E * B; i += gthreads) {
      const int x = (int)(i / B), j = (int)(i - (int64_t)x * B);
      const int64_t slot = (int64_t)cs[x] + tots[wave][x] + j;
      if (slot < cs[x + 1]) sorted[slot] = pad;
    }
    for (int64_t i = (int64_t)total + gtid; i < sorted_len; i += gthreads) sorted[i] = pad;
  }
}

// ---------------------------------------------------------------------------
// Large inputs: the same sort spread over the chip in three launches.  The flat
// ids are cut into NC contiguous wave-chunks of `tiles_per_chunk` 64-id tiles
// (four chunks = four waves per workgroup).  The workspace holds
//   hist[E][NC]   tokens of expert e in chunk c, turned by the scan kernel into
//                 the exclusive prefix over the chunks (the chunk's offset
//                 inside expert e's run)
//   cumsum[E+1]   padded exclusive scan over the experts
// Chunks are ascending and each wave walks its chunk in order, so the order
// inside an expert stays ascending token index.
// ---------------------------------------------------------------------------
constexpr int kChunkWaves = 4;           // waves (= chunks) per workgroup of the count / scatter kernels
constexpr int kMaxChunks = 1024;
constexpr int64_t kMultiThreshold = 16384;  // ids above which the three-launch path pays off

struct ChunkPlan {
  int num_chunks;        // multiple of kChunkWaves
  int64_t tiles_per_chunk;
};
static ChunkPlan plan_chunks(int64_t numel) {
  const int64_t tiles = (numel + 63) >> 6;
  int64_t nc = (tiles + kAlignBatch - 1) / kAlignBatch;  // aim at one 8-tile batch per chunk
  if (nc > kMaxChunks) nc = kMaxChunks;
  nc = (nc + kChunkWaves - 1) / kChunkWaves * kChunkWaves;
  ChunkPlan p;
  p.num_chunks = (int)nc;
  p.tiles_per_chunk = (tiles + nc - 1) / nc;
  return p;
}
static int64_t align_workspace_ints(int num_chunks, int E) {
  return (int64_t)E * num_chunks + E + 1;
}

template <typename IdT>
__global__ __launch_bounds__(64 * kChunkWaves) void moe_align_count_kernel(
    const IdT* __restrict__ ids, int64_t numel, int E, int nbits, int num_chunks,
    int64_t tiles_per_chunk, int32_t* __restrict__ hist) {
  __shared__ int32_t cnt[kChunkWaves * kAlignMaxExperts];  // [wave][E]
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int chunk = blockIdx.x * kChunkWaves + wave;
  int32_t* my = cnt + wave * E;
  for (int i = lane; i < E; i += 64) my[i] = 0;  // each wave clears and reads only its own row
  const int64_t tiles_total = (numel + 63) >> 6;
  const int64_t tile_lo = chunk * tiles_per_chunk;
  int64_t tile_hi = tile_lo + tiles_per_chunk;
  if (tile_hi > tiles_total) tile_hi = tiles_total;
  const rsrc_t rid = id_rsrc(ids, tile_lo << 6, numel);  // this wave's chunk
  for (int64_t t0 = tile_lo; t0 < tile_hi; t0 += kAlignBatch) {
    int e[kAlignBatch];
#pragma unroll
    for (int u = 0; u < kAlignBatch; ++u) {
      const int64_t i = ((t0 + u) << 6) + lane;
      const IdT raw = buf_load_id<IdT>(
          rid, (uint32_t)((((t0 + u - tile_lo) << 6) + lane) * (int64_t)sizeof(IdT)));
      e[u] = (t0 + u < tile_hi && i < numel) ? checked_expert(raw, E) : -1;
    }
#pragma unroll
    for (int u = 0; u < kAlignBatch; ++u) {
      if (t0 + u < tile_hi) {
        const bool valid = e[u] >= 0;
        const TileMatch m = match_expert(e[u], valid, nbits);
        if (valid && m.rank == 0) atomicAdd(&my[e[u]], m.count);
      }
    }
  }
  // LDS operations of one wave complete in order: the row is final here
  for (int i = lane; i < E; i += 64) hist[(int64_t)i * num_chunks + chunk] = my[i];
}

// One workgroup: per expert an exclusive scan over the chunks, then the padded prefix over the
// experts, expert ids, padding slots.
__global__ __launch_bounds__(1024) void moe_align_scan_kernel(
    int32_t* __restrict__ hist, int32_t* __restrict__ cumsum_out, int64_t numel, int E, int B,
    int num_chunks, int32_t* __restrict__ sorted, int64_t sorted_len,
    int32_t* __restrict__ expert_ids, int64_t expert_ids_len, int32_t* __restrict__ post_pad,
    int fill_pad) {
  __shared__ int32_t tot[kAlignMaxExperts];
  __shared__ int32_t cumsum[kAlignMaxExperts + 1];
  const int tid = threadIdx.x, nthr = blockDim.x, wave = tid >> 6, lane = tid & 63, W = nthr >> 6;
  for (int x = wave; x < E; x += W) {  // a wave scans one expert's row of num_chunks counts
    int32_t* row = hist + (int64_t)x * num_chunks;
    constexpr int kSegs = kMaxChunks / 64;
    int c[kSegs];
#pragma unroll
    for (int j = 0; j < kSegs; ++j) {  // the whole row is fetched before the first use
      const int i = j * 64 + lane;
      c[j] = i < num_chunks ? row[i] : 0;
    }
    int carry = 0;
#pragma unroll
    for (int j = 0; j < kSegs; ++j) {
      if (j * 64 < num_chunks) {
        int v = c[j];
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
          const int y = __shfl_up(v, off, 64);
          if (lane >= off) v += y;
        }
        const int i = j * 64 + lane;
        if (i < num_chunks) row[i] = carry + v - c[j];
        carry += __shfl(v, 63, 64);
      }
    }
    if (lane == 0) tot[x] = carry;
  }
  __syncthreads();
  if (wave == 0) {
    int carry = 0;
    for (int base = 0; base < E; base += 64) {
      const int i = base + lane;
      int x = i < E ? (tot[i] + B - 1) / B * B : 0;
#pragma unroll
      for (int off = 1; off < 64; off <<= 1) {
        const int y = __shfl_up(x, off, 64);
        if (lane >= off) x += y;
      }
      if (i < E) cumsum[i + 1] = carry + x;
      carry += __shfl(x, 63, 64);
    }
    if (lane == 0) {
      cumsum[0] = 0;
      *post_pad = carry;
    }
  }
  __syncthreads();
  for (int i = tid; i <= E; i += nthr) cumsum_out[i] = cumsum[i];
  const int total = cumsum[E];
  const int nblk = total / B;
  for (int b = tid; b < nblk; b += nthr) {
    if (b < expert_ids_len) {
      const int pos = b * B;
      int lo = 0, hi = E;
      while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (cumsum[mid] <= pos) lo = mid; else hi = mid;
      }
      expert_ids[b] = lo;
    }
  }
  if (fill_pad) {
    const int32_t pad = (int32_t)numel;
    for (int64_t i = tid; i < (int64_t)E * B; i += nthr) {
      const int x = (int)(i / B), j = (int)(i - (int64_t)x * B);
      const int64_t slot = (int64_t)cumsum[x] + tot[x] + j;
      if (slot < cumsum[x + 1]) sorted[slot] = pad;
    }
    for (int64_t i = (int64_t)total + tid; i < sorted_len; i += nthr) sorted[i] = pad;
  }
}

template <typename IdT>
__global__ __launch_bounds__(64 * kChunkWaves) void moe_align_scatter_kernel(
    const IdT* __restrict__ ids, int64_t numel, int E, int nbits, int num_chunks,
    int64_t tiles_per_chunk, const int32_t* __restrict__ hist,
    const int32_t* __restrict__ cumsum, int32_t* __restrict__ sorted, int64_t sorted_len) {
  __shared__ int32_t pos[kChunkWaves * kAlignMaxExperts];  // [wave][E]: next slot of expert e
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int chunk = blockIdx.x * kChunkWaves + wave;
  int32_t* my = pos + wave * E;
  for (int i = lane; i < E; i += 64) my[i] = cumsum[i] + hist[(int64_t)i * num_chunks + chunk];
  const int64_t tiles_total = (numel + 63) >> 6;
  const int64_t tile_lo = chunk * tiles_per_chunk;
  int64_t tile_hi = tile_lo + tiles_per_chunk;
  if (tile_hi > tiles_total) tile_hi = tiles_total;
  const rsrc_t rid = id_rsrc(ids, tile_lo << 6, numel);  // this wave's chunk
  for (int64_t t0 = tile_lo; t0 < tile_hi; t0 += kAlignBatch) {
    int e[kAlignBatch];
#pragma unroll
    for (int u = 0; u < kAlignBatch; ++u) {
      const int64_t i = ((t0 + u) << 6) + lane;
      const IdT raw = buf_load_id<IdT>(
          rid, (uint32_t)((((t0 + u - tile_lo) << 6) + lane) * (int64_t)sizeof(IdT)));
      e[u] = (t0 + u < tile_hi && i < numel) ? checked_expert(raw, E) : -1;
    }
#pragma unroll
    for (int u = 0; u < kAlignBatch; ++u) {
      if (t0 + u < tile_hi) {
        const bool valid = e[u] >= 0;
        const TileMatch m = match_expert(e[u], valid, nbits);
        if (valid) {
          int32_t* c = &my[e[u]];
          const int64_t slot = (int64_t)*c + m.rank;  // read by the whole group before the add
          if (slot < sorted_len) sorted[slot] = (int32_t)(((t0 + u) << 6) + lane);
          if (m.rank == 0) atomicAdd(c, m.count);
        }
      }
    }
  }
}

template <typename IdT>
static int launch_align(const void* ids, int64_t numel, int E, int B, int32_t* sorted,
                        int64_t sorted_len, int32_t* expert_ids, int64_t expert_ids_len,
                        int32_t* post_pad, int fill_pad, void* workspace, int64_t workspace_bytes,
                        hipStream_t st) {
  int nbits = 0;
  while ((1 << nbits) < E) ++nbits;
  const IdT* idp = reinterpret_cast<const IdT*>(ids);
  const bool one_launch = E <= kHistMaxExperts && numel <= kOneLaunchMaxIds;
  if (numel > kMultiThreshold && !one_launch && workspace != nullptr) {
    const ChunkPlan plan = plan_chunks(numel);
    if (workspace_bytes >= align_workspace_ints(plan.num_chunks, E) * 4 &&
        (reinterpret_cast<uintptr_t>(workspace) & 3u) == 0) {
      int32_t* hist = reinterpret_cast<int32_t*>(workspace);
      int32_t* cumsum = hist + (int64_t)E * plan.num_chunks;
      const dim3 grid((unsigned)(plan.num_chunks / kChunkWaves)), block(64 * kChunkWaves);
      hipLaunchKernelGGL((moe_align_count_kernel<IdT>), grid, block, 0, st, idp, numel, E, nbits,
                         plan.num_chunks, plan.tiles_per_chunk, hist);
      hipLaunchKernelGGL(moe_align_scan_kernel, dim3(1), dim3(1024), 0, st, hist, cumsum, numel, E,
                         B, plan.num_chunks, sorted, sorted_len, expert_ids, expert_ids_len,
                         post_pad, fill_pad);
      hipLaunchKernelGGL((moe_align_scatter_kernel<IdT>), grid, block, 0, st, idp, numel, E, nbits,
                         plan.num_chunks, plan.tiles_per_chunk, hist, cumsum, sorted, sorted_len);
      return launch_status();
    }
  }
  if (one_launch && E <= kFewMaxExperts && numel > 64 * kFewWaves && aligned16(ids)) {
    // one tile per wave, four waves per workgroup: at most 64 workgroups
    const int64_t tiles = (numel + 63) >> 6;
    const int64_t groups = (tiles + kFewWaves - 1) / kFewWaves;
#define SK_ALIGN_FEW(ACCS)                                                                       \
  hipLaunchKernelGGL((moe_align_few_experts_kernel<IdT, ACCS>), dim3((unsigned)groups),         \
                     dim3(64 * kFewWaves), 0, st, idp, numel, E, B, sorted, sorted_len,          \
                     expert_ids, expert_ids_len, post_pad, fill_pad)
    if (E <= 8) SK_ALIGN_FEW(2);
    else if (E <= 16) SK_ALIGN_FEW(4);
    else SK_ALIGN_FEW(8);
#undef SK_ALIGN_FEW
    return launch_status();
  }
  if (one_launch && numel > 64 * kFewWaves) {
    const int64_t tiles = (numel + 63) >> 6;
    const int64_t groups = (tiles + kFewWaves - 1) / kFewWaves;
    hipLaunchKernelGGL((moe_align_lds_hist_kernel<IdT>), dim3((unsigned)groups),
                       dim3(64 * kFewWaves), 0, st, idp, numel, E, B, nbits, sorted, sorted_len,
                       expert_ids, expert_ids_len, post_pad, fill_pad);
    return launch_status();
  }
  const int threads = E <= 512 ? 1024 : 512;
  hipLaunchKernelGGL((moe_align_kernel<IdT>), dim3(1), dim3(threads), 0, st, idp, numel, E, B,
                     nbits, sorted, sorted_len, expert_ids, expert_ids_len, post_pad, fill_pad);
  return launch_status();
}

// ---------------------------------------------------------------------------
// Scratch of the entry point that allocates nothing.  `scratch` is a host-side
// stand-in for the device array, not a device address: host code goes through
// the address hipGetSymbolAddress returns for the current device, fetched once
// per device (every GPU holds its own copy of the array at its own address).
// ---------------------------------------------------------------------------
constexpr int64_t kStaticScratchInts = SARATHI_MOE_ALIGN_STATIC_SCRATCH_BYTES / 4;
static __device__ __align__(256) int32_t scratch[kStaticScratchInts];

constexpr int kMaxDevices = 64;
static std::atomic<int32_t*> g_scratch_ptr[kMaxDevices];

// Device address of `scratch` on the current device, or null with *status set.
static int32_t* static_scratch(int* status) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
    *status = SARATHI_ERR_LAUNCH;
    return nullptr;
  }
  int32_t* p = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (p == nullptr) {
    void* sym = nullptr;
    if (hipGetSymbolAddress(&sym, HIP_SYMBOL(scratch)) != hipSuccess || sym == nullptr) {
      (void)hipGetLastError();
      *status = SARATHI_ERR_LAUNCH;
      return nullptr;
    }
    p = reinterpret_cast<int32_t*>(sym);
    // two threads racing here fetch the same address for the same device
    g_scratch_ptr[dev].store(p, std::memory_order_release);
  }
  return p;
}

}  // namespace sarathi_hip

extern "C" int64_t sarathi_moe_align_workspace_bytes(int64_t numel, int num_experts) {
  using namespace sarathi_hip;
  if (numel <= kMultiThreshold || num_experts <= 0 || num_experts > kAlignMaxExperts) return 0;
  if (numel <= kOneLaunchMaxIds && num_experts <= kHistMaxExperts) return 0;  // one-launch kernels
  return align_workspace_ints(plan_chunks(numel).num_chunks, num_experts) * 4;
}

extern "C" int sarathi_moe_align_block_size(const void* topk_ids, int id_dtype, int64_t numel,
                                            int num_experts, int block_size,
                                            int32_t* sorted_token_ids, int64_t sorted_len,
                                            int32_t* expert_ids, int64_t expert_ids_len,
                                            int32_t* num_tokens_post_pad, int fill_pad,
                                            void* workspace, int64_t workspace_bytes,
                                            void* stream) {
  using namespace sarathi_hip;
  if (!num_tokens_post_pad) return SARATHI_ERR_INVALID_ARG;
  // empty output buffers (no ids and block_size 1) legitimately come with null pointers
  if ((sorted_len > 0 && !sorted_token_ids) || (expert_ids_len > 0 && !expert_ids))
    return SARATHI_ERR_INVALID_ARG;
  if (numel < 0 || (numel > 0 && !topk_ids) || num_experts <= 0 || block_size <= 0 ||
      sorted_len < 0 || expert_ids_len < 0 || workspace_bytes < 0)
    return SARATHI_ERR_INVALID_ARG;
  if (num_experts > kAlignMaxExperts) return SARATHI_ERR_UNSUPPORTED;
  // worst case of num_tokens_post_pad: every non-empty expert wastes block_size - 1 slots
  const int64_t nonempty_max = numel < num_experts ? numel : num_experts;
  const int64_t worst = numel + nonempty_max * ((int64_t)block_size - 1);
  if (worst > 0x7fffffffLL) return SARATHI_ERR_UNSUPPORTED;
  if (sorted_len < worst || expert_ids_len * (int64_t)block_size < worst)
    return SARATHI_ERR_INVALID_ARG;
  hipStream_t st = (hipStream_t)stream;
#define SK_ALIGN(T)                                                                      \
  return launch_align<T>(topk_ids, numel, num_experts, block_size, sorted_token_ids,     \
                         sorted_len, expert_ids, expert_ids_len, num_tokens_post_pad,    \
                         fill_pad, workspace, workspace_bytes, st)
  switch (id_dtype) {
    case SARATHI_IDTYPE_U8: SK_ALIGN(uint8_t);
    case SARATHI_IDTYPE_I8: SK_ALIGN(int8_t);
    case SARATHI_IDTYPE_I16: SK_ALIGN(int16_t);
    case SARATHI_IDTYPE_I32: SK_ALIGN(int32_t);
    case SARATHI_IDTYPE_I64: SK_ALIGN(int64_t);
    default: return SARATHI_ERR_UNSUPPORTED;
  }
#undef SK_ALIGN
}

extern "C" int sarathi_moe_align_block_size_static(const void* topk_ids, int id_dtype,
                                                   int64_t numel, int num_experts,
                                                   int block_size, int32_t* sorted_token_ids,
                                                   int64_t sorted_len, int32_t* expert_ids,
                                                   int64_t expert_ids_len,
                                                   int32_t* num_tokens_post_pad, int fill_pad,
                                                   void* stream) {
  using namespace sarathi_hip;
  // 0 for inputs that take one of the one-launch paths, which use no global scratch
  const int64_t need = sarathi_moe_align_workspace_bytes(numel, num_experts);
  if (need > SARATHI_MOE_ALIGN_STATIC_SCRATCH_BYTES) return SARATHI_ERR_SCRATCH_LIMIT;
  int32_t* ws = nullptr;
  if (need > 0) {
    int status = SARATHI_OK;
    ws = static_scratch(&status);
    if (ws == nullptr) return status;
  }
  // every word of the scratch that the scan and scatter kernels read is written by the count
  // and scan kernels of the same call, so nothing has to be cleared between calls
  return sarathi_moe_align_block_size(topk_ids, id_dtype, numel, num_experts, block_size,
                                      sorted_token_ids, sorted_len, expert_ids, expert_ids_len,
                                      num_tokens_post_pad, fill_pad, ws, need, stream);
}
