// Device-side pieces of moe_align_block_size shared by the stand-alone kernels (moe_align.hip)
// and the fused routing kernel (moe_fused_routing.hip).
#pragma once

#include "vec16.h"
#include "../../include/sarathi_ops.h"

namespace sarathi_hip {

constexpr int kAlignMaxExperts = SARATHI_MOE_MAX_EXPERTS;  // 1024
constexpr int kAlignCntInts = 8192;                        // W * E <= 8192
constexpr int kAlignBatch = 8;                             // tiles loaded ahead per wave

struct TileMatch {
  int rank;   // lanes below this one holding the same expert
  int count;  // lanes holding the same expert
};

// Bit-serial match: after the loop `peers` has a bit for every valid lane of
// the wave whose expert id equals this lane's.
SK_DEV TileMatch match_expert(int e, bool valid, int nbits) {
  unsigned long long peers = __ballot(valid);
  for (int b = 0; b < nbits; ++b) {
    const bool bit = (e >> b) & 1;
    const unsigned long long bal = __ballot(valid && bit);
    peers &= bit ? bal : ~bal;
  }
  const unsigned long long below = (1ull << (threadIdx.x & 63)) - 1ull;
  TileMatch m;
  m.rank = __popcll(peers & below);
  m.count = __popcll(peers);
  return m;
}

// Ids are fetched with raw buffer loads from a resource that covers the wave's part of the array:
// positions past the end return 0 from the hardware range check and are discarded afterwards by
// position, so no load sits under a per-lane condition.  (A plain load under one,
// `i < numel ? ids[i] : -1`, compiles to a branch around the load with a wait for it right
// behind -- the optimiser does the same to an unconditional load that feeds only one arm of a
// select -- so a batch of such loads runs one after the other, 0.15 us each from L2, instead of
// all being in flight together.)  COHERENT: the ids were written by other workgroups of the same
// launch; the load is marked sc1 so that it does not hit in this compute unit's own cache.
template <typename IdT, bool COHERENT = false> SK_DEV IdT buf_load_id(rsrc_t r, uint32_t byte_off) {
  constexpr int kPolicy = COHERENT ? 16 : 0;
  if constexpr (sizeof(IdT) == 1) return (IdT)__builtin_amdgcn_raw_buffer_load_b8(r, byte_off, 0, kPolicy);
  else if constexpr (sizeof(IdT) == 2) return (IdT)__builtin_amdgcn_raw_buffer_load_b16(r, byte_off, 0, kPolicy);
  else if constexpr (sizeof(IdT) == 4) return (IdT)__builtin_amdgcn_raw_buffer_load_b32(r, byte_off, 0, kPolicy);
  else {
    const u32x2 v = __builtin_amdgcn_raw_buffer_load_b64(r, byte_off, 0, kPolicy);
    return (IdT)(((uint64_t)v.y << 32) | v.x);
  }
}
// Resource over ids[first, numel), at most 4 GiB - 1 of it (callers stay far below that).
template <typename IdT> SK_DEV rsrc_t id_rsrc(const IdT* ids, int64_t first, int64_t numel) {
  const int64_t left = first < numel ? (numel - first) * (int64_t)sizeof(IdT) : 0;
  return make_rsrc(ids + (first < numel ? first : 0), left < 0xffffffffLL ? (uint32_t)left : 0xffffffffu);
}

// ids outside [0, E) become -1 (skipped); done in 64 bits so wide ids cannot wrap into range
template <typename IdT> SK_DEV int checked_expert(IdT raw, int E) {
  const int64_t v = (int64_t)raw;
  return (v >= 0 && v < E) ? (int)v : -1;
}

// The whole sort by one workgroup of W = blockDim.x / 64 waves (a power of two, at most 16).
// LDS: cnt[W * E] (tokens of expert e in wave w's chunk, indexed [e][w]), tot[E] (tokens per
// expert), cumsum[E + 1] (padded exclusive scan).
// COHERENT: the ids were written by other workgroups of the same launch (as device-scope atomics,
// completed before this workgroup was chosen); read them with device-scope loads, which do not
// hit in this compute unit's own cache.
template <typename IdT, bool COHERENT = false>
SK_DEV void align_single_workgroup(const IdT* __restrict__ ids, int64_t numel, int E, int B, int nbits,
                                   int32_t* __restrict__ sorted, int64_t sorted_len,
                                   int32_t* __restrict__ expert_ids, int64_t expert_ids_len,
                                   int32_t* __restrict__ post_pad, int fill_pad, int32_t* cnt,
                                   int32_t* tot, int32_t* cumsum) {

  const int tid = threadIdx.x;
  const int nthr = blockDim.x;
  const int W = nthr >> 6;  // 16 or 8: a power of two
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // uniform, and the compiler knows it
  const int lane = tid & 63;

  for (int i = tid; i < W * E; i += nthr) cnt[i] = 0;
  __syncthreads();

  // chunk of this wave: whole tiles, ascending
  const int64_t tiles_total = (numel + 63) >> 6;
  const int64_t tiles_per_wave = (tiles_total + W - 1) / W;
  const int64_t tile_lo = wave * tiles_per_wave;
  int64_t tile_hi = tile_lo + tiles_per_wave;
  if (tile_hi > tiles_total) tile_hi = tiles_total;
  // small inputs: the wave's whole chunk stays in registers between the two passes
  const bool resident = tiles_per_wave <= kAlignBatch;

  const rsrc_t rid = id_rsrc(ids, tile_lo << 6, numel);  // this wave's chunk
  auto load_batch = [&](int64_t t0, int (&e)[kAlignBatch]) {
#pragma unroll
    for (int u = 0; u < kAlignBatch; ++u) {
      const int64_t i = ((t0 + u) << 6) + lane;
      const IdT raw = buf_load_id<IdT, COHERENT>(
          rid, (uint32_t)((((t0 + u - tile_lo) << 6) + lane) * (int64_t)sizeof(IdT)));
      e[u] = (t0 + u < tile_hi && i < numel) ? checked_expert(raw, E) : -1;
    }
  };
  // cnt is indexed [e * W + wave]; only this wave touches its column, so plain LDS adds suffice
  // the matches of a batch are kept (`mt`) so that a resident chunk need not be matched again
  // in the scatter pass
  auto count_batch = [&](int64_t t0, const int (&e)[kAlignBatch], TileMatch (&mt)[kAlignBatch]) {
#pragma unroll
    for (int u = 0; u < kAlignBatch; ++u) {
      if (t0 + u < tile_hi) {  // wave-uniform
        const bool valid = e[u] >= 0;
        mt[u] = match_expert(e[u], valid, nbits);
        if (valid && mt[u].rank == 0) atomicAdd(&cnt[e[u] * W + wave], mt[u].count);
      }
    }
  };
  auto scatter_batch = [&](int64_t t0, const int (&e)[kAlignBatch],
                           const TileMatch (&mt)[kAlignBatch], bool have_matches) {
#pragma unroll
    for (int u = 0; u < kAlignBatch; ++u) {
      if (t0 + u < tile_hi) {
        const bool valid = e[u] >= 0;
        const TileMatch m = have_matches ? mt[u] : match_expert(e[u], valid, nbits);
        if (valid) {
          int32_t* c = &cnt[e[u] * W + wave];
          const int base = *c;  // every lane of the group reads before the leader's add below
          const int64_t slot = (int64_t)cumsum[e[u]] + base + m.rank;
          if (slot < sorted_len) sorted[slot] = (int32_t)(((t0 + u) << 6) + lane);
          if (m.rank == 0) atomicAdd(c, m.count);
        }
      }
    }
  };

  // ---- 1. count
  int held[kAlignBatch];
  TileMatch held_match[kAlignBatch];
  if (resident) {
    load_batch(tile_lo, held);
    count_batch(tile_lo, held, held_match);
  } else {
    for (int64_t t0 = tile_lo; t0 < tile_hi; t0 += kAlignBatch) {
      int e[kAlignBatch];
      TileMatch scratch[kAlignBatch];
      load_batch(t0, e);
      count_batch(t0, e, scratch);
    }
  }
  __syncthreads();

  // ---- 2. exclusive scan over the W waves of every expert: W consecutive lanes own one expert
  for (int i = tid; i < W * E; i += nthr) {
    const int w = i & (W - 1);
    const int c = cnt[i];
    int x = c;
#pragma unroll
    for (int off = 1; off < 16; off <<= 1) {
      const int y = __shfl_up(x, off, 16);
      if (off < W && w >= off) x += y;
    }
    cnt[i] = x - c;
    if (w == W - 1) tot[i / W] = x;
  }
  __syncthreads();
  // padded prefix over the experts
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

  // ---- 3. scatter
  if (resident) {
    scatter_batch(tile_lo, held, held_match, true);
  } else {
    for (int64_t t0 = tile_lo; t0 < tile_hi; t0 += kAlignBatch) {
      int e[kAlignBatch];
      load_batch(t0, e);
      scatter_batch(t0, e, held_match, false);
    }
  }

  // ---- 4. expert id of every block, padding slots
  const int total = cumsum[E];
  const int nblk = total / B;
  for (int b = tid; b < nblk; b += nthr) {
    if (b < expert_ids_len) {
      const int pos = b * B;
      int lo = 0, hi = E;  // invariant: cumsum[lo] <= pos < cumsum[hi]
      while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (cumsum[mid] <= pos) lo = mid; else hi = mid;
      }
      expert_ids[b] = lo;
    }
  }
  if (fill_pad) {
    const int32_t pad = (int32_t)numel;
    // an expert's run ends with fewer than B padding slots
    for (int64_t i = tid; i < (int64_t)E * B; i += nthr) {
      const int x = (int)(i / B), j = (int)(i - (int64_t)x * B);
      const int64_t slot = (int64_t)cumsum[x] + tot[x] + j;
      if (slot < cumsum[x + 1]) sorted[slot] = pad;
    }
    for (int64_t i = (int64_t)total + tid; i < sorted_len; i += nthr) sorted[i] = pad;
  }
}

}  // namespace sarathi_hip
