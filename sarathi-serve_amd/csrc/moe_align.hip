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
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int chunk = blockIdx.x * kChunkWaves + wave;
  int32_t* my = cnt + wave * E;
  for (int i = lane; i < E; i += 64) my[i] = 0;  // each wave clears and reads only its own row
  const int64_t tiles_total = (numel + 63) >> 6;
  const int64_t tile_lo = chunk * tiles_per_chunk;
  int64_t tile_hi = tile_lo + tiles_per_chunk;
  if (tile_hi > tiles_total) tile_hi = tiles_total;
  for (int64_t t0 = tile_lo; t0 < tile_hi; t0 += kAlignBatch) {
    int e[kAlignBatch];
#pragma unroll
    for (int u = 0; u < kAlignBatch; ++u) {
      const int64_t i = ((t0 + u) << 6) + lane;
      e[u] = (t0 + u < tile_hi && i < numel) ? checked_expert(ids[i], E) : -1;
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
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int chunk = blockIdx.x * kChunkWaves + wave;
  int32_t* my = pos + wave * E;
  for (int i = lane; i < E; i += 64) my[i] = cumsum[i] + hist[(int64_t)i * num_chunks + chunk];
  const int64_t tiles_total = (numel + 63) >> 6;
  const int64_t tile_lo = chunk * tiles_per_chunk;
  int64_t tile_hi = tile_lo + tiles_per_chunk;
  if (tile_hi > tiles_total) tile_hi = tiles_total;
  for (int64_t t0 = tile_lo; t0 < tile_hi; t0 += kAlignBatch) {
    int e[kAlignBatch];
#pragma unroll
    for (int u = 0; u < kAlignBatch; ++u) {
      const int64_t i = ((t0 + u) << 6) + lane;
      e[u] = (t0 + u < tile_hi && i < numel) ? checked_expert(ids[i], E) : -1;
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
  if (numel > kMultiThreshold && workspace != nullptr) {
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
  // 0 for inputs that take the single-workgroup path, which uses no global scratch
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
