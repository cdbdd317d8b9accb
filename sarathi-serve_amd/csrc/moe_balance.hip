// Even fill of an expert's slot blocks, for the grouped expert GEMM.
//
// moe_align_block_size (sarathi/model_executor/layers/fused_moe/fused_moe.py:151-204 of the
// reference) fills an expert's blocks greedily: with 1064 slots and blocks of 256 an expert gets
// four full blocks and a fifth with 40 slots.  In the grouped GEMM a block is a tile of work; the
// tile of a nearly empty block still pulls its whole weight tile but computes almost nothing, ends
// early, and from then on the workgroups that share weight and token tiles in L2 run out of step
// (measured on the Mixtral layer: 3.4x instead of 1.6x the operand bytes over the fabric, 8-10 %
// of the GEMM time).  This kernel rewrites the sorted ids so that an expert's slots are spread
// evenly over the same blocks, in units of the GEMM's 32-slot tile: the expert's ceil(cnt / 32)
// tiles are dealt to its blocks as evenly as they go (the first blocks take the odd ones), in
// unchanged slot order, and the rest of every block is padding (the GEMM kernels skip 32-slot tiles
// that hold only padding, wherever they are).  An expert with 1030 slots gets 224 / 224 / 224 /
// 192 / 166 (7 / 7 / 7 / 6 / 6 tiles) instead of 256 / 256 / 256 / 256 / 6.  Same blocks per expert, same order of an
// expert's slots, expert_ids and num_tokens_post_padded unchanged; the GEMM's results are bit for
// bit the same (a slot's dot products do not depend on where in a block the slot sits).  No
// counterpart in the reference; fused_experts applies it to its own, internal copy of the sort.
//
// A GEMM workgroup whose waves split the block's slots between them (two wave rows of 128 slots at
// 256-slot blocks) is done when its fuller row is: a block of 224 slots laid out from its start is
// 4 + 3 tiles and costs as much as a full one.  With rows_per_block = R the deal is over the
// expert's nb * R row ranges of block / R slots, each filled from its own start: 1030 slots over
// 5 blocks x 2 rows are 4 4 | 4 3 | 3 3 | 3 3 | 3 3 tiles, 17 tile times instead of 20 (16 if the
// expert had 1024 slots).
#include "vec16.h"
#include "launch.h"

namespace sarathi_hip {

// One workgroup per expert (blockIdx.x < num_experts) plus one that fills the entries at and
// beyond num_tokens_post_padded with the padding value.
__global__ __launch_bounds__(256) void moe_balance_blocks_kernel(
    const int32_t* __restrict__ sorted_in, int32_t* __restrict__ sorted_out,
    const int32_t* __restrict__ expert_ids, const int32_t* __restrict__ post_pad,
    int64_t sorted_len, int num_experts, int block, int pad_value, int granule, int rows) {
  __shared__ int first_blk, last_blk, valid_last;
  const int tid = threadIdx.x;
  int64_t end = *post_pad;
  if (end > sorted_len) end = sorted_len;
  const int nblk_total = (int)(end / block);
  if ((int)blockIdx.x == num_experts) {
    for (int64_t i = end + tid; i < sorted_len; i += 256) sorted_out[i] = pad_value;
    return;
  }
  const int e = blockIdx.x;
  if (tid == 0) {
    first_blk = nblk_total;
    last_blk = -1;
    valid_last = 0;
  }
  __syncthreads();
  int lo = nblk_total, hi = -1;
  for (int b = tid; b < nblk_total; b += 256)
    if (expert_ids[b] == e) {
      lo = b < lo ? b : lo;
      hi = b > hi ? b : hi;
    }
  if (hi >= 0) {
    atomicMin(&first_blk, lo);
    atomicMax(&last_blk, hi);
  }
  __syncthreads();
  const int b0 = first_blk, b1 = last_blk;
  if (b1 < 0) return;  // the expert has no block (uniform)
  const int nb = b1 - b0 + 1;
  const int64_t base = (int64_t)b0 * block;
  // all blocks but the last are full in moe_align_block_size's layout
  int c = 0;
  for (int i = tid; i < block; i += 256) c += sorted_in[(int64_t)b1 * block + i] != pad_value;
  if (c) atomicAdd(&valid_last, c);
  __syncthreads();
  const int cnt = (nb - 1) * block + valid_last;
  // the expert's slots in whole tiles of `granule`, dealt to the row ranges of its blocks as evenly
  // as they go: the first `extra` ranges take one tile more than the others
  const int range = block / rows, ranges = nb * rows;
  const int tiles = (cnt + granule - 1) / granule;
  const int base_tiles = tiles / ranges, extra = tiles - base_tiles * ranges;
  for (int i = tid; i < nb * block; i += 256) {
    const int j = i / range, off = i - j * range;
    const int mine = (base_tiles + (j < extra ? 1 : 0)) * granule;            // slots of range j
    const int before = (j * base_tiles + (j < extra ? j : extra)) * granule;  // slots of ranges < j
    const int r = before + off;
    sorted_out[base + i] = (off < mine && r < cnt) ? sorted_in[base + r] : pad_value;
  }
}

// The two remedies for a partly filled last block, chosen per expert (256-slot blocks, the
// four-wave kernel with riders).  An expert whose last block holds at most as many 32-slot tiles
// as it has full blocks keeps the greedy layout and gets riders: tile j of the last block goes
// along with the expert's j-th block, and the last block is skipped.  Any other expert gets the
// even fill over the two 128-slot wave rows of each of its blocks and no riders.  Same
// workgroup layout as the kernel above: one per expert plus one for the tail of both outputs.
// `ride` as moe_gemm_rider.hip reads it: -2 skip the block, >= 0 first slot of the tile that
// rides with this block, -1 neither.
__global__ __launch_bounds__(256) void moe_plan_blocks_kernel(
    const int32_t* __restrict__ sorted_in, int32_t* __restrict__ sorted_out,
    const int32_t* __restrict__ expert_ids, const int32_t* __restrict__ post_pad,
    int64_t sorted_len, int num_experts, int pad_value, int32_t* __restrict__ ride,
    int ride_len) {
  constexpr int block = 256, granule = 32, rows = 2;
  __shared__ int first_blk, last_blk, valid_last;
  const int tid = threadIdx.x;
  int64_t end = *post_pad;
  if (end > sorted_len) end = sorted_len;
  const int nblk_total = (int)(end / block);
  if ((int)blockIdx.x == num_experts) {
    for (int64_t i = end + tid; i < sorted_len; i += 256) sorted_out[i] = pad_value;
    for (int b = nblk_total + tid; b < ride_len; b += 256) ride[b] = -1;
    return;
  }
  const int e = blockIdx.x;
  if (tid == 0) {
    first_blk = nblk_total;
    last_blk = -1;
    valid_last = 0;
  }
  __syncthreads();
  int lo = nblk_total, hi = -1;
  for (int b = tid; b < nblk_total; b += 256)
    if (expert_ids[b] == e) {
      lo = b < lo ? b : lo;
      hi = b > hi ? b : hi;
    }
  if (hi >= 0) {
    atomicMin(&first_blk, lo);
    atomicMax(&last_blk, hi);
  }
  __syncthreads();
  const int b0 = first_blk, b1 = last_blk;
  if (b1 < 0) return;  // the expert has no block (uniform)
  const int nb = b1 - b0 + 1;
  const int64_t base = (int64_t)b0 * block;
  int c = 0;  // ids are 0 .. pad_value - 1, padding is pad_value
  for (int i = tid; i < block; i += 256)
    c += (uint32_t)sorted_in[(int64_t)b1 * block + i] < (uint32_t)pad_value;
  if (c) atomicAdd(&valid_last, c);
  __syncthreads();
  const int tiles_last = (valid_last + granule - 1) / granule;
  if (nb > 1 && tiles_last <= nb - 1) {  // riders, greedy layout kept
    for (int i = tid; i < nb * block; i += 256) sorted_out[base + i] = sorted_in[base + i];
    for (int b = tid; b < nb; b += 256)
      ride[b0 + b] = b == nb - 1 ? -2 : b < tiles_last ? b1 * block + granule * b : -1;
    return;
  }
  for (int b = tid; b < nb; b += 256) ride[b0 + b] = -1;
  const int cnt = (nb - 1) * block + valid_last;
  const int range = block / rows, ranges = nb * rows;
  const int tiles = (cnt + granule - 1) / granule;
  const int base_tiles = tiles / ranges, extra = tiles - base_tiles * ranges;
  for (int i = tid; i < nb * block; i += 256) {
    const int j = i / range, off = i - j * range;
    const int mine = (base_tiles + (j < extra ? 1 : 0)) * granule;
    const int before = (j * base_tiles + (j < extra ? j : extra)) * granule;
    const int r = before + off;
    sorted_out[base + i] = (off < mine && r < cnt) ? sorted_in[base + r] : pad_value;
  }
}

}  // namespace sarathi_hip

extern "C" int sarathi_moe_plan_blocks(const int32_t* sorted_in, int32_t* sorted_out,
                                       const int32_t* expert_ids,
                                       const int32_t* num_tokens_post_pad, int64_t sorted_len,
                                       int num_experts, int block_m, int pad_value,
                                       int32_t* riders, int64_t riders_len, void* stream) {
  using namespace sarathi_hip;
  if (sorted_len < 0 || num_experts <= 0 || block_m <= 0 || riders_len < 0)
    return SARATHI_ERR_INVALID_ARG;
  if (block_m != 256) return SARATHI_ERR_UNSUPPORTED;
  if (riders_len < (sorted_len + block_m - 1) / block_m) return SARATHI_ERR_INVALID_ARG;
  if (sorted_len == 0) return SARATHI_OK;
  if (!sorted_in || !sorted_out || !expert_ids || !num_tokens_post_pad || !riders ||
      sorted_in == sorted_out)
    return SARATHI_ERR_INVALID_ARG;
  if (num_experts > 1024 || sorted_len > 0x7fffffffLL || riders_len > 0x7fffffffLL)
    return SARATHI_ERR_UNSUPPORTED;
  hipLaunchKernelGGL(moe_plan_blocks_kernel, dim3((unsigned)num_experts + 1), dim3(256), 0,
                     (hipStream_t)stream, sorted_in, sorted_out, expert_ids, num_tokens_post_pad,
                     sorted_len, num_experts, pad_value, riders, (int)riders_len);
  return launch_status();
}

extern "C" int sarathi_moe_balance_blocks(const int32_t* sorted_in, int32_t* sorted_out,
                                          const int32_t* expert_ids,
                                          const int32_t* num_tokens_post_pad, int64_t sorted_len,
                                          int num_experts, int block_size, int pad_value,
                                          int granule, int rows_per_block, void* stream) {
  using namespace sarathi_hip;
  if (sorted_len < 0 || num_experts <= 0 || block_size <= 0 || granule <= 0 || rows_per_block <= 0 ||
      block_size % rows_per_block != 0 || (block_size / rows_per_block) % granule != 0)
    return SARATHI_ERR_INVALID_ARG;
  if (sorted_len == 0) return SARATHI_OK;
  if (!sorted_in || !sorted_out || !expert_ids || !num_tokens_post_pad || sorted_in == sorted_out)
    return SARATHI_ERR_INVALID_ARG;
  if (num_experts > 1024 || sorted_len > 0x7fffffffLL) return SARATHI_ERR_UNSUPPORTED;
  hipLaunchKernelGGL(moe_balance_blocks_kernel, dim3((unsigned)num_experts + 1), dim3(256), 0,
                     (hipStream_t)stream, sorted_in, sorted_out, expert_ids, num_tokens_post_pad,
                     sorted_len, num_experts, block_size, pad_value, granule, rows_per_block);
  return launch_status();
}
