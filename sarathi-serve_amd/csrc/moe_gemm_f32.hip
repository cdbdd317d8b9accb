// Grouped expert GEMM for float32 tensors.
//
// The reference's fused_experts admits float32 activations and weights
// (sarathi/model_executor/layers/fused_moe/fused_moe.py:430).  Its Triton kernel then multiplies the
// float32 operands, accumulates in float32, converts the accumulator to `compute_type` and stores
// it (fused_moe.py:121-148), and the launcher passes compute_type = float16 for every dtype but
// bfloat16 (fused_moe.py:466): a float32 GEMM output is rounded through float16 on its way to the
// float32 tensor.  This kernel does the same: exact float32 products on the matrix cores
// (v_mfma_f32_32x32x2_f32), float32 accumulation, optional routing weight, one rounding to float16,
// stored as float32.
//
// Not a tuned path (no reference model runs its experts in float32): a workgroup of four waves
// owns 32 slots x 128 output columns, wave w the 32 columns from 32 w on; both operands pass
// through LDS in K-steps of 32 (rows padded to 36 floats), the next K-step's global loads are in
// flight while the current one is multiplied.  Any block size that is a multiple of 32 works: a
// block is swept as block_m / 32 independent tiles.  Row-major weights only; the gated-SiLU
// epilogue of the 16-bit kernels does not exist here (fused_experts runs silu_and_mul on its own).
#include "moe_gemm_common.h"
#include "launch.h"

namespace sarathi_hip {

constexpr int kF32TileM = 32;    // slots per workgroup
constexpr int kF32TileN = 128;   // output columns per workgroup
constexpr int kF32BK = 32;       // K elements per step
constexpr int kF32Pitch = 36;    // floats per LDS row (16-byte aligned, rows spread over the banks)

typedef float f32x4 __attribute__((ext_vector_type(4)));

struct MoeGemmF32Args {
  const float* a;            // [tokens, K]
  const float* b;            // [E, N, K]
  float* c;                  // [tokens * top_k, N]
  const float* topk_weights;
  const int32_t* sorted_token_ids;
  const int32_t* expert_ids;
  const int32_t* num_tokens_post_padded;
  int64_t a_row_stride, b_expert_stride, c_row_stride;  // elements
  int32_t num_valid, em, N, K, top_k, block_m;
};

template <bool MUL_WEIGHT>
__global__ __launch_bounds__(256) void moe_gemm_f32_kernel(MoeGemmF32Args g) {
  __shared__ __attribute__((aligned(16))) float tok_lds[kF32TileM * kF32Pitch];
  __shared__ __attribute__((aligned(16))) float wgt_lds[kF32TileN * kF32Pitch];
  const int slot0 = blockIdx.y * kF32TileM;
  if (slot0 >= *g.num_tokens_post_padded) return;
  const int expert = g.expert_ids[slot0 / g.block_m];
  const int n0 = blockIdx.x * kF32TileN;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l32 = lane & 31, grp = lane >> 5;

  // global -> registers -> LDS: thread t moves floats [4 (t & 7), 4 (t & 7) + 4) of rows (t >> 3) + 32 j
  const int row = tid >> 3, kq = (tid & 7) * 4;
  const int slot_index = slot0 + row;
  const int sid_in = slot_index < g.em ? g.sorted_token_ids[slot_index] : g.num_valid;
  const bool a_valid = sid_in < g.num_valid;
  if (__syncthreads_count(a_valid) == 0) return;  // a tile of padding only
  const float* a_ptr = g.a + (a_valid ? (int64_t)(sid_in / g.top_k) * g.a_row_stride : 0) + kq;
  const float* b_base = g.b + (int64_t)expert * g.b_expert_stride + kq;
  const float* b_ptr[4];
  bool b_valid[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int n = n0 + row + 32 * j;
    b_valid[j] = n < g.N;
    b_ptr[j] = b_base + (int64_t)(b_valid[j] ? n : 0) * g.K;
  }
  const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
  f32x4 ra, rb[4];
  auto load_step = [&](int k0) {
    const bool k_ok = k0 + kq < g.K;  // K is a multiple of 4
    ra = a_valid && k_ok ? *reinterpret_cast<const f32x4*>(a_ptr + k0) : zero;
#pragma unroll
    for (int j = 0; j < 4; ++j)
      rb[j] = b_valid[j] && k_ok ? *reinterpret_cast<const f32x4*>(b_ptr[j] + k0) : zero;
  };
  auto store_step = [&]() {
    *reinterpret_cast<f32x4*>(&tok_lds[row * kF32Pitch + kq]) = ra;
#pragma unroll
    for (int j = 0; j < 4; ++j)
      *reinterpret_cast<f32x4*>(&wgt_lds[(row + 32 * j) * kF32Pitch + kq]) = rb[j];
  };

  f32x16 acc;
#pragma unroll
  for (int i = 0; i < 16; ++i) acc[i] = 0.f;
  // weights are the MFMA "A" operand (lane: column l32 of this wave, k = grp), tokens the "B"
  // operand (lane: slot l32, k = grp): a lane ends up with 4 x 4 consecutive columns of one slot
  const float* w_row = &wgt_lds[(wave * 32 + l32) * kF32Pitch + grp];
  const float* t_row = &tok_lds[l32 * kF32Pitch + grp];

  load_step(0);
  for (int k0 = 0; k0 < g.K; k0 += kF32BK) {
    store_step();
    __syncthreads();
    if (k0 + kF32BK < g.K) load_step(k0 + kF32BK);
#pragma unroll
    for (int s = 0; s < kF32BK / 2; ++s)
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(w_row[2 * s], t_row[2 * s], acc, 0, 0, 0);
    __syncthreads();
  }

  const int out_index = slot0 + l32;
  const int sid = out_index < g.em ? g.sorted_token_ids[out_index] : g.num_valid;
  if (sid >= g.num_valid) return;
  float scale = 1.f;
  if constexpr (MUL_WEIGHT) scale = g.topk_weights[sid];
  float* crow = g.c + (int64_t)sid * g.c_row_stride;
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const int n = n0 + wave * 32 + q * 8 + grp * 4;
    float v[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      float x = acc[q * 4 + e];
      if constexpr (MUL_WEIGHT) x *= scale;
      v[e] = (float)(_Float16)x;  // the reference's accumulator.to(float16) before the store
    }
    if (n + 3 < g.N) {
      *reinterpret_cast<f32x4*>(crow + n) = f32x4{v[0], v[1], v[2], v[3]};
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (n + e < g.N) crow[n + e] = v[e];
    }
  }
}

// Entry used by sarathi_moe_grouped_gemm for dtype float32.
int launch_moe_gemm_f32(const void* a, const void* b, void* c, const float* topk_weights,
                        const int32_t* sorted_token_ids, const int32_t* expert_ids,
                        const int32_t* num_tokens_post_padded, int64_t num_valid_tokens,
                        int64_t sorted_len, int64_t n, int64_t k, int64_t a_row_stride,
                        int64_t b_expert_stride, int64_t c_row_stride, int block_m, int top_k,
                        int epilogue, int b_layout, hipStream_t st) {
  if (b_layout != SARATHI_MOE_B_ROW_MAJOR || epilogue == SARATHI_MOE_EPILOGUE_SILU_AND_MUL)
    return SARATHI_ERR_UNSUPPORTED;
  if (block_m <= 0 || block_m % kF32TileM != 0) return SARATHI_ERR_UNSUPPORTED;
  // 16-byte operand pieces and output pieces
  if (k % 4 != 0 || a_row_stride % 4 != 0 || b_expert_stride % 4 != 0 || c_row_stride % 4 != 0 ||
      !aligned16(a) || !aligned16(b) || !aligned16(c))
    return SARATHI_ERR_UNSUPPORTED;
  if (num_valid_tokens > 0x7fffffffLL || sorted_len > 0x7fffffffLL || n > 0x7fffffffLL ||
      k > 0x7fffffffLL)
    return SARATHI_ERR_UNSUPPORTED;
  if (sorted_len == 0 || num_valid_tokens == 0) return SARATHI_OK;
  const int64_t tiles = (sorted_len + kF32TileM - 1) / kF32TileM;
  const int64_t n_blocks = (n + kF32TileN - 1) / kF32TileN;
  if (tiles > kMaxGridY || n_blocks > 0x7fffffffLL) return SARATHI_ERR_UNSUPPORTED;
  MoeGemmF32Args g;
  g.a = static_cast<const float*>(a);
  g.b = static_cast<const float*>(b);
  g.c = static_cast<float*>(c);
  g.topk_weights = topk_weights;
  g.sorted_token_ids = sorted_token_ids;
  g.expert_ids = expert_ids;
  g.num_tokens_post_padded = num_tokens_post_padded;
  g.a_row_stride = a_row_stride;
  g.b_expert_stride = b_expert_stride;
  g.c_row_stride = c_row_stride;
  g.num_valid = (int32_t)num_valid_tokens;
  g.em = (int32_t)sorted_len;
  g.N = (int32_t)n;
  g.K = (int32_t)k;
  g.top_k = top_k;
  g.block_m = block_m;
  const dim3 grid((unsigned)n_blocks, (unsigned)tiles);
  if (epilogue == SARATHI_MOE_EPILOGUE_ROUTED_WEIGHT)
    hipLaunchKernelGGL(moe_gemm_f32_kernel<true>, grid, dim3(256), 0, st, g);
  else
    hipLaunchKernelGGL(moe_gemm_f32_kernel<false>, grid, dim3(256), 0, st, g);
  return launch_status();
}

}  // namespace sarathi_hip
