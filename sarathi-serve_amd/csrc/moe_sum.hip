// Sum of a token's top-k expert outputs for gfx950: out[t, :] = sum_j in[t, j, :].
//
// The last step of the reference's fused_experts
// (sarathi/model_executor/layers/fused_moe/fused_moe.py:539-543: torch.sum over dim 1 of the
// [tokens, top_k, hidden] output of the down projection, into the result tensor): fp32
// accumulation over j in ascending order, one rounding to the tensor dtype.  A streaming op like
// silu_and_mul.  Rows of up to 8 KiB with top_k 1 or 2 (Mixtral) take moe_sum_rows_kernel: ONE wave
// per R consecutive tokens, all top_k * 8 * R loads issued before the first add, rows as buffer
// resources, a one-dimensional grid.  Fewer, fatter one-wave workgroups are what the memory
// system rewards at these sizes (a launch of N one-wave workgroups costs the dispatcher 0.2 ns
// each, and more bytes in flight per wave hide more of the ramp): the [2304, 1, 4096] case, a
// plain copy, takes 9.5 us as 18432 one-segment workgroups and 6.4-7.1 us as 768-2304 row waves.
// Everything else takes the general kernel: one 64-lane workgroup per 1 KiB segment of an output
// row, top_k 16-byte loads and one 16-byte store per lane.
#include "vec16.h"
#include "launch.h"

namespace sarathi_hip {

constexpr int kSumSeg = 64;    // lanes per workgroup of the streaming kernel
constexpr int kSumBlock = 256;  // element-wise fallback

template <int DT>
__global__ __launch_bounds__(kSumSeg) void moe_sum_kernel(
    void* __restrict__ out, const void* __restrict__ in, uint32_t row_bytes, int top_k,
    int64_t in_token_stride_bytes, int64_t in_k_stride_bytes, int64_t out_stride_bytes) {
  constexpr int N = VecElems<DT>::value;
  const int64_t row = (int64_t)blockIdx.z * kMaxGridY + blockIdx.y;
  const char* tok = reinterpret_cast<const char*>(in) + row * in_token_stride_bytes;
  const uint32_t off = (blockIdx.x * kSumSeg + threadIdx.x) * 16u;
  Vec<DT> acc, x;
  acc.unpack(buf_load16<kStreamLoad>(make_rsrc(tok, row_bytes), off));
  for (int j = 1; j < top_k; ++j) {
    x.unpack(buf_load16<kStreamLoad>(make_rsrc(tok + j * in_k_stride_bytes, row_bytes), off));
#pragma unroll
    for (int i = 0; i < N; ++i) acc.f[i] += x.f[i];
  }
  const rsrc_t ro = make_rsrc(reinterpret_cast<char*>(out) + row * out_stride_bytes, row_bytes);
  buf_store16<kStreamStore>(ro, off, acc.pack());
}

// One wave per R consecutive tokens; a row has at most 64 * VPL vectors; TOPK is 1 or 2.
template <int DT, int TOPK, int VPL, int R>
__global__ __launch_bounds__(kSumSeg) void moe_sum_rows_kernel(
    void* __restrict__ out, const void* __restrict__ in, uint32_t row_bytes,
    int64_t in_token_stride_bytes, int64_t in_k_stride_bytes, int64_t out_stride_bytes,
    int64_t num_rows) {
  constexpr int N = VecElems<DT>::value;
  const int64_t row0 = (int64_t)blockIdx.x * R;
  const uint32_t off0 = threadIdx.x * 16u;
  u32x4 v[R][TOPK][VPL];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const uint32_t live = row0 + r < num_rows ? row_bytes : 0u;  // rows past the end: no traffic
    const char* tok = reinterpret_cast<const char*>(in) + (row0 + r) * in_token_stride_bytes;
#pragma unroll
    for (int j = 0; j < TOPK; ++j) {
      const rsrc_t ri = make_rsrc(tok + j * in_k_stride_bytes, live);
#pragma unroll
      for (int u = 0; u < VPL; ++u) v[r][j][u] = buf_load16<kStreamLoad>(ri, off0 + u * 1024u);
    }
  }
  // every load is issued before the first wait (left alone, the scheduler starts storing after
  // ten loads and issues the rest one by one)
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const uint32_t live = row0 + r < num_rows ? row_bytes : 0u;
    const rsrc_t ro =
        make_rsrc(reinterpret_cast<char*>(out) + (row0 + r) * out_stride_bytes, live);
#pragma unroll
    for (int u = 0; u < VPL; ++u) {
      Vec<DT> acc;
      acc.unpack(v[r][0][u]);
      if constexpr (TOPK == 2) {
        Vec<DT> x;
        x.unpack(v[r][1][u]);
#pragma unroll
        for (int i = 0; i < N; ++i) acc.f[i] += x.f[i];
      }
      buf_store16<kStreamStore>(ro, off0 + u * 1024u, acc.pack());
    }
  }
}

template <int DT>
__global__ __launch_bounds__(kSumBlock) void moe_sum_generic_kernel(
    void* __restrict__ out, const void* __restrict__ in, int64_t hidden, int top_k,
    int64_t in_token_stride, int64_t in_k_stride, int64_t out_stride) {
  const int64_t row = blockIdx.x;
  for (int64_t i = threadIdx.x; i < hidden; i += kSumBlock) {
    float acc = load_elem<DT>(in, row * in_token_stride + i);
    for (int j = 1; j < top_k; ++j) acc += load_elem<DT>(in, row * in_token_stride + j * in_k_stride + i);
    store_elem<DT>(out, row * out_stride + i, acc);
  }
}

template <int DT>
static int launch_moe_sum(void* out, const void* in, int64_t T, int top_k, int64_t hidden,
                          int64_t in_token_stride, int64_t in_k_stride, int64_t out_stride,
                          hipStream_t st) {
  constexpr int N = VecElems<DT>::value;
  constexpr int EB = ElemBytes<DT>::value;
  const bool vec_ok = (hidden % N == 0) && (in_token_stride % N == 0) && (in_k_stride % N == 0) &&
                      (out_stride % N == 0) && aligned16(out) && aligned16(in) &&
                      hidden * EB <= 0x7fffffffLL;
  if (T > 0x7fffffffLL) return SARATHI_ERR_UNSUPPORTED;
  if (!vec_ok) {
    hipLaunchKernelGGL((moe_sum_generic_kernel<DT>), dim3((unsigned)T), dim3(kSumBlock), 0, st, out,
                       in, hidden, top_k, in_token_stride, in_k_stride, out_stride);
    return launch_status();
  }
  const int64_t segs = (hidden / N + kSumSeg - 1) / kSumSeg;
  if (segs <= 8 && top_k <= 2) {
    // whole rows per wave; two or three tokens per wave where that divides evenly over the
    // compute units (top-2: at most two, to stay inside the register file)
    const int rows = pick_rows_per_workgroup(T, top_k == 1 ? 3 : 2);
    const dim3 grid((unsigned)((T + rows - 1) / rows));
    const uint32_t row_bytes = (uint32_t)(hidden * EB);
#define SK_SUM_ROWS(TOPK, VPL, R)                                                              \
  hipLaunchKernelGGL((moe_sum_rows_kernel<DT, TOPK, VPL, R>), grid, dim3(kSumSeg), 0, st, out, \
                     in, row_bytes, in_token_stride * EB, in_k_stride * EB, out_stride * EB, T)
#define SK_SUM_VPL(TOPK, R)                     \
  do {                                          \
    if (segs <= 2) SK_SUM_ROWS(TOPK, 2, R);     \
    else if (segs <= 4) SK_SUM_ROWS(TOPK, 4, R); \
    else SK_SUM_ROWS(TOPK, 8, R);               \
  } while (0)
    if (top_k == 1) {
      if (rows == 3) SK_SUM_VPL(1, 3);
      else if (rows == 2) SK_SUM_VPL(1, 2);
      else SK_SUM_VPL(1, 1);
    } else {
      if (rows == 2) SK_SUM_VPL(2, 2);
      else SK_SUM_VPL(2, 1);
    }
#undef SK_SUM_VPL
#undef SK_SUM_ROWS
    return launch_status();
  }
  // rows above 65535 spill into grid.z; the last z-slice may run past T, so launch it apart
  const int64_t full_z = T / kMaxGridY, rem = T % kMaxGridY;
  const char* inb = reinterpret_cast<const char*>(in);
  char* outb = reinterpret_cast<char*>(out);
  if (full_z > 0) {
    hipLaunchKernelGGL((moe_sum_kernel<DT>), dim3((unsigned)segs, kMaxGridY, (unsigned)full_z),
                       dim3(kSumSeg), 0, st, out, in, (uint32_t)(hidden * EB), top_k,
                       in_token_stride * EB, in_k_stride * EB, out_stride * EB);
  }
  if (rem > 0) {
    const int64_t r0 = full_z * kMaxGridY;
    hipLaunchKernelGGL((moe_sum_kernel<DT>), dim3((unsigned)segs, (unsigned)rem, 1), dim3(kSumSeg), 0,
                       st, outb + r0 * out_stride * EB, inb + r0 * in_token_stride * EB,
                       (uint32_t)(hidden * EB), top_k, in_token_stride * EB, in_k_stride * EB,
                       out_stride * EB);
  }
  return launch_status();
}

}  // namespace sarathi_hip

extern "C" int sarathi_moe_sum(void* out, const void* input, int64_t num_tokens, int64_t top_k,
                               int64_t hidden, int64_t in_token_stride, int64_t in_k_stride,
                               int64_t out_row_stride, int dtype, void* stream) {
  using namespace sarathi_hip;
  if (num_tokens < 0 || top_k <= 0 || hidden < 0) return SARATHI_ERR_INVALID_ARG;
  if (num_tokens == 0 || hidden == 0) return SARATHI_OK;
  if (!out || !input || in_k_stride < hidden || in_token_stride < hidden || out_row_stride < hidden)
    return SARATHI_ERR_INVALID_ARG;
  if (top_k > SARATHI_MOE_MAX_EXPERTS) return SARATHI_ERR_UNSUPPORTED;
  hipStream_t st = (hipStream_t)stream;
  switch (dtype) {
    case kF32: return launch_moe_sum<kF32>(out, input, num_tokens, (int)top_k, hidden, in_token_stride, in_k_stride, out_row_stride, st);
    case kF16: return launch_moe_sum<kF16>(out, input, num_tokens, (int)top_k, hidden, in_token_stride, in_k_stride, out_row_stride, st);
    case kBF16: return launch_moe_sum<kBF16>(out, input, num_tokens, (int)top_k, hidden, in_token_stride, in_k_stride, out_row_stride, st);
    default: return SARATHI_ERR_UNSUPPORTED;
  }
}
