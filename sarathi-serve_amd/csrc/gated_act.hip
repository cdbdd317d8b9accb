// silu_and_mul, gelu_new and gelu_fast for gfx950.
//
// Replaces csrc/activation_kernels.cu:8-114 of the reference (one block per
// token, 2-byte __ldg loads, a per-thread loop over the row).  These are pure
// streaming ops, so the whole design is about bytes in flight: a thread owns
// one 16-byte column slot of ROWS consecutive token rows, issues all of its
// 16-byte loads before the first use, and writes 16-byte stores.  A block is
// 256 lanes wide (4 KiB contiguous per row segment), the grid is
// (row groups) x (column chunks), i.e. thousands of blocks for 256 CUs.
//
// Arithmetic, rounding points as in the reference (fp32 math, T = tensor dtype):
//   silu_and_mul: out = T( f32(T( x / (1 + exp(-x)) )) * y )
//   gelu_new / gelu_fast: the mixed T / fp32 sequences of
//   csrc/activation_kernels.cu:86-98.
// exp and the reciprocal use the hardware v_exp_f32 / v_rcp_f32 (1 ulp each);
// after the rounding to a 16-bit dtype that is far inside the 1e-2 tolerance.
#include "vec16.h"
#include "launch.h"

namespace sarathi_hip {

constexpr int kActBlock = 256;

SK_DEV float silu_f32(float x) {
  // x * sigmoid(x) = x / (1 + 2^(-x * log2 e))
  float e = __builtin_amdgcn_exp2f(x * -1.4426950408889634f);
  return x * __builtin_amdgcn_rcpf(1.0f + e);
}

// tanh(u) = 1 - 2 / (1 + e^{2u}); the clamp keeps e^{2u} finite
SK_DEV float tanh_f32(float u) {
  float c = u < -15.f ? -15.f : (u > 15.f ? 15.f : u);  // NaN passes through
  float e = __builtin_amdgcn_exp2f(c * 2.8853900817779268f);
  return 1.0f - 2.0f * __builtin_amdgcn_rcpf(1.0f + e);
}

// ---- silu_and_mul ------------------------------------------------------------

template <int DT, int ROWS>
__global__ __launch_bounds__(kActBlock) void silu_and_mul_kernel(
    void* __restrict__ out, const void* __restrict__ in, int64_t num_tokens, int nvec_d,
    int64_t in_stride_vec, int64_t out_stride_vec) {
  constexpr int N = VecElems<DT>::value;
  const int col = blockIdx.y * kActBlock + threadIdx.x;
  if (col >= nvec_d) return;
  const int64_t row0 = (int64_t)blockIdx.x * ROWS;

  u32x4 xr[ROWS], yr[ROWS];
#pragma unroll
  for (int r = 0; r < ROWS; ++r) {
    const int64_t row = row0 + r;
    if (row < num_tokens) {
      xr[r] = load16_stream(in, row * in_stride_vec + col);
      yr[r] = load16_stream(in, row * in_stride_vec + nvec_d + col);
    }
  }
#pragma unroll
  for (int r = 0; r < ROWS; ++r) {
    const int64_t row = row0 + r;
    if (row < num_tokens) {
      Vec<DT> x, y;
      x.unpack(xr[r]);
      y.unpack(yr[r]);
#pragma unroll
      for (int i = 0; i < N; ++i) x.f[i] = rnd<DT>(silu_f32(x.f[i])) * y.f[i];
      store16_stream(out, row * out_stride_vec + col, x.pack());
    }
  }
}

template <int DT>
__global__ __launch_bounds__(kActBlock) void silu_and_mul_generic_kernel(
    void* __restrict__ out, const void* __restrict__ in, int64_t d, int64_t in_stride,
    int64_t out_stride) {
  const int64_t row = blockIdx.x;
  for (int64_t i = threadIdx.x; i < d; i += kActBlock) {
    float x = load_elem<DT>(in, row * in_stride + i);
    float y = load_elem<DT>(in, row * in_stride + d + i);
    store_elem<DT>(out, row * out_stride + i, rnd<DT>(silu_f32(x)) * y);
  }
}

template <int DT>
static int launch_silu(void* out, const void* in, int64_t T, int64_t d, int64_t in_stride,
                       int64_t out_stride, hipStream_t st) {
  constexpr int N = VecElems<DT>::value;
  constexpr int ROWS = 4;
  const bool vec_ok = (d % N == 0) && (in_stride % N == 0) && (out_stride % N == 0) &&
                      aligned16(out) && aligned16(in);
  if (T > 0x7fffffffLL) return SARATHI_ERR_UNSUPPORTED;
  if (!vec_ok) {
    hipLaunchKernelGGL((silu_and_mul_generic_kernel<DT>), dim3((unsigned)T), dim3(kActBlock), 0,
                       st, out, in, d, in_stride, out_stride);
    return launch_status();
  }
  const int64_t nvec_d = d / N;
  const int64_t chunks = (nvec_d + kActBlock - 1) / kActBlock;
  if (chunks > 65535) return SARATHI_ERR_UNSUPPORTED;
  dim3 grid((unsigned)((T + ROWS - 1) / ROWS), (unsigned)chunks);
  hipLaunchKernelGGL((silu_and_mul_kernel<DT, ROWS>), grid, dim3(kActBlock), 0, st, out, in, T,
                     (int)nvec_d, in_stride / N, out_stride / N);
  return launch_status();
}

// ---- gelu_new / gelu_fast ----------------------------------------------------

template <int DT> SK_DEV float gelu_new_elem(float x) {
  float x3 = rnd<DT>(rnd<DT>(x * x) * x);
  float a = rnd<DT>(0.044715f * x3);
  float b = rnd<DT>(x + a);
  float c = rnd<DT>(0.79788456f * b);
  float t = rnd<DT>(tanh_f32(c));
  return rnd<DT>(0.5f * x) * rnd<DT>(1.0f + t);
}
template <int DT> SK_DEV float gelu_fast_elem(float x) {
  float a = rnd<DT>(x * 0.79788456f);
  float b = rnd<DT>(0.044715f * x);
  float c = rnd<DT>(b * x);
  float e = rnd<DT>(1.0f + c);
  float u = rnd<DT>(a * e);
  float t = rnd<DT>(tanh_f32(u));
  return rnd<DT>(0.5f * x) * rnd<DT>(1.0f + t);
}

// Flat element-wise kernel over n16 16-byte vectors plus a scalar tail.
template <int DT, bool FAST, int UNROLL>
__global__ __launch_bounds__(kActBlock) void gelu_kernel(void* __restrict__ out,
                                                         const void* __restrict__ in,
                                                         int64_t n16, int64_t numel) {
  constexpr int N = VecElems<DT>::value;
  const int64_t base = ((int64_t)blockIdx.x * UNROLL) * kActBlock + threadIdx.x;
  u32x4 raw[UNROLL];
#pragma unroll
  for (int u = 0; u < UNROLL; ++u) {
    int64_t v = base + (int64_t)u * kActBlock;
    if (v < n16) raw[u] = load16_stream(in, v);
  }
#pragma unroll
  for (int u = 0; u < UNROLL; ++u) {
    int64_t v = base + (int64_t)u * kActBlock;
    if (v < n16) {
      Vec<DT> x;
      x.unpack(raw[u]);
#pragma unroll
      for (int i = 0; i < N; ++i)
        x.f[i] = FAST ? gelu_fast_elem<DT>(x.f[i]) : gelu_new_elem<DT>(x.f[i]);
      store16_stream(out, v, x.pack());
    }
  }
  // tail elements (numel not a multiple of the vector width): first block only
  if (blockIdx.x == 0) {
    int64_t i = n16 * N + threadIdx.x;
    if (i < numel) {
      float x = load_elem<DT>(in, i);
      store_elem<DT>(out, i, FAST ? gelu_fast_elem<DT>(x) : gelu_new_elem<DT>(x));
    }
  }
}

// Base pointers that are not 16-byte aligned: one element per lane.
template <int DT, bool FAST>
__global__ __launch_bounds__(kActBlock) void gelu_scalar_kernel(void* __restrict__ out,
                                                                const void* __restrict__ in,
                                                                int64_t numel) {
  const int64_t i = (int64_t)blockIdx.x * kActBlock + threadIdx.x;
  if (i < numel) {
    float x = load_elem<DT>(in, i);
    store_elem<DT>(out, i, FAST ? gelu_fast_elem<DT>(x) : gelu_new_elem<DT>(x));
  }
}

template <int DT, bool FAST>
static int launch_gelu(void* out, const void* in, int64_t numel, hipStream_t st) {
  constexpr int N = VecElems<DT>::value;
  constexpr int UNROLL = 4;
  if (!(aligned16(out) && aligned16(in))) {
    int64_t blocks = (numel + kActBlock - 1) / kActBlock;
    if (blocks > 0x7fffffffLL) return SARATHI_ERR_UNSUPPORTED;
    hipLaunchKernelGGL((gelu_scalar_kernel<DT, FAST>), dim3((unsigned)blocks), dim3(kActBlock), 0,
                       st, out, in, numel);
    return launch_status();
  }
  const int64_t n16 = numel / N;
  int64_t blocks = (n16 + (int64_t)UNROLL * kActBlock - 1) / ((int64_t)UNROLL * kActBlock);
  if (blocks < 1) blocks = 1;
  if (blocks > 0x7fffffffLL) return SARATHI_ERR_UNSUPPORTED;
  hipLaunchKernelGGL((gelu_kernel<DT, FAST, UNROLL>), dim3((unsigned)blocks), dim3(kActBlock), 0,
                     st, out, in, n16, numel);
  return launch_status();
}

template <bool FAST>
static int dispatch_gelu(void* out, const void* in, int64_t T, int64_t d, int dtype,
                         void* stream) {
  if (!out || !in) return SARATHI_ERR_INVALID_ARG;
  if (T < 0 || d <= 0) return SARATHI_ERR_INVALID_ARG;
  if (T == 0) return SARATHI_OK;
  hipStream_t st = (hipStream_t)stream;
  const int64_t numel = T * d;
  switch (dtype) {
    case kBF16: return launch_gelu<kBF16, FAST>(out, in, numel, st);
    case kF16: return launch_gelu<kF16, FAST>(out, in, numel, st);
    case kF32: return launch_gelu<kF32, FAST>(out, in, numel, st);
    default: return SARATHI_ERR_UNSUPPORTED;
  }
}

}  // namespace sarathi_hip

extern "C" int sarathi_silu_and_mul(void* out, const void* input, int64_t num_tokens, int64_t d,
                                    int64_t input_row_stride, int64_t out_row_stride, int dtype,
                                    void* stream) {
  using namespace sarathi_hip;
  if (!out || !input) return SARATHI_ERR_INVALID_ARG;
  if (num_tokens < 0 || d <= 0 || input_row_stride < 2 * d || out_row_stride < d)
    return SARATHI_ERR_INVALID_ARG;
  if (num_tokens == 0) return SARATHI_OK;
  hipStream_t st = (hipStream_t)stream;
  switch (dtype) {
    case kBF16:
      return launch_silu<kBF16>(out, input, num_tokens, d, input_row_stride, out_row_stride, st);
    case kF16:
      return launch_silu<kF16>(out, input, num_tokens, d, input_row_stride, out_row_stride, st);
    case kF32:
      return launch_silu<kF32>(out, input, num_tokens, d, input_row_stride, out_row_stride, st);
    default: return SARATHI_ERR_UNSUPPORTED;
  }
}

extern "C" int sarathi_gelu_new(void* out, const void* input, int64_t num_tokens, int64_t d,
                                int dtype, void* stream) {
  return sarathi_hip::dispatch_gelu<false>(out, input, num_tokens, d, dtype, stream);
}

extern "C" int sarathi_gelu_fast(void* out, const void* input, int64_t num_tokens, int64_t d,
                                 int dtype, void* stream) {
  return sarathi_hip::dispatch_gelu<true>(out, input, num_tokens, d, dtype, stream);
}
