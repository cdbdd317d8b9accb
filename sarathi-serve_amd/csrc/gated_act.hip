// silu_and_mul, gelu_new and gelu_fast for gfx950.
//
// Replaces csrc/activation_kernels.cu:8-114 of the reference (one block per
// token, 2-byte __ldg loads, a per-thread loop over the row).  These are pure
// streaming ops.  What measured fastest on MI355X is the opposite of a fat
// persistent kernel: one 64-lane workgroup per 1 KiB segment of a row, every
// lane doing exactly one 16-byte load per input stream and one 16-byte store,
// with workgroup ids running along the row first and then down the rows, so
// that the workgroups in flight at any moment sweep memory linearly (the same
// kernel with row-major workgroup order is ~12 % slower, and every extra vector
// per lane costs a few percent).  Row bases live in scalar registers as buffer
// resources; ragged row ends are clipped by the hardware range check.
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

constexpr int kActBlock = 256;   // element-wise fallback kernels
constexpr int kRowSeg = 64;      // lanes per workgroup of the streaming kernels

// tanh(u) = 1 - 2 / (1 + e^{2u}).  No clamp is needed: for large u the exponential is +inf, whose
// reciprocal is 0 (result 1); for very negative u it is 0 (result -1); NaN passes through.
SK_DEV float tanh_f32(float u) {
  float e = __builtin_amdgcn_exp2f(u * 2.8853900817779268f);
  return 1.0f - 2.0f * __builtin_amdgcn_rcpf(1.0f + e);
}

// ---- silu_and_mul ------------------------------------------------------------

template <int DT>
__global__ __launch_bounds__(kRowSeg) void silu_and_mul_kernel(
    void* __restrict__ out, const void* __restrict__ in, uint32_t half_row_bytes,
    int64_t in_stride_bytes, int64_t out_stride_bytes) {
  constexpr int N = VecElems<DT>::value;
  const int64_t row = (int64_t)blockIdx.z * kMaxGridY + blockIdx.y;
  const rsrc_t rx = make_rsrc(reinterpret_cast<const char*>(in) + row * in_stride_bytes,
                              half_row_bytes);
  const rsrc_t ry = make_rsrc(
      reinterpret_cast<const char*>(in) + row * in_stride_bytes + half_row_bytes, half_row_bytes);
  const rsrc_t ro = make_rsrc(reinterpret_cast<char*>(out) + row * out_stride_bytes,
                              half_row_bytes);
  const uint32_t off = (blockIdx.x * kRowSeg + threadIdx.x) * 16u;
  Vec<DT> x, y;
  x.unpack(buf_load16<kStreamLoad>(rx, off));
  y.unpack(buf_load16<kStreamLoad>(ry, off));
#pragma unroll
  for (int i = 0; i < N; ++i) x.f[i] = rnd<DT>(silu_f32(x.f[i])) * y.f[i];
  buf_store16<kStreamStore>(ro, off, x.pack());
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
  constexpr int EB = ElemBytes<DT>::value;
  const bool vec_ok = (d % N == 0) && (in_stride % N == 0) && (out_stride % N == 0) &&
                      aligned16(out) && aligned16(in) && d * EB <= 0x7fffffffLL;
  if (T > 0x7fffffffLL) return SARATHI_ERR_UNSUPPORTED;
  if (!vec_ok) {
    hipLaunchKernelGGL((silu_and_mul_generic_kernel<DT>), dim3((unsigned)T), dim3(kActBlock), 0,
                       st, out, in, d, in_stride, out_stride);
    return launch_status();
  }
  const int64_t nvec_d = d / N;
  const int64_t segs = (nvec_d + kRowSeg - 1) / kRowSeg;
  // rows above 65535 spill into grid.z; the last z-slice may run past T, so launch it apart
  const int64_t full_z = T / kMaxGridY, rem = T % kMaxGridY;
  const char* inb = reinterpret_cast<const char*>(in);
  char* outb = reinterpret_cast<char*>(out);
  if (full_z > 0) {
    hipLaunchKernelGGL((silu_and_mul_kernel<DT>), dim3((unsigned)segs, kMaxGridY, (unsigned)full_z),
                       dim3(kRowSeg), 0, st, out, in, (uint32_t)(d * EB), in_stride * EB,
                       out_stride * EB);
  }
  if (rem > 0) {
    const int64_t r0 = full_z * kMaxGridY;
    hipLaunchKernelGGL((silu_and_mul_kernel<DT>), dim3((unsigned)segs, (unsigned)rem, 1),
                       dim3(kRowSeg), 0, st, outb + r0 * out_stride * EB,
                       inb + r0 * in_stride * EB, (uint32_t)(d * EB), in_stride * EB,
                       out_stride * EB);
  }
  return launch_status();
}

// ---- gelu_new / gelu_fast ----------------------------------------------------

// Two elements at a time, so that every rounding to a 16-bit dtype is one packed conversion for
// the pair (these kernels are bound by their instruction count: nine roundings per element).
template <int DT> SK_DEV f32x2 gelu_new_pair(float x0, float x1) {
  f32x2 q = rnd2<DT>(x0 * x0, x1 * x1);
  const f32x2 x3 = rnd2<DT>(q.x * x0, q.y * x1);
  const f32x2 a = rnd2<DT>(0.044715f * x3.x, 0.044715f * x3.y);
  const f32x2 b = rnd2<DT>(x0 + a.x, x1 + a.y);
  const f32x2 c = rnd2<DT>(0.79788456f * b.x, 0.79788456f * b.y);
  const f32x2 t = rnd2<DT>(tanh_f32(c.x), tanh_f32(c.y));
  const f32x2 h = rnd2<DT>(0.5f * x0, 0.5f * x1);
  const f32x2 o = rnd2<DT>(1.0f + t.x, 1.0f + t.y);
  f32x2 r = {h.x * o.x, h.y * o.y};
  return r;
}
template <int DT> SK_DEV f32x2 gelu_fast_pair(float x0, float x1) {
  const f32x2 a = rnd2<DT>(x0 * 0.79788456f, x1 * 0.79788456f);
  const f32x2 b = rnd2<DT>(0.044715f * x0, 0.044715f * x1);
  const f32x2 c = rnd2<DT>(b.x * x0, b.y * x1);
  const f32x2 e = rnd2<DT>(1.0f + c.x, 1.0f + c.y);
  const f32x2 u = rnd2<DT>(a.x * e.x, a.y * e.y);
  const f32x2 t = rnd2<DT>(tanh_f32(u.x), tanh_f32(u.y));
  const f32x2 h = rnd2<DT>(0.5f * x0, 0.5f * x1);
  const f32x2 o = rnd2<DT>(1.0f + t.x, 1.0f + t.y);
  f32x2 r = {h.x * o.x, h.y * o.y};
  return r;
}
template <int DT> SK_DEV float gelu_new_elem(float x) { return gelu_new_pair<DT>(x, x).x; }
template <int DT> SK_DEV float gelu_fast_elem(float x) { return gelu_fast_pair<DT>(x, x).x; }

// Flat element-wise kernel: the tensor is cut into spans of kGeluSpan bytes (one
// buffer resource each, grid.y), a workgroup handles 1 KiB of a span.  Elements
// past the last whole vector go through the scalar tail in workgroup (0, 0).
constexpr uint32_t kGeluSpan = 1u << 30;

template <int DT, bool FAST>
__global__ __launch_bounds__(kRowSeg) void gelu_kernel(void* __restrict__ out,
                                                       const void* __restrict__ in,
                                                       int64_t vec_bytes, int64_t numel) {
  constexpr int N = VecElems<DT>::value;
  const int64_t span0 = (int64_t)blockIdx.y * kGeluSpan;
  const int64_t left = vec_bytes - span0;
  const uint32_t span_bytes = left < (int64_t)kGeluSpan ? (uint32_t)left : kGeluSpan;
  const rsrc_t ri = make_rsrc(reinterpret_cast<const char*>(in) + span0, span_bytes);
  const rsrc_t ro = make_rsrc(reinterpret_cast<char*>(out) + span0, span_bytes);
  const uint32_t off = (blockIdx.x * kRowSeg + threadIdx.x) * 16u;
  Vec<DT> x;
  x.unpack(buf_load16<kStreamLoad>(ri, off));
#pragma unroll
  for (int i = 0; i < N; i += 2) {
    const f32x2 r = FAST ? gelu_fast_pair<DT>(x.f[i], x.f[i + 1]) : gelu_new_pair<DT>(x.f[i], x.f[i + 1]);
    x.f[i] = r.x;
    x.f[i + 1] = r.y;
  }
  buf_store16<kStreamStore>(ro, off, x.pack());
  if (blockIdx.x == 0 && blockIdx.y == 0) {
    const int64_t i = vec_bytes / ElemBytes<DT>::value + threadIdx.x;
    if (i < numel) {
      float v = load_elem<DT>(in, i);
      store_elem<DT>(out, i, FAST ? gelu_fast_elem<DT>(v) : gelu_new_elem<DT>(v));
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
  if (!(aligned16(out) && aligned16(in))) {
    int64_t blocks = (numel + kActBlock - 1) / kActBlock;
    if (blocks > 0x7fffffffLL) return SARATHI_ERR_UNSUPPORTED;
    hipLaunchKernelGGL((gelu_scalar_kernel<DT, FAST>), dim3((unsigned)blocks), dim3(kActBlock), 0,
                       st, out, in, numel);
    return launch_status();
  }
  const int64_t vec_bytes = numel / N * 16;
  int64_t spans = (vec_bytes + kGeluSpan - 1) / kGeluSpan;
  if (spans < 1) spans = 1;
  if (spans > kMaxGridY) return SARATHI_ERR_UNSUPPORTED;
  const int64_t first_span = vec_bytes < (int64_t)kGeluSpan ? vec_bytes : (int64_t)kGeluSpan;
  int64_t segs = (first_span / 16 + kRowSeg - 1) / kRowSeg;
  if (segs < 1) segs = 1;
  hipLaunchKernelGGL((gelu_kernel<DT, FAST>), dim3((unsigned)segs, (unsigned)spans), dim3(kRowSeg),
                     0, st, out, in, vec_bytes, numel);
  return launch_status();
}

template <bool FAST>
static int dispatch_gelu(void* out, const void* in, int64_t T, int64_t d, int dtype,
                         void* stream) {
  if (T > 0 && (!out || !in)) return SARATHI_ERR_INVALID_ARG;  // empty tensors have no data
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
  if (num_tokens > 0 && (!out || !input)) return SARATHI_ERR_INVALID_ARG;
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
