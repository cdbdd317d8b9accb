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
//
// gelu_new / gelu_fast cost about 30 vector instructions per element (nine roundings to the tensor
// dtype), which bounds the streaming kernel at 0.51-0.56 of the HBM rate.  On a 16-bit dtype the
// op is a function of 65536 bit patterns, so large tensors go through a table instead: a kernel
// evaluates the same arithmetic once for every pattern (128 KiB per op and dtype, kept in a
// file-scope device array and built on the first large call on a device), and a persistent kernel
// (one 1024-thread workgroup per compute unit, the table copied into LDS) turns every element into
// one 2-byte LDS read: two vector instructions per element, same bits as the arithmetic path
// (measured at [2304, 14336] bf16: 27.4 -> 23.9 us, 0.60 -> 0.69 of the HBM rate).
#include <atomic>
#include <mutex>
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

// ---- 16-bit dtypes, large tensors: the op as a table over all 65536 bit patterns -------------

constexpr int kTableThreads = 1024;
constexpr uint32_t kTableBytes = 65536u * 2u;
// below this many elements the arithmetic kernel is as fast or faster (the persistent kernel pays
// its launch and 128 KiB of table per compute unit before the first element; measured on bf16
// rows of 14336: 7.3 M elements 7.5 against 8.2 us, 11 M 10.5 / 10.6, 14.7 M 13.1 / 12.6,
// 33 M 27.4 / 23.9, 66 M 53.5 / 44.4)
#ifndef SARATHI_GELU_TABLE_MIN_ELEMS
#define SARATHI_GELU_TABLE_MIN_ELEMS (int64_t(12) << 20)
#endif
constexpr int64_t kTableMinElems = SARATHI_GELU_TABLE_MIN_ELEMS;
constexpr int kTableKinds = 4;  // (gelu_new, gelu_fast) x (f16, bf16)
static __device__ __align__(256) uint16_t gelu_tables[kTableKinds][65536];

template <int DT, bool FAST>
__global__ __launch_bounds__(kTableThreads) void gelu_table_build_kernel(uint16_t* __restrict__ table) {
  const uint32_t bits = blockIdx.x * kTableThreads + threadIdx.x;
  Vec<DT> x;
  x.unpack(u32x4{bits, 0u, 0u, 0u});
  const float r = FAST ? gelu_fast_elem<DT>(x.f[0]) : gelu_new_elem<DT>(x.f[0]);
  table[bits] = (uint16_t)(pack2<DT>(r, r) & 0xffffu);
}

// One workgroup per compute unit.  The first vector of every lane is requested before the table
// is copied into LDS, and the next one while the current one is looked up (two, four or six
// vectors in flight per lane measured 5-8 % slower at 33 M and 66 M elements: the lookups, not
// the loads, set the pace).
__global__ __launch_bounds__(kTableThreads) void gelu_table_kernel(
    void* __restrict__ out, const void* __restrict__ in, const uint16_t* __restrict__ table,
    uint32_t vec_bytes, uint32_t vecs) {
  extern __shared__ uint16_t lds_table[];
  const rsrc_t ri = make_rsrc(in, vec_bytes), ro = make_rsrc(out, vec_bytes);
  const uint32_t stride = gridDim.x * kTableThreads;
  uint32_t i = blockIdx.x * kTableThreads + threadIdx.x;
  u32x4 next = buf_load16<kStreamLoad>(ri, i * 16u);  // beyond vec_bytes: zeros, never stored
  {
    const u32x4* src = reinterpret_cast<const u32x4*>(table);
    u32x4* dst = reinterpret_cast<u32x4*>(lds_table);
    u32x4 t[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) t[j] = src[j * kTableThreads + threadIdx.x];
#pragma unroll
    for (int j = 0; j < 8; ++j) dst[j * kTableThreads + threadIdx.x] = t[j];
  }
  __syncthreads();
  for (; i < vecs; i += stride) {
    const u32x4 cur = next;
    next = buf_load16<kStreamLoad>(ri, (i + stride) * 16u);
    u32x4 r;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const uint32_t w = cur[j];
      r[j] = (uint32_t)lds_table[w & 0xffffu] | ((uint32_t)lds_table[w >> 16] << 16);
    }
    buf_store16<kStreamStore>(ro, i * 16u, r);
  }
}

// Per device and table: 0 = not built, 1 = build launched on `stream`, `built` recorded behind it,
// 2 = the build has completed.  A call may read the table when it is complete, or when the call's
// own stream is the one the build was launched on (stream order).  Nothing here waits.
struct GeluTableState {
  std::mutex lock;
  int phase = 0;
  hipStream_t stream = nullptr;
  hipEvent_t built = nullptr;
  uint16_t* table = nullptr;
  bool lds_raised = false;
};
constexpr int kMaxTableDevices = 64;
static GeluTableState g_gelu_table_state[kMaxTableDevices][kTableKinds];

// The device address of the table for (DT, FAST) if this call on `st` may use it, else null (the
// caller then runs the arithmetic kernel).  Launches the build on the first call.
template <int DT, bool FAST>
static const uint16_t* gelu_table_for(hipStream_t st) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxTableDevices) {
    (void)hipGetLastError();
    return nullptr;
  }
  constexpr int kind = (FAST ? 1 : 0) * 2 + (DT == kBF16 ? 1 : 0);
  GeluTableState& s = g_gelu_table_state[dev][kind];
  std::lock_guard<std::mutex> guard(s.lock);
  if (s.phase == 2) return s.table;
  // a stream under capture records launches for later: only a finished table is safe there
  hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(st, &capturing) != hipSuccess || capturing != hipStreamCaptureStatusNone) {
    (void)hipGetLastError();
    return nullptr;
  }
  if (s.phase == 1) {
    if (hipEventQuery(s.built) == hipSuccess) {
      s.phase = 2;
      return s.table;
    }
    (void)hipGetLastError();  // hipErrorNotReady
    return st == s.stream ? s.table : nullptr;
  }
  // first call on this device: address of this device's copy of the array, LDS limit, build
  void* sym = nullptr;
  if (hipGetSymbolAddress(&sym, HIP_SYMBOL(gelu_tables)) != hipSuccess || sym == nullptr ||
      hipFuncSetAttribute(reinterpret_cast<const void*>(gelu_table_kernel),
                          hipFuncAttributeMaxDynamicSharedMemorySize, (int)kTableBytes) != hipSuccess ||
      hipEventCreateWithFlags(&s.built, hipEventDisableTiming) != hipSuccess) {
    (void)hipGetLastError();
    return nullptr;
  }
  s.table = reinterpret_cast<uint16_t*>(sym) + (size_t)kind * 65536;
  hipLaunchKernelGGL((gelu_table_build_kernel<DT, FAST>), dim3(65536 / kTableThreads),
                     dim3(kTableThreads), 0, st, s.table);
  if (hipGetLastError() != hipSuccess || hipEventRecord(s.built, st) != hipSuccess) {
    (void)hipGetLastError();
    (void)hipEventDestroy(s.built);
    s.built = nullptr;
    return nullptr;
  }
  s.stream = st;
  s.phase = 1;
  return s.table;
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
  if constexpr (DT != kF32) {
    // (vecs + 2 * grid * 1024) * 16 must stay below 2^32: tensors up to 2 GiB
    if (numel >= kTableMinElems && vec_bytes <= (int64_t(1) << 31)) {
      if (const uint16_t* table = gelu_table_for<DT, FAST>(st)) {
        const uint32_t vecs = (uint32_t)(vec_bytes / 16);
        hipLaunchKernelGGL(gelu_table_kernel, dim3((unsigned)compute_units()), dim3(kTableThreads),
                           kTableBytes, st, out, in, table, (uint32_t)vec_bytes, vecs);
        if (numel % N != 0) {  // the elements past the last whole vector
          const int64_t done = numel / N * N;
          hipLaunchKernelGGL((gelu_scalar_kernel<DT, FAST>), dim3(1), dim3(kActBlock), 0, st,
                             reinterpret_cast<char*>(out) + done * ElemBytes<DT>::value,
                             reinterpret_cast<const char*>(in) + done * ElemBytes<DT>::value,
                             numel - done);
        }
        return launch_status();
      }
    }
  }
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
