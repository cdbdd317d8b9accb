// rms_norm and fused_add_rms_norm for gfx950.
//
// Replaces csrc/layernorm_kernels.cu:11-62 of the reference (one 1024-thread
// block per token, 2-byte loads, the row read twice, a two-level shared-memory
// reduction).  Here one small workgroup owns one token row and keeps it in
// registers: the row is read from HBM exactly once with 16-byte loads that are
// all issued before the first use, and written with 16-byte stores.  Workgroup
// ids walk the rows, i.e. memory, linearly.  How many lanes share a row is
// chosen per shape (see launch_rms): a single wave per row where that fits,
// otherwise 2..16 waves.  The sum of squares is folded inside each wave with
// DPP; the waves of a row combine through one LDS word each and one barrier.
//
// Arithmetic (rounding points as in the reference):
//   ss = sum f32(x)^2 ; s = rsqrt(ss / H + eps)
//   out = T( f32(T(f32(x) * s)) * f32(w) )
// and for the fused op first z = T(f32(x) + f32(r)), residual <- z, x := z.
#include "vec16.h"
#include "launch.h"

namespace sarathi_hip {

// WAVES = waves per row (1, 2, 4, 8 or 16), VPL = 16-byte vectors per lane;
// the row has nvec <= 64 * WAVES * VPL vectors.
template <int DT, int WAVES, int VPL, bool FUSED>
__global__ __launch_bounds__(64 * WAVES) void rms_norm_row_kernel(
    void* out,        // FUSED: the `input` tensor, updated in place
    void* in_or_res,  // FUSED: the residual tensor, updated in place
    const void* __restrict__ weight, float eps, uint32_t row_bytes, float hidden_f,
    int64_t out_stride_bytes, int64_t in_stride_bytes) {
  constexpr int N = VecElems<DT>::value;
  constexpr int TPR = 64 * WAVES;
  __shared__ float partial[WAVES];
  const int64_t row = blockIdx.x;
  const rsrc_t rin = make_rsrc(reinterpret_cast<char*>(in_or_res) + row * in_stride_bytes, row_bytes);
  const rsrc_t rout = make_rsrc(reinterpret_cast<char*>(out) + row * out_stride_bytes, row_bytes);
  const rsrc_t rw = make_rsrc(weight, row_bytes);
  const uint32_t off0 = threadIdx.x * 16u;

  // lanes past the end of the row read zeros and their stores are dropped
  u32x4 raw[VPL];
#pragma unroll
  for (int j = 0; j < VPL; ++j) raw[j] = buf_load16<kStreamLoad>(rin, off0 + j * (TPR * 16u));
  if constexpr (FUSED) {
    u32x4 hid[VPL];
#pragma unroll
    for (int j = 0; j < VPL; ++j) hid[j] = buf_load16<kStreamLoad>(rout, off0 + j * (TPR * 16u));
#pragma unroll
    for (int j = 0; j < VPL; ++j) {
      Vec<DT> a, b;
      a.unpack(raw[j]);
      b.unpack(hid[j]);
#pragma unroll
      for (int i = 0; i < N; ++i) a.f[i] = b.f[i] + a.f[i];
      raw[j] = a.pack();  // z, rounded to the dtype
      buf_store16<kStreamStore>(rin, off0 + j * (TPR * 16u), raw[j]);
    }
  }
  // weight vectors are shared by every row and stay cache resident; fetch them
  // now so their latency overlaps the reduction
  u32x4 wraw[VPL];
#pragma unroll
  for (int j = 0; j < VPL; ++j) wraw[j] = buf_load16<kCached>(rw, off0 + j * (TPR * 16u));

  float ss = 0.f;
#pragma unroll
  for (int j = 0; j < VPL; ++j) {
    Vec<DT> a;
    a.unpack(raw[j]);
#pragma unroll
    for (int i = 0; i < N; ++i) ss = __builtin_fmaf(a.f[i], a.f[i], ss);
  }
  ss = wave64_sum(ss);
  if constexpr (WAVES > 1) {
    if ((threadIdx.x & 63) == 0) partial[threadIdx.x >> 6] = ss;
    lds_barrier();  // the residual stores and weight loads issued above stay in flight
    float t = partial[0];
#pragma unroll
    for (int k = 1; k < WAVES; ++k) t += partial[k];
    ss = t;
  }
  const float s = __builtin_amdgcn_rsqf(ss / hidden_f + eps);

#pragma unroll
  for (int j = 0; j < VPL; ++j) {
    Vec<DT> a, w;
    a.unpack(raw[j]);
    w.unpack(wraw[j]);
#pragma unroll
    for (int i = 0; i < N; ++i) a.f[i] = rnd<DT>(a.f[i] * s) * w.f[i];
    buf_store16<kStreamStore>(rout, off0 + j * (TPR * 16u), a.pack());
  }
}

// R consecutive rows per one-wave workgroup, for rows of up to 64 * VPL vectors.  The weight
// vectors are fetched once for the R rows, the loads of all R rows are issued before the first
// wait, and the rows are then finished one after the other, so row 0 is on its way out while row
// 2 is still arriving.  The launch has R times fewer workgroups, each with R times the bytes in
// flight.  On MI355X at 2304 rows of 4096 bf16 (three rows per workgroup = three workgroups per
// compute unit): fused op 13.8 -> 12.4 us; a plain copy kernel shows the same pattern (2304 waves
// of 8 KiB each 7.1 us, 768 waves of 24 KiB each 6.4 us).  It only pays
// when the workgroups divide evenly over the compute units; pick_rows_per_workgroup() decides.
// Rows at or beyond num_rows get an empty buffer resource: their loads return zeros and their
// stores are dropped.
template <int DT, int VPL, int R, bool FUSED>
__global__ __launch_bounds__(64) void rms_norm_wave_rows_kernel(
    void* out, void* in_or_res, const void* __restrict__ weight, float eps, uint32_t row_bytes,
    float hidden_f, uint32_t out_stride_vecs, uint32_t in_stride_vecs, uint32_t num_rows) {
  // Twelve dwords of arguments: all of them are preloaded into scalar registers at wave launch
  // (the hardware preloads at most 14), so the first load waits for no argument fetch.  With the
  // strides as 64-bit byte counts the row count fell outside and every wave spent about a
  // microsecond on a scalar load before its first row load.  Strides are in 16-byte vectors.
  constexpr int N = VecElems<DT>::value;
  const int64_t out_stride_bytes = (int64_t)out_stride_vecs * 16, in_stride_bytes = (int64_t)in_stride_vecs * 16;
  const int64_t row0 = (int64_t)blockIdx.x * R;
  const rsrc_t rw = make_rsrc(weight, row_bytes);
  const uint32_t off0 = threadIdx.x * 16u;
  u32x4 wraw[VPL];
#pragma unroll
  for (int j = 0; j < VPL; ++j) wraw[j] = buf_load16<kCached>(rw, off0 + j * 1024u);
  rsrc_t rin[R], rout[R];
  u32x4 raw[R][VPL], hid[R][VPL];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const uint32_t live = row0 + r < num_rows ? row_bytes : 0u;
    rin[r] = make_rsrc(reinterpret_cast<char*>(in_or_res) + (row0 + r) * in_stride_bytes, live);
    rout[r] = make_rsrc(reinterpret_cast<char*>(out) + (row0 + r) * out_stride_bytes, live);
#pragma unroll
    for (int j = 0; j < VPL; ++j) raw[r][j] = buf_load16<kStreamLoad>(rin[r], off0 + j * 1024u);
    if constexpr (FUSED) {
#pragma unroll
      for (int j = 0; j < VPL; ++j) hid[r][j] = buf_load16<kStreamLoad>(rout[r], off0 + j * 1024u);
    }
  }
  __builtin_amdgcn_sched_barrier(0);  // every load is issued before the first wait

#pragma unroll
  for (int r = 0; r < R; ++r) {
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < VPL; ++j) {
      Vec<DT> a;
      a.unpack(raw[r][j]);
      if constexpr (FUSED) {
        Vec<DT> b;
        b.unpack(hid[r][j]);
#pragma unroll
        for (int i = 0; i < N; ++i) a.f[i] = b.f[i] + a.f[i];
        raw[r][j] = a.pack();  // z, rounded to the dtype
        buf_store16<kStreamStore>(rin[r], off0 + j * 1024u, raw[r][j]);
        a.unpack(raw[r][j]);
      }
#pragma unroll
      for (int i = 0; i < N; ++i) ss = __builtin_fmaf(a.f[i], a.f[i], ss);
    }
    ss = wave64_sum(ss);
    const float s = __builtin_amdgcn_rsqf(ss / hidden_f + eps);
#pragma unroll
    for (int j = 0; j < VPL; ++j) {
      Vec<DT> a, w;
      a.unpack(raw[r][j]);
      w.unpack(wraw[j]);
#pragma unroll
      for (int i = 0; i < N; i += 2) {
        const f32x2 t = rnd2<DT>(a.f[i] * s, a.f[i + 1] * s);
        a.f[i] = t.x * w.f[i];
        a.f[i + 1] = t.y * w.f[i + 1];
      }
      buf_store16<kStreamStore>(rout[r], off0 + j * 1024u, a.pack());
    }
  }
}

// One wave per row for the fused op, rows of up to 64 * VPL vectors: the x and residual loads of the
// row are all issued before the first wait, z = T(x + r), its sum of squares and the normalised row
// are formed in registers, and only then are the 2 * VPL stores issued, back to back.  Holding the
// stores back keeps a wave from writing while its neighbours on the memory channels are still
// reading: at 2304 rows of 4096 bf16 on MI355X 12.15 us against 13.4 us with the residual stores
// issued as soon as z is known and 12.6 us for three rows per wave, and the grid (one workgroup per
// row) has no row counts it prefers.
template <int DT, int VPL>
__global__ __launch_bounds__(64) void fused_add_rms_norm_wave_kernel(
    void* out, void* res, const void* __restrict__ weight, float eps, uint32_t row_bytes,
    float hidden_f, int64_t out_stride_bytes, int64_t res_stride_bytes) {
  constexpr int N = VecElems<DT>::value;
  const int64_t row = blockIdx.x;
  const rsrc_t rres = make_rsrc(reinterpret_cast<char*>(res) + row * res_stride_bytes, row_bytes);
  const rsrc_t rout = make_rsrc(reinterpret_cast<char*>(out) + row * out_stride_bytes, row_bytes);
  const rsrc_t rw = make_rsrc(weight, row_bytes);
  const uint32_t off0 = threadIdx.x * 16u;
  u32x4 raw[VPL], hid[VPL];
#pragma unroll
  for (int j = 0; j < VPL; ++j) raw[j] = buf_load16<kStreamLoad>(rres, off0 + j * 1024u);
#pragma unroll
  for (int j = 0; j < VPL; ++j) hid[j] = buf_load16<kStreamLoad>(rout, off0 + j * 1024u);
  float ss = 0.f;
#pragma unroll
  for (int j = 0; j < VPL; ++j) {
    Vec<DT> a, b;
    a.unpack(raw[j]);
    b.unpack(hid[j]);
#pragma unroll
    for (int i = 0; i < N; ++i) a.f[i] = b.f[i] + a.f[i];
    raw[j] = a.pack();  // z, rounded to the dtype
    a.unpack(raw[j]);
#pragma unroll
    for (int i = 0; i < N; ++i) ss = __builtin_fmaf(a.f[i], a.f[i], ss);
  }
  ss = wave64_sum(ss);
  const float s = __builtin_amdgcn_rsqf(ss / hidden_f + eps);
#pragma unroll
  for (int j = 0; j < VPL; ++j) {
    Vec<DT> a, w;
    a.unpack(raw[j]);
    // The weight row is cache resident; its loads are written where they are used and left to the
    // compiler to hoist.  Issued in front, together with the row's own loads, they cost the
    // float16 build 0.6 us at 2304 rows of 4096 (14.0 -> 13.4 us; bfloat16, whose weight loads the
    // compiler had already moved behind the reduction, 13.05 either way).
    w.unpack(buf_load16<kCached>(rw, off0 + j * 1024u));
#pragma unroll
    for (int i = 0; i < N; i += 2) {
      const f32x2 t = rnd2<DT>(a.f[i] * s, a.f[i + 1] * s);
      a.f[i] = t.x * w.f[i];
      a.f[i + 1] = t.y * w.f[i + 1];
    }
    hid[j] = a.pack();
  }
  __builtin_amdgcn_sched_barrier(0);  // no store is issued before the last result is formed
#pragma unroll
  for (int j = 0; j < VPL; ++j) buf_store16<kStreamStore>(rres, off0 + j * 1024u, raw[j]);
#pragma unroll
  for (int j = 0; j < VPL; ++j) buf_store16<kStreamStore>(rout, off0 + j * 1024u, hid[j]);
}


// Any shape / alignment: one 256-thread block per row, element-wise accesses,
// the row re-read from cache for the second pass.
template <int DT, bool FUSED>
__global__ __launch_bounds__(256) void rms_norm_generic_kernel(
    void* out, void* in_or_res, const void* __restrict__ weight, float eps, int hidden,
    float hidden_f, int64_t out_stride, int64_t in_stride) {
  __shared__ float partial[4];
  const int64_t row = blockIdx.x;
  const int64_t ib = row * in_stride, ob = row * out_stride;
  float ss = 0.f;
  for (int i = threadIdx.x; i < hidden; i += 256) {
    float x = load_elem<DT>(in_or_res, ib + i);
    if constexpr (FUSED) {
      x = rnd<DT>(load_elem<DT>(out, ob + i) + x);
      store_elem<DT>(in_or_res, ib + i, x);
    }
    ss = __builtin_fmaf(x, x, ss);
  }
  ss = wave64_sum(ss);
  if ((threadIdx.x & 63) == 0) partial[threadIdx.x >> 6] = ss;
  __syncthreads();  // also orders the residual stores above before the re-read below
  ss = (partial[0] + partial[1]) + (partial[2] + partial[3]);
  const float s = __builtin_amdgcn_rsqf(ss / hidden_f + eps);
  for (int i = threadIdx.x; i < hidden; i += 256) {
    float x = load_elem<DT>(in_or_res, ib + i);
    store_elem<DT>(out, ob + i, rnd<DT>(x * s) * load_elem<DT>(weight, i));
  }
}

template <int DT, bool FUSED>
static int launch_rms(void* out, void* in, const void* w, float eps, int64_t T, int64_t H,
                      int64_t out_stride, int64_t in_stride, hipStream_t st) {
  constexpr int N = VecElems<DT>::value;
  constexpr int EB = ElemBytes<DT>::value;
  const float hidden_f = (float)H;
  if (T > 0x7fffffffLL) return SARATHI_ERR_UNSUPPORTED;
  const bool vec_ok = (H % N == 0) && (out_stride % N == 0) && (in_stride % N == 0) &&
                      aligned16(out) && aligned16(in) && aligned16(w) && (H / N) <= 1024 * 4;
  if (!vec_ok) {
    hipLaunchKernelGGL((rms_norm_generic_kernel<DT, FUSED>), dim3((unsigned)T), dim3(256), 0, st,
                       out, in, w, eps, (int)H, hidden_f, out_stride, in_stride);
    return launch_status();
  }
  const int nvec = (int)(H / N);
  const uint32_t row_bytes = (uint32_t)(H * EB);
  dim3 grid((unsigned)T);
#define SK_RMS_CASE(WAVES, VPL)                                                               \
  hipLaunchKernelGGL((rms_norm_row_kernel<DT, WAVES, VPL, FUSED>), grid, dim3(64 * WAVES), 0, \
                     st, out, in, w, eps, row_bytes, hidden_f, out_stride * EB, in_stride * EB)
  // Fused op on rows of 129..512 vectors from 4 rows per compute unit on: one wave per row with the
  // stores held back, a grid with no row counts it prefers.  Against the shapes below, bf16, on
  // separately allocated tensors, rows of 4096: 2048 rows 11.9 -> 11.4 us, 2560 15.8 -> 14.6,
  // 3584 21.3 -> 19.5, 4608 27.3 -> 25.8, 8192 46.7 -> 45.2, 32768 181 -> 178 (65536: 370 against 378,
  // left to the shapes below); rows of 3072 alike; rows of 2048 (four vectors per lane): 4096 rows
  // 12.4 -> 11.9, 4608 13.8 -> 13.4, but 8192 rows 22.7 against 23.7 and 16384 43.7 against 48.8.
  // Smaller batches want more waves per row.
  if constexpr (FUSED) {
    const int64_t units = compute_units();
    if (nvec > 128 && nvec <= 512 && T > 4 * units && T <= (nvec <= 256 ? 24 : 160) * units) {
      if (nvec <= 256)
        hipLaunchKernelGGL((fused_add_rms_norm_wave_kernel<DT, 4>), grid, dim3(64), 0, st, out, in, w,
                           eps, row_bytes, hidden_f, out_stride * EB, in_stride * EB);
      else
        hipLaunchKernelGGL((fused_add_rms_norm_wave_kernel<DT, 8>), grid, dim3(64), 0, st, out, in, w,
                           eps, row_bytes, hidden_f, out_stride * EB, in_stride * EB);
      return launch_status();
    }
  }
  // Fused op on rows of 257..512 vectors outside that range: two or three rows per one-wave
  // workgroup where the row count makes that come out even over the compute units.  (The plain
  // norm gains nothing from several rows per wave, from holding its stores back, or from two
  // waves per row: 7.1, 7.3, 7.5, 7.7 us at 2304 x 4096; nor from workgroups of two, three or four
  // independent one-row waves: 7.6, 7.4, 8.6 us against 7.4 for that kernel with one wave.)
  if (FUSED && nvec > 256 && nvec <= 512 && out_stride / N <= 0xffffffffLL &&
      in_stride / N <= 0xffffffffLL) {
    const int rows_per_wg = pick_rows_per_workgroup(T, 3);
    const dim3 rgrid((unsigned)((T + rows_per_wg - 1) / rows_per_wg));
#define SK_RMS_ROWS(R)                                                                           \
  hipLaunchKernelGGL((rms_norm_wave_rows_kernel<DT, 8, R, FUSED>), rgrid, dim3(64), 0, st, out,  \
                     in, w, eps, row_bytes, hidden_f, (uint32_t)(out_stride / N),                 \
                     (uint32_t)(in_stride / N), (uint32_t)T)
    if (rows_per_wg == 3) {
      SK_RMS_ROWS(3);
      return launch_status();
    }
    if (rows_per_wg == 2) {
      SK_RMS_ROWS(2);
      return launch_status();
    }
#undef SK_RMS_ROWS
  }
  // Rows of 513..1024 vectors (hidden sizes 4104..8192 in 16-bit types), 4 rows per compute unit
  // and up: one wave per row (10..16 vectors per lane) for as long as every wave of the launch is
  // resident at once, so that the launch is one read phase followed by one write phase.  bf16, cold,
  // separately allocated tensors, multi-wave shape below -> one wave; plain norm: rows of 5120,
  // 1024 rows 5.5 -> 4.9 us, 2304 10.0 -> 8.8, 4096 15.6 -> 14.8 (4608: 17.5 against 19.3); rows of
  // 7168, 2304 rows 13.1 -> 11.4, 3072 16.4 -> 15.2 (3584: 18.9 against 21.2); rows of 8192, 2048
  // rows 13.3 -> 11.3, 3072 18.5 -> 17.2 (3584: 21.0 against 23.7).  Fused op (stores held back):
  // rows of 5120, 2304 rows 16.8 -> 15.3, 3072 21.5 -> 20.0 (3584: 24.8 against 25.8); rows of
  // 7168, 2048 rows 20.5 -> 18.6 (2560 equal, 3072 behind); rows of 8192, 2048 rows 22.8 -> 20.9
  // (2560: 27.8 against 28.3).  Below 4 rows per unit the multi-wave shapes are ahead.
  if (nvec > 512 && nvec <= 1024) {
    const int64_t units = compute_units();
    const int vpl = 2 * ((nvec + 127) / 128);  // 10, 12, 14 or 16
    const int64_t cap = FUSED ? (vpl == 10 ? 12 : 8) : (vpl <= 12 ? 16 : 12);
    if (T >= 4 * units && T <= cap * units) {
#define SK_RMS_WAVE(VPL)                                                                         \
  case VPL:                                                                                      \
    if constexpr (FUSED)                                                                         \
      hipLaunchKernelGGL((fused_add_rms_norm_wave_kernel<DT, VPL>), grid, dim3(64), 0, st, out,  \
                         in, w, eps, row_bytes, hidden_f, out_stride * EB, in_stride * EB);      \
    else                                                                                         \
      SK_RMS_CASE(1, VPL);                                                                       \
    return launch_status();
      switch (vpl) {
        SK_RMS_WAVE(10) SK_RMS_WAVE(12) SK_RMS_WAVE(14) SK_RMS_WAVE(16)
      }
#undef SK_RMS_WAVE
    }
  }
  // One row per workgroup.  Shapes measured on MI355X at H = 4096 and H = 8192 (bf16).  The plain
  // norm is fastest with a whole row of up to 512 vectors in ONE wave (no LDS, no barrier) and
  // four vectors per lane beyond that; the fused op, which holds two rows' worth of loads, is
  // fastest with two vectors per lane and proportionally more waves.
  if (nvec <= 64) SK_RMS_CASE(1, 1);
  else if (nvec <= 128) SK_RMS_CASE(1, 2);
  else if (FUSED) {
    if (nvec <= 256) SK_RMS_CASE(2, 2);
    else if (nvec <= 512) SK_RMS_CASE(4, 2);
    else if (nvec <= 1024) SK_RMS_CASE(8, 2);
    else if (nvec <= 2048) SK_RMS_CASE(16, 2);
    else SK_RMS_CASE(16, 4);
  } else {
    if (nvec <= 256) SK_RMS_CASE(1, 4);
    else if (nvec <= 512) SK_RMS_CASE(1, 8);
    else if (nvec <= 1024) SK_RMS_CASE(4, 4);
    else if (nvec <= 2048) SK_RMS_CASE(8, 4);
    else SK_RMS_CASE(16, 4);
  }
#undef SK_RMS_CASE
  return launch_status();
}

template <bool FUSED>
static int dispatch_rms(void* out, void* in, const void* w, float eps, int64_t T, int64_t H,
                        int64_t out_stride, int64_t in_stride, int dtype, void* stream) {
  if (T > 0 && (!out || !in || !w)) return SARATHI_ERR_INVALID_ARG;  // empty tensors have no data
  if (T < 0 || H <= 0 || out_stride < H || in_stride < H) return SARATHI_ERR_INVALID_ARG;
  if (H > 0x7fffffffLL) return SARATHI_ERR_UNSUPPORTED;
  if (T == 0) return SARATHI_OK;
  hipStream_t st = (hipStream_t)stream;
  switch (dtype) {
    case kBF16: return launch_rms<kBF16, FUSED>(out, in, w, eps, T, H, out_stride, in_stride, st);
    case kF16: return launch_rms<kF16, FUSED>(out, in, w, eps, T, H, out_stride, in_stride, st);
    case kF32: return launch_rms<kF32, FUSED>(out, in, w, eps, T, H, out_stride, in_stride, st);
    default: return SARATHI_ERR_UNSUPPORTED;
  }
}

}  // namespace sarathi_hip

extern "C" int sarathi_rms_norm(void* out, const void* input, const void* weight, float epsilon,
                                int64_t num_tokens, int64_t hidden_size,
                                int64_t input_row_stride, int64_t out_row_stride, int dtype,
                                void* stream) {
  return sarathi_hip::dispatch_rms<false>(out, const_cast<void*>(input), weight, epsilon,
                                          num_tokens, hidden_size, out_row_stride,
                                          input_row_stride, dtype, stream);
}

extern "C" int sarathi_fused_add_rms_norm(void* input, void* residual, const void* weight,
                                          float epsilon, int64_t num_tokens, int64_t hidden_size,
                                          int64_t input_row_stride, int64_t residual_row_stride,
                                          int dtype, void* stream) {
  return sarathi_hip::dispatch_rms<true>(input, residual, weight, epsilon, num_tokens,
                                         hidden_size, input_row_stride, residual_row_stride,
                                         dtype, stream);
}
