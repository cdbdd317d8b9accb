// A plain device-to-device copy in the shapes the streaming ops of this library launch: one-wave
// workgroups, every lane VPL 16-byte loads (all issued before the first store) and VPL 16-byte
// stores, workgroup ids walking memory linearly, the library's streaming cache policies.  It is
// what bench.py measures as the ceiling of a launch that moves a given number of bytes: no
// arithmetic, no row structure, nothing to wait for but the data.  No counterpart in the reference.
//
// Measured on MI355X, 18.9 MB in + 18.9 MB out, cold: 1 KiB per wave 7.2 us, 8 KiB 7.1 us,
// 16 KiB 7.4 us, 18 KiB (1024 waves, one per SIMD) 6.6 us, 24 KiB 6.4 us, 36 KiB 6.5 us,
// 48 KiB 7.6 us: launches of at most one wave per SIMD are the fast ones.
#include "vec16.h"
#include "launch.h"

namespace sarathi_hip {

template <int VPL>
__global__ __launch_bounds__(64) void stream_copy_kernel(void* __restrict__ dst,
                                                         const void* __restrict__ src,
                                                         uint32_t span_bytes) {
  const rsrc_t ri = make_rsrc(src, span_bytes), ro = make_rsrc(dst, span_bytes);
  const uint32_t off0 = blockIdx.x * (VPL * 1024u) + threadIdx.x * 16u;
  u32x4 v[VPL];
#pragma unroll
  for (int j = 0; j < VPL; ++j) v[j] = buf_load16<kStreamLoad>(ri, off0 + j * 1024u);
  // left alone, the scheduler starts storing after about ten loads and issues the rest one by one
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int j = 0; j < VPL; ++j) buf_store16<kStreamStore>(ro, off0 + j * 1024u, v[j]);
}

template <int VPL>
static int launch_copy(void* dst, const void* src, int64_t bytes, hipStream_t st) {
  const int64_t per_wg = (int64_t)VPL * 1024;
  const unsigned grid = (unsigned)((bytes + per_wg - 1) / per_wg);
  hipLaunchKernelGGL((stream_copy_kernel<VPL>), dim3(grid), dim3(64), 0, st, dst, src,
                     (uint32_t)bytes);
  return launch_status();
}

}  // namespace sarathi_hip

extern "C" int sarathi_stream_copy(void* dst, const void* src, int64_t bytes, int kib_per_wave,
                                   void* stream) {
  using namespace sarathi_hip;
  if (bytes < 0 || (bytes > 0 && (!dst || !src))) return SARATHI_ERR_INVALID_ARG;
  if (bytes == 0) return SARATHI_OK;
  // lanes past the end are clipped by the buffer resource, whole 16-byte vectors only
  if ((bytes & 15) != 0 || !aligned16(dst) || !aligned16(src)) return SARATHI_ERR_INVALID_ARG;
  if (bytes > 0xffffffffLL) return SARATHI_ERR_UNSUPPORTED;  // one buffer resource
  hipStream_t st = (hipStream_t)stream;
  switch (kib_per_wave) {
    case 1: return launch_copy<1>(dst, src, bytes, st);
    case 2: return launch_copy<2>(dst, src, bytes, st);
    case 4: return launch_copy<4>(dst, src, bytes, st);
    case 8: return launch_copy<8>(dst, src, bytes, st);
    case 12: return launch_copy<12>(dst, src, bytes, st);
    case 16: return launch_copy<16>(dst, src, bytes, st);
    case 18: return launch_copy<18>(dst, src, bytes, st);
    case 24: return launch_copy<24>(dst, src, bytes, st);
    case 36: return launch_copy<36>(dst, src, bytes, st);
    case 48: return launch_copy<48>(dst, src, bytes, st);
    default: return SARATHI_ERR_UNSUPPORTED;
  }
}
