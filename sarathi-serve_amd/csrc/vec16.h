// 16-byte vector access and dtype conversion helpers for gfx950 kernels.
//
// Every dense kernel in this library moves data as one 16-byte global access
// per lane (global_load_dwordx4 / global_store_dwordx4): 8 bf16 or fp16
// elements, or 4 fp32 elements.  Arithmetic is always fp32; `rnd<DT>()` is the
// "cast to the tensor dtype and widen again" step that the reference's
// scalar_t arithmetic performs between operations.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace sarathi_hip {

enum : int { kF32 = 0, kF16 = 1, kBF16 = 2 };

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));

#define SK_DEV __device__ __forceinline__

template <int DT> struct ElemBytes { static constexpr int value = 2; };
template <> struct ElemBytes<kF32> { static constexpr int value = 4; };

// elements per 16-byte vector
template <int DT> struct VecElems { static constexpr int value = 16 / ElemBytes<DT>::value; };

// Bit reinterpretation of by-value scalars.  Vector elements must go through
// these (i.e. be copied to a scalar first): __builtin_bit_cast applied directly
// to an ext-vector element expression reads element 0 with this compiler.
SK_DEV float as_f32(uint32_t w) { return __builtin_bit_cast(float, w); }
SK_DEV uint32_t as_u32(float f) { return __builtin_bit_cast(uint32_t, f); }

// ---- packed 32-bit word <-> two floats -------------------------------------

template <int DT> SK_DEV f32x2 unpack2(uint32_t w);
template <> SK_DEV f32x2 unpack2<kBF16>(uint32_t w) {
  f32x2 r;
  r.x = __builtin_bit_cast(float, w << 16);
  r.y = __builtin_bit_cast(float, w & 0xffff0000u);
  return r;
}
template <> SK_DEV f32x2 unpack2<kF16>(uint32_t w) {
  return __builtin_convertvector(__builtin_bit_cast(f16x2, w), f32x2);
}

// round-to-nearest-even pack (v_cvt_pk_bf16_f32 / v_cvt_f16_f32 on gfx950)
template <int DT> SK_DEV uint32_t pack2(float a, float b);
template <> SK_DEV uint32_t pack2<kBF16>(float a, float b) {
  f32x2 v = {a, b};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));
}
template <> SK_DEV uint32_t pack2<kF16>(float a, float b) {
  f32x2 v = {a, b};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, f16x2));
}

// Round a float to the tensor dtype and widen again.
template <int DT> SK_DEV float rnd(float f);
template <> SK_DEV float rnd<kF32>(float f) { return f; }
template <> SK_DEV float rnd<kBF16>(float f) { return (float)(__bf16)f; }
template <> SK_DEV float rnd<kF16>(float f) { return (float)(_Float16)f; }

// Round two floats to the tensor dtype and widen again with ONE packed conversion (half the
// conversions of two rnd<DT>() calls; same results).
template <int DT> SK_DEV f32x2 rnd2(float a, float b) {
  if constexpr (DT == kF32) {
    f32x2 r = {a, b};
    return r;
  } else {
    return unpack2<DT>(pack2<DT>(a, b));
  }
}

// ---- a 16-byte vector as an array of floats --------------------------------

template <int DT> struct Vec {
  static constexpr int N = VecElems<DT>::value;
  float f[N];

  SK_DEV void unpack(u32x4 v) {
    if constexpr (DT == kF32) {
#pragma unroll
      for (int i = 0; i < 4; ++i) f[i] = as_f32(v[i]);
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        f32x2 p = unpack2<DT>(v[i]);
        f[2 * i] = p.x;
        f[2 * i + 1] = p.y;
      }
    }
  }
  // rounds to the dtype
  SK_DEV u32x4 pack() const {
    u32x4 v;
    if constexpr (DT == kF32) {
#pragma unroll
      for (int i = 0; i < 4; ++i) v[i] = as_u32(f[i]);
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) v[i] = pack2<DT>(f[2 * i], f[2 * i + 1]);
    }
    return v;
  }
};

// ---- activation shared by silu_and_mul and the gated GEMM epilogue ---------------------------

SK_DEV float silu_f32(float x) {
  // x * sigmoid(x) = x / (1 + 2^(-x * log2 e))
  float e = __builtin_amdgcn_exp2f(x * -1.4426950408889634f);
  return x * __builtin_amdgcn_rcpf(1.0f + e);
}

// ---- global memory ---------------------------------------------------------

// 16-byte accesses go through raw buffer instructions: the base pointer of the
// row (or tensor) a workgroup works on lives in scalar registers as a buffer
// resource, lanes supply 32-bit byte offsets, and the hardware drops accesses
// at or beyond `bytes` (loads return 0, stores are discarded), so ragged row
// ends need no branch.  A resource spans at most 4 GiB - 1.
//
// Cache policy bits of the access (gfx940+): 1 = sc0, 2 = nt, 16 = sc1.
//   kStreamLoad  nt      read-once data: do not keep it in L2 / Infinity Cache
//   kStreamStore nt|sc1  write-once data: written through, measured ~3 % faster
//                        than nt alone on MI355X copies
//   kCached      0       rows that are re-read by many workgroups (weights,
//                        cos/sin cache)
// The two streaming policies can be overridden at compile time for tuning runs.
#ifndef SARATHI_STREAM_LOAD_POLICY
#define SARATHI_STREAM_LOAD_POLICY 2
#endif
#ifndef SARATHI_STREAM_STORE_POLICY
#define SARATHI_STREAM_STORE_POLICY (2 | 16)
#endif
typedef __amdgpu_buffer_rsrc_t rsrc_t;
constexpr int kCached = 0;
constexpr int kStreamLoad = SARATHI_STREAM_LOAD_POLICY;
constexpr int kStreamStore = SARATHI_STREAM_STORE_POLICY;

SK_DEV rsrc_t make_rsrc(const void* base, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, bytes, 0x00020000);
}
template <int POLICY> SK_DEV u32x4 buf_load16(rsrc_t r, uint32_t byte_off) {
  return __builtin_amdgcn_raw_buffer_load_b128(r, byte_off, 0, POLICY);
}
template <int POLICY> SK_DEV void buf_store16(rsrc_t r, uint32_t byte_off, u32x4 v) {
  __builtin_amdgcn_raw_buffer_store_b128(v, r, byte_off, 0, POLICY);
}
template <int POLICY> SK_DEV u32x2 buf_load8(rsrc_t r, uint32_t byte_off) {
  return __builtin_amdgcn_raw_buffer_load_b64(r, byte_off, 0, POLICY);
}

// Element-wise accessors for the unaligned fallback paths.
template <int DT> SK_DEV float load_elem(const void* base, int64_t i) {
  if constexpr (DT == kF32) return reinterpret_cast<const float*>(base)[i];
  else if constexpr (DT == kBF16)
    return __builtin_bit_cast(float, (uint32_t)reinterpret_cast<const uint16_t*>(base)[i] << 16);
  else return (float)reinterpret_cast<const _Float16*>(base)[i];
}
template <int DT> SK_DEV void store_elem(void* base, int64_t i, float v) {
  if constexpr (DT == kF32) reinterpret_cast<float*>(base)[i] = v;
  else if constexpr (DT == kBF16) reinterpret_cast<__bf16*>(base)[i] = (__bf16)v;
  else reinterpret_cast<_Float16*>(base)[i] = (_Float16)v;
}

// ---- waits and the workgroup barrier for LDS exchanges ---------------------------

// Waits until at most N of this wave's vector-memory operations (loads and stores alike on
// gfx9) are outstanding.
template <int N> SK_DEV void wait_vmcnt() { asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory"); }

// Orders LDS traffic only: a wave waits for its own LDS operations and then meets the others.
// Global loads and stores issued before it stay in flight across it (prefetches, streaming
// stores).  __syncthreads() promises no more than that for global memory on this target: its
// fences are workgroup scope, and when all waves of a workgroup share a compute unit the
// compiler may satisfy them without a `vmcnt(0)` (it usually waits for fewer operations, or
// none).  Data that has to be visible outside the workgroup needs an explicit
// wait_vmcnt<0>() (for write-through stores) or a wider fence.  Use this barrier only where
// the data exchanged through it lives in LDS.
SK_DEV void lds_barrier() {
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// ---- wave64 reductions -------------------------------------------------------

// Adds `v` across the 64 lanes of a wave; every lane returns the total.
// Four DPP steps fold each row of 16 lanes (quad swaps, then the half-row and
// row mirrors, which are valid folds because each group being mirrored is
// already uniform), then the four row totals are read as scalars and added.
template <int CTRL> SK_DEV float dpp_fold_add(float x) {
  int y = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL, 0xf, 0xf, false);
  return x + __builtin_bit_cast(float, y);
}
SK_DEV float wave64_sum(float v) {
  v = dpp_fold_add<0xB1>(v);   // quad_perm [1,0,3,2]
  v = dpp_fold_add<0x4E>(v);   // quad_perm [2,3,0,1]
  v = dpp_fold_add<0x141>(v);  // row_half_mirror
  v = dpp_fold_add<0x140>(v);  // row_mirror
  int b = __builtin_bit_cast(int, v);
  float r0 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 0));
  float r1 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 16));
  float r2 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 32));
  float r3 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 48));
  return (r0 + r1) + (r2 + r3);
}

SK_DEV float wave64_max(float v) {
#pragma unroll
  for (int m = 32; m > 0; m >>= 1) v = fmaxf(v, __shfl_xor(v, m, 64));
  return v;
}

}  // namespace sarathi_hip
