// rotary_embedding (GPT-NeoX and GPT-J layouts) for gfx950.
//
// Replaces csrc/pos_encoding_kernels.cu:8-127 of the reference (one block per
// token, every thread touching four 2-byte values that sit 128 B apart, `int`
// offsets).  Here the unit of work is one 16-byte slot of one head:
//   NeoX : the lane loads 8 (fp32: 4) consecutive x at offset c and the
//          matching y at offset rot/2 + c of the head, plus the 16-byte cos and
//          sin vectors at the same offset c of the token's cache row, rotates
//          them in registers and writes both vectors back;
//   GPT-J: x and y interleave, so one 16-byte vector already holds whole
//          pairs; cos and sin come from two half-width loads.
// threadIdx.x walks the slots of a head and threadIdx.y the heads (q heads
// first, then k heads), so no integer division is needed, and each thread
// handles TOK consecutive tokens with all loads issued first.  Row offsets are
// 64-bit.  q and k rows may be views into a packed qkv buffer (row stride !=
// row width); elements at or beyond rot_dim inside a head are not touched.
//
// Arithmetic is the reference's scalar_t arithmetic: each product and the final
// sum round to the tensor dtype (csrc/pos_encoding_kernels.cu:32-35):
//   x' = T( T(x*cos) - T(y*sin) ),  y' = T( T(y*cos) + T(x*sin) ).
#include "vec16.h"
#include "launch.h"

namespace sarathi_hip {

struct RopeArgs {
  const int64_t* positions;
  void* query;
  void* key;
  const void* cache;
  int64_t num_tokens;
  int64_t q_stride;  // elements
  int64_t k_stride;  // elements
  int num_heads;
  int num_kv_heads;
  int head_size;
  int rot_dim;
};

template <int DT> SK_DEV float mul_r(float a, float b) { return rnd<DT>(a * b); }

template <int DT, bool NEOX, int TOK>
__global__ __launch_bounds__(1024) void rope_vec_kernel(RopeArgs a) {
  constexpr int N = VecElems<DT>::value;
  const int slot = threadIdx.x;  // 16-byte slot inside the head's x half (NeoX) / head (GPT-J)
  const int total_heads = a.num_heads + a.num_kv_heads;
  const int64_t tok0 = (int64_t)blockIdx.x * TOK;
  const int embed = a.rot_dim >> 1;

  for (int head = threadIdx.y; head < total_heads; head += blockDim.y) {
    const bool is_q = head < a.num_heads;
    char* base = reinterpret_cast<char*>(is_q ? a.query : a.key);
    const int64_t stride = is_q ? a.q_stride : a.k_stride;
    const int h = is_q ? head : head - a.num_heads;
    constexpr int EB = ElemBytes<DT>::value;

    u32x4 xv[TOK], yv[TOK], cv[TOK], sv[TOK];
    char* xp[TOK];
#pragma unroll
    for (int t = 0; t < TOK; ++t) {
      const int64_t tok = tok0 + t;
      if (tok < a.num_tokens) {
        xp[t] = base + (tok * stride + (int64_t)h * a.head_size) * EB;
        const char* crow =
            reinterpret_cast<const char*>(a.cache) + a.positions[tok] * a.rot_dim * EB;
        if constexpr (NEOX) {
          xv[t] = *reinterpret_cast<const u32x4*>(xp[t] + slot * 16);
          yv[t] = *reinterpret_cast<const u32x4*>(xp[t] + embed * EB + slot * 16);
          cv[t] = *reinterpret_cast<const u32x4*>(crow + slot * 16);
          sv[t] = *reinterpret_cast<const u32x4*>(crow + embed * EB + slot * 16);
        } else {
          xv[t] = *reinterpret_cast<const u32x4*>(xp[t] + slot * 16);
          u32x2 c2 = *reinterpret_cast<const u32x2*>(crow + slot * 8);
          u32x2 s2 = *reinterpret_cast<const u32x2*>(crow + embed * EB + slot * 8);
          cv[t] = (u32x4){c2.x, c2.y, 0, 0};
          sv[t] = (u32x4){s2.x, s2.y, 0, 0};
        }
      }
    }
#pragma unroll
    for (int t = 0; t < TOK; ++t) {
      const int64_t tok = tok0 + t;
      if (tok < a.num_tokens) {
        Vec<DT> x, y, c, s;
        x.unpack(xv[t]);
        c.unpack(cv[t]);
        s.unpack(sv[t]);
        if constexpr (NEOX) {
          y.unpack(yv[t]);
          Vec<DT> ox, oy;
#pragma unroll
          for (int i = 0; i < N; ++i) {
            ox.f[i] = mul_r<DT>(x.f[i], c.f[i]) - mul_r<DT>(y.f[i], s.f[i]);
            oy.f[i] = mul_r<DT>(y.f[i], c.f[i]) + mul_r<DT>(x.f[i], s.f[i]);
          }
          *reinterpret_cast<u32x4*>(xp[t] + slot * 16) = ox.pack();
          *reinterpret_cast<u32x4*>(xp[t] + embed * EB + slot * 16) = oy.pack();
        } else {
          Vec<DT> o;
#pragma unroll
          for (int i = 0; i < N / 2; ++i) {
            float xe = x.f[2 * i], ye = x.f[2 * i + 1];
            o.f[2 * i] = mul_r<DT>(xe, c.f[i]) - mul_r<DT>(ye, s.f[i]);
            o.f[2 * i + 1] = mul_r<DT>(ye, c.f[i]) + mul_r<DT>(xe, s.f[i]);
          }
          *reinterpret_cast<u32x4*>(xp[t] + slot * 16) = o.pack();
        }
      }
    }
  }
}

// Any alignment / rot_dim: one thread per rotated pair, one block per token.
template <int DT, bool NEOX>
__global__ __launch_bounds__(256) void rope_generic_kernel(RopeArgs a) {
  const int64_t tok = blockIdx.x;
  const int embed = a.rot_dim >> 1;
  const int64_t crow = a.positions[tok] * a.rot_dim;
  const int nq = a.num_heads * embed;
  const int total = (a.num_heads + a.num_kv_heads) * embed;
  for (int i = threadIdx.x; i < total; i += 256) {
    const bool is_q = i < nq;
    void* arr = is_q ? a.query : a.key;
    const int j = is_q ? i : i - nq;
    const int h = j / embed, r = j - h * embed;
    const int64_t hb = tok * (is_q ? a.q_stride : a.k_stride) + (int64_t)h * a.head_size;
    const int64_t xi = hb + (NEOX ? r : 2 * r), yi = hb + (NEOX ? embed + r : 2 * r + 1);
    const float c = load_elem<DT>(a.cache, crow + r), s = load_elem<DT>(a.cache, crow + embed + r);
    const float x = load_elem<DT>(arr, xi), y = load_elem<DT>(arr, yi);
    store_elem<DT>(arr, xi, mul_r<DT>(x, c) - mul_r<DT>(y, s));
    store_elem<DT>(arr, yi, mul_r<DT>(y, c) + mul_r<DT>(x, s));
  }
}

template <int DT, bool NEOX>
static int launch_rope(const RopeArgs& a, hipStream_t st) {
  constexpr int N = VecElems<DT>::value;
  constexpr int EB = ElemBytes<DT>::value;
  if (a.num_tokens > 0x7fffffffLL) return SARATHI_ERR_UNSUPPORTED;
  const int embed = a.rot_dim / 2;
  // 16-byte slots per head: NeoX covers the x half (the y half rides along), GPT-J the whole
  // rotated span
  const int span = NEOX ? embed : a.rot_dim;
  const bool vec_ok = (span % N == 0) && (span / N <= 1024) && ((a.head_size * EB) % 16 == 0) &&
                      ((a.q_stride * EB) % 16 == 0) && ((a.k_stride * EB) % 16 == 0) &&
                      ((a.rot_dim * EB) % 16 == 0) && ((embed * EB) % (NEOX ? 16 : 8) == 0) &&
                      aligned16(a.query) && aligned16(a.key) && aligned16(a.cache);
  if (!vec_ok) {
    hipLaunchKernelGGL((rope_generic_kernel<DT, NEOX>), dim3((unsigned)a.num_tokens), dim3(256),
                       0, st, a);
    return launch_status();
  }
  constexpr int TOK = 2;
  const int slots = span / N;
  const int heads = a.num_heads + a.num_kv_heads;
  int by = 1024 / slots;
  if (by > heads) by = heads;
  dim3 block((unsigned)slots, (unsigned)by);
  dim3 grid((unsigned)((a.num_tokens + TOK - 1) / TOK));
  hipLaunchKernelGGL((rope_vec_kernel<DT, NEOX, TOK>), grid, block, 0, st, a);
  return launch_status();
}

}  // namespace sarathi_hip

extern "C" int sarathi_rotary_embedding(const int64_t* positions, void* query, void* key,
                                        const void* cos_sin_cache, int64_t num_tokens,
                                        int num_heads, int num_kv_heads, int head_size,
                                        int rot_dim, int64_t query_stride, int64_t key_stride,
                                        int is_neox, int dtype, void* stream) {
  using namespace sarathi_hip;
  if (!positions || !query || !key || !cos_sin_cache) return SARATHI_ERR_INVALID_ARG;
  if (num_tokens < 0 || num_heads <= 0 || num_kv_heads < 0 || head_size <= 0 || rot_dim <= 0 ||
      (rot_dim & 1) || rot_dim > head_size)
    return SARATHI_ERR_INVALID_ARG;
  if (query_stride < (int64_t)num_heads * head_size ||
      key_stride < (int64_t)num_kv_heads * head_size)
    return SARATHI_ERR_INVALID_ARG;
  if (num_tokens == 0) return SARATHI_OK;
  RopeArgs a{positions, query,     key,          cos_sin_cache, num_tokens, query_stride,
             key_stride, num_heads, num_kv_heads, head_size,     rot_dim};
  hipStream_t st = (hipStream_t)stream;
#define SK_ROPE(DT) (is_neox ? launch_rope<DT, true>(a, st) : launch_rope<DT, false>(a, st))
  switch (dtype) {
    case kBF16: return SK_ROPE(kBF16);
    case kF16: return SK_ROPE(kF16);
    case kF32: return SK_ROPE(kF32);
    default: return SARATHI_ERR_UNSUPPORTED;
  }
#undef SK_ROPE
}
