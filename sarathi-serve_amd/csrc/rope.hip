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
// A workgroup is one wave: 64 consecutive slots of one token's q row or of its
// k row (8 heads of 128 at bf16).  Workgroup ids run over the q segments, then
// the k segments, then the tokens, so the waves in flight sweep the packed qkv
// buffer linearly.  The token's q row, k row and cos/sin cache row are scalar
// buffer resources (the position is a scalar load); lanes past the last head
// are clipped by the hardware range check, so the kernel has no branches.
// Elements at or beyond rot_dim inside a head are not touched.
//
// Arithmetic is the reference's scalar_t arithmetic: each product and the final
// sum round to the tensor dtype (csrc/pos_encoding_kernels.cu:32-35):
//   x' = T( T(x*cos) - T(y*sin) ),  y' = T( T(y*cos) + T(x*sin) ).
#include "vec16.h"
#include "launch.h"

namespace sarathi_hip {

constexpr uint32_t kClipped = 0x80000000u;  // byte offset beyond any row: access is dropped

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

// Kernel arguments are laid out so that everything the first loads need sits in
// the first 56 bytes, which the hardware preloads into scalar registers at wave
// launch: the wave can issue its q/k loads without waiting for an argument fetch,
// and only then fetches the token's position and, from it, the cos/sin row.
//   geom  = head_bytes | embed_bytes << 16          (bytes of one head / of rot_dim/2)
//   heads = num_heads | num_kv_heads << 12 | slot_shift << 24
// slot_shift = log2(16-byte slots per head); NeoX counts the slots of the x half,
// GPT-J those of the whole rotated span.
template <int DT, bool NEOX>
__global__ __launch_bounds__(64) void rope_seg_kernel(
    const int64_t* __restrict__ positions, void* query, void* key, const void* __restrict__ cache,
    int64_t q_stride_bytes, int64_t k_stride_bytes, uint32_t geom, uint32_t heads) {
  constexpr int N = VecElems<DT>::value;
  const uint32_t head_bytes = geom & 0xffffu, embed_bytes = geom >> 16;
  const int num_heads = heads & 0xfffu, num_kv_heads = (heads >> 12) & 0xfffu;
  const int slot_shift = heads >> 24;
  const int q_blocks = ((num_heads << slot_shift) + 63) >> 6;
  const int64_t tok = (int64_t)blockIdx.z * kMaxGridY + blockIdx.y;
  const bool is_q = (int)blockIdx.x < q_blocks;  // uniform over the wave
  const int item = ((int)blockIdx.x - (is_q ? 0 : q_blocks)) * 64 + (int)threadIdx.x;
  const int nheads = is_q ? num_heads : num_kv_heads;
  const int h = item >> slot_shift;
  const uint32_t slot = item & ((1 << slot_shift) - 1);
  char* base = reinterpret_cast<char*>(is_q ? query : key) +
               tok * (is_q ? q_stride_bytes : k_stride_bytes);
  const rsrc_t rd = make_rsrc(base, (uint32_t)nheads * head_bytes);
  const uint32_t xoff = h < nheads ? (uint32_t)h * head_bytes + slot * 16u : kClipped;

  u32x4 xr, yr;
  xr = buf_load16<kStreamLoad>(rd, xoff);
  if constexpr (NEOX) yr = buf_load16<kStreamLoad>(rd, xoff + embed_bytes);
  // keep the position fetch (and everything hanging off it) behind the loads above
  __builtin_amdgcn_sched_barrier(0);
  const rsrc_t rc = make_rsrc(
      reinterpret_cast<const char*>(cache) + positions[tok] * (int64_t)(2 * embed_bytes),
      2 * embed_bytes);

  u32x4 cr, sr;
  if constexpr (NEOX) {
    cr = buf_load16<kCached>(rc, slot * 16u);
    sr = buf_load16<kCached>(rc, embed_bytes + slot * 16u);
  } else {
    const u32x2 c2 = buf_load8<kCached>(rc, slot * 8u);
    const u32x2 s2 = buf_load8<kCached>(rc, embed_bytes + slot * 8u);
    cr = (u32x4){c2.x, c2.y, 0, 0};
    sr = (u32x4){s2.x, s2.y, 0, 0};
  }
  // all four loads are in flight before the first result is waited for
  __builtin_amdgcn_sched_barrier(0);

  Vec<DT> x, c, s;
  x.unpack(xr);
  c.unpack(cr);
  s.unpack(sr);
  if constexpr (NEOX) {
    Vec<DT> y, ox, oy;
    y.unpack(yr);
#pragma unroll
    for (int i = 0; i < N; ++i) {
      ox.f[i] = mul_r<DT>(x.f[i], c.f[i]) - mul_r<DT>(y.f[i], s.f[i]);
      oy.f[i] = mul_r<DT>(y.f[i], c.f[i]) + mul_r<DT>(x.f[i], s.f[i]);
    }
    buf_store16<kStreamStore>(rd, xoff, ox.pack());
    buf_store16<kStreamStore>(rd, xoff + embed_bytes, oy.pack());
  } else {
    Vec<DT> o;
#pragma unroll
    for (int i = 0; i < N / 2; ++i) {
      const float xe = x.f[2 * i], ye = x.f[2 * i + 1];
      o.f[2 * i] = mul_r<DT>(xe, c.f[i]) - mul_r<DT>(ye, s.f[i]);
      o.f[2 * i + 1] = mul_r<DT>(ye, c.f[i]) + mul_r<DT>(xe, s.f[i]);
    }
    buf_store16<kStreamStore>(rd, xoff, o.pack());
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
  const int64_t q_row_bytes = (int64_t)a.num_heads * a.head_size * EB;
  const int64_t k_row_bytes = (int64_t)a.num_kv_heads * a.head_size * EB;
  const bool vec_ok = (span % N == 0) && ((a.head_size * EB) % 16 == 0) &&
                      ((a.q_stride * EB) % 16 == 0) && ((a.k_stride * EB) % 16 == 0) &&
                      ((a.rot_dim * EB) % 16 == 0) && ((embed * EB) % (NEOX ? 16 : 8) == 0) &&
                      aligned16(a.query) && aligned16(a.key) && aligned16(a.cache) &&
                      q_row_bytes < (int64_t)kClipped && k_row_bytes < (int64_t)kClipped;
  if (!vec_ok) {
    hipLaunchKernelGGL((rope_generic_kernel<DT, NEOX>), dim3((unsigned)a.num_tokens), dim3(256),
                       0, st, a);
    return launch_status();
  }
  const int slots = span / N;
  int slot_shift = 0;
  while ((1 << slot_shift) < slots) ++slot_shift;
  const int64_t head_bytes = (int64_t)a.head_size * EB;
  // the packed-argument kernel needs power-of-two slots and fields that fit their bit widths
  const bool packable = (1 << slot_shift) == slots && head_bytes < 65536 && embed * EB < 65536 &&
                        a.num_heads < 4096 && a.num_kv_heads < 4096;
  if (!packable) {
    hipLaunchKernelGGL((rope_generic_kernel<DT, NEOX>), dim3((unsigned)a.num_tokens), dim3(256),
                       0, st, a);
    return launch_status();
  }
  const uint32_t geom = (uint32_t)head_bytes | ((uint32_t)(embed * EB) << 16);
  const uint32_t heads =
      (uint32_t)a.num_heads | ((uint32_t)a.num_kv_heads << 12) | ((uint32_t)slot_shift << 24);
  const int64_t q_blocks = ((int64_t)a.num_heads * slots + 63) / 64;
  const int64_t k_blocks = ((int64_t)a.num_kv_heads * slots + 63) / 64;
  const unsigned gx = (unsigned)(q_blocks + k_blocks);
  const int64_t qsb = a.q_stride * EB, ksb = a.k_stride * EB;
  // tokens above 65535 spill into grid.z; the ragged remainder is launched apart
  const int64_t full_z = a.num_tokens / kMaxGridY, rem = a.num_tokens % kMaxGridY;
  if (full_z > 0)
    hipLaunchKernelGGL((rope_seg_kernel<DT, NEOX>), dim3(gx, kMaxGridY, (unsigned)full_z), dim3(64),
                       0, st, a.positions, a.query, a.key, a.cache, qsb, ksb, geom, heads);
  if (rem > 0) {
    const int64_t t0 = full_z * kMaxGridY;
    hipLaunchKernelGGL((rope_seg_kernel<DT, NEOX>), dim3(gx, (unsigned)rem, 1), dim3(64), 0, st,
                       a.positions + t0, reinterpret_cast<char*>(a.query) + t0 * qsb,
                       reinterpret_cast<char*>(a.key) + t0 * ksb, a.cache, qsb, ksb, geom, heads);
  }
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
