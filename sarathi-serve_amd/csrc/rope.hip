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
#include "kv_dest.h"
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

// ---- rotary embedding fused with the paged KV-cache append -------------------------------------
//
// The reference rotates q and k in place (models/llama.py:178) and then copies k and v into the
// paged cache with flashinfer's append_paged_kv_cache (attention/flashinfer_attention_wrapper.py:
// 262-273).  Fused, the rotated k goes straight from registers to its cache entry (k is read once
// and, unless the caller asks for the in-place result too, written once), and v is copied by the
// same launch.  Workgroup ids run over the q segments, the k segments and then the 16-byte pieces
// of the v row of one token.  Needs rot_dim == head_size (so the rotated span is the whole head).
template <int DT, bool NEOX>
__global__ __launch_bounds__(64) void rope_append_seg_kernel(
    void* query, void* key, const void* __restrict__ value, uint32_t q_stride_bytes,
    uint32_t k_stride_bytes, uint32_t v_stride_bytes, uint32_t geom, uint32_t heads,
    uint32_t write_key, const int64_t* __restrict__ positions, const void* __restrict__ cache,
    KvDest d) {
  constexpr int N = VecElems<DT>::value;
  const uint32_t head_bytes = geom & 0xffffu, embed_bytes = geom >> 16;
  const int num_heads = heads & 0xfffu, num_kv_heads = (heads >> 12) & 0xfffu;
  const int slot_shift = heads >> 24;
  const int q_blocks = ((num_heads << slot_shift) + 63) >> 6;
  const int k_blocks = ((num_kv_heads << slot_shift) + 63) >> 6;
  const int64_t tok = (int64_t)blockIdx.z * kMaxGridY + blockIdx.y;
  const uint32_t kv_row_bytes = (uint32_t)num_kv_heads * head_bytes;
  const bool appended = tok < d.nnz;  // uniform over the wave

  if ((int)blockIdx.x >= q_blocks + k_blocks) {  // a piece of the v row: plain copy
    if (!appended) return;
    const uint32_t off = (((int)blockIdx.x - q_blocks - k_blocks) * 64u + threadIdx.x) * 16u;
    const char* src = reinterpret_cast<const char*>(value) + tok * (int64_t)v_stride_bytes;
    const u32x4 v = buf_load16<kStreamLoad>(make_rsrc(src, kv_row_bytes), off);
    char* dst = reinterpret_cast<char*>(d.v_cache) + kv_entry_offset(d, tok);
    buf_store16<kKvStore>(make_rsrc(dst, kv_row_bytes), off, v);
    return;
  }

  const bool is_q = (int)blockIdx.x < q_blocks;
  const int item = ((int)blockIdx.x - (is_q ? 0 : q_blocks)) * 64 + (int)threadIdx.x;
  const int nheads = is_q ? num_heads : num_kv_heads;
  const int h = item >> slot_shift;
  const uint32_t slot = item & ((1 << slot_shift) - 1);
  char* base = reinterpret_cast<char*>(is_q ? query : key) +
               tok * (int64_t)(is_q ? q_stride_bytes : k_stride_bytes);
  const rsrc_t rd = make_rsrc(base, (uint32_t)nheads * head_bytes);
  const uint32_t xoff = h < nheads ? (uint32_t)h * head_bytes + slot * 16u : kClipped;

  u32x4 xr, yr;
  xr = buf_load16<kStreamLoad>(rd, xoff);
  if constexpr (NEOX) yr = buf_load16<kStreamLoad>(rd, xoff + embed_bytes);
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
  // destination of a k segment: resolved while the data loads are in flight
  const bool to_cache = !is_q && appended;
  rsrc_t rk = rd;
  if (to_cache)
    rk = make_rsrc(reinterpret_cast<char*>(d.k_cache) + kv_entry_offset(d, tok), kv_row_bytes);
  const bool in_place = is_q || write_key != 0 || !appended;
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
    const u32x4 px = ox.pack(), py = oy.pack();
    if (in_place) {
      buf_store16<kStreamStore>(rd, xoff, px);
      buf_store16<kStreamStore>(rd, xoff + embed_bytes, py);
    }
    if (to_cache) {
      buf_store16<kKvStore>(rk, xoff, px);
      buf_store16<kKvStore>(rk, xoff + embed_bytes, py);
    }
  } else {
    Vec<DT> o;
#pragma unroll
    for (int i = 0; i < N / 2; ++i) {
      const float xe = x.f[2 * i], ye = x.f[2 * i + 1];
      o.f[2 * i] = mul_r<DT>(xe, c.f[i]) - mul_r<DT>(ye, s.f[i]);
      o.f[2 * i + 1] = mul_r<DT>(ye, c.f[i]) + mul_r<DT>(xe, s.f[i]);
    }
    const u32x4 po = o.pack();
    if (in_place) buf_store16<kStreamStore>(rd, xoff, po);
    if (to_cache) buf_store16<kKvStore>(rk, xoff, po);
  }
}

// Any alignment / rot_dim < head_size: one workgroup per token.
template <int DT, bool NEOX>
__global__ __launch_bounds__(256) void rope_append_generic_kernel(RopeArgs a, const void* value,
                                                                  int64_t v_stride, int write_key,
                                                                  KvDest d) {
  constexpr int EB = ElemBytes<DT>::value;
  const int64_t tok = blockIdx.x;
  const int embed = a.rot_dim >> 1;
  const int64_t crow = a.positions[tok] * a.rot_dim;
  const bool appended = tok < d.nnz;
  const int64_t e = appended ? kv_entry_offset(d, tok) : 0;
  void* kc = reinterpret_cast<char*>(d.k_cache) + e;
  void* vc = reinterpret_cast<char*>(d.v_cache) + e;
  const int nq = a.num_heads * embed;
  const int total = (a.num_heads + a.num_kv_heads) * embed;
  for (int i = threadIdx.x; i < total; i += 256) {
    const bool is_q = i < nq;
    void* arr = is_q ? a.query : a.key;
    const int j = is_q ? i : i - nq;
    const int h = j / embed, r = j - h * embed;
    const int64_t hl = (int64_t)h * a.head_size;  // offset of the head inside its row
    const int64_t hb = tok * (is_q ? a.q_stride : a.k_stride) + hl;
    const int xo = NEOX ? r : 2 * r, yo = NEOX ? embed + r : 2 * r + 1;
    const float c = load_elem<DT>(a.cache, crow + r), s = load_elem<DT>(a.cache, crow + embed + r);
    const float x = load_elem<DT>(arr, hb + xo), y = load_elem<DT>(arr, hb + yo);
    const float ox = mul_r<DT>(x, c) - mul_r<DT>(y, s), oy = mul_r<DT>(y, c) + mul_r<DT>(x, s);
    if (is_q || write_key || !appended) {
      store_elem<DT>(arr, hb + xo, ox);
      store_elem<DT>(arr, hb + yo, oy);
    }
    if (!is_q && appended) {
      store_elem<DT>(kc, hl + xo, ox);
      store_elem<DT>(kc, hl + yo, oy);
    }
  }
  if (!appended) return;
  // the un-rotated tail of every k head, then the v row
  const int tail = a.head_size - a.rot_dim;
  for (int i = threadIdx.x; i < a.num_kv_heads * tail; i += 256) {
    const int h = i / tail, r = a.rot_dim + (i - h * tail);
    const int64_t hl = (int64_t)h * a.head_size + r;
    store_elem<DT>(kc, hl, load_elem<DT>(a.key, tok * a.k_stride + hl));
  }
  (void)EB;
  for (int i = threadIdx.x; i < a.num_kv_heads * a.head_size; i += 256)
    store_elem<DT>(vc, i, load_elem<DT>(value, tok * v_stride + i));
}

template <int DT, bool NEOX>
static int launch_rope_append(const RopeArgs& a, const void* value, int64_t v_stride,
                              int write_key, const KvDest& d, hipStream_t st) {
  constexpr int N = VecElems<DT>::value;
  constexpr int EB = ElemBytes<DT>::value;
  if (a.num_tokens > 0x7fffffffLL) return SARATHI_ERR_UNSUPPORTED;
  const int embed = a.rot_dim / 2;
  const int span = NEOX ? embed : a.rot_dim;
  const int64_t q_row_bytes = (int64_t)a.num_heads * a.head_size * EB;
  const int64_t k_row_bytes = (int64_t)a.num_kv_heads * a.head_size * EB;
  const int64_t qsb = a.q_stride * EB, ksb = a.k_stride * EB, vsb = v_stride * EB;
  const int slots = span / N > 0 ? span / N : 1;
  int slot_shift = 0;
  while ((1 << slot_shift) < slots) ++slot_shift;
  const int64_t head_bytes = (int64_t)a.head_size * EB;
  const bool vec_ok =
      a.rot_dim == a.head_size && (span % N == 0) && (head_bytes % 16 == 0) && (qsb % 16 == 0) &&
      (ksb % 16 == 0) && (vsb % 16 == 0) && ((embed * EB) % (NEOX ? 16 : 8) == 0) &&
      aligned16(a.query) && aligned16(a.key) && aligned16(value) && aligned16(a.cache) &&
      aligned16(d.k_cache) && aligned16(d.v_cache) && d.page_stride_bytes % 16 == 0 &&
      d.entry_stride_bytes % 16 == 0 && q_row_bytes < (int64_t)kClipped &&
      k_row_bytes < (int64_t)kClipped && qsb < (1LL << 32) && ksb < (1LL << 32) &&
      vsb < (1LL << 32) && (1 << slot_shift) == slots && head_bytes < 65536 &&
      embed * EB < 65536 && a.num_heads < 4096 && a.num_kv_heads < 4096;
  if (!vec_ok) {
    hipLaunchKernelGGL((rope_append_generic_kernel<DT, NEOX>), dim3((unsigned)a.num_tokens),
                       dim3(256), 0, st, a, value, v_stride, write_key, d);
    return launch_status();
  }
  const uint32_t geom = (uint32_t)head_bytes | ((uint32_t)(embed * EB) << 16);
  const uint32_t heads =
      (uint32_t)a.num_heads | ((uint32_t)a.num_kv_heads << 12) | ((uint32_t)slot_shift << 24);
  const int64_t q_blocks = ((int64_t)a.num_heads * slots + 63) / 64;
  const int64_t k_blocks = ((int64_t)a.num_kv_heads * slots + 63) / 64;
  const int64_t v_blocks = (k_row_bytes / 16 + 63) / 64;
  const unsigned gx = (unsigned)(q_blocks + k_blocks + v_blocks);
  const int64_t full_z = a.num_tokens / kMaxGridY, rem = a.num_tokens % kMaxGridY;
  if (full_z > 0)
    hipLaunchKernelGGL((rope_append_seg_kernel<DT, NEOX>), dim3(gx, kMaxGridY, (unsigned)full_z),
                       dim3(64), 0, st, a.query, a.key, value, (uint32_t)qsb, (uint32_t)ksb,
                       (uint32_t)vsb, geom, heads, (uint32_t)write_key, a.positions, a.cache, d);
  if (rem > 0) {
    const int64_t t0 = full_z * kMaxGridY;
    KvDest dr = d;
    if (dr.slot_mapping) {
      dr.slot_mapping += t0;
    } else {
      dr.batch_indices += t0;
      dr.positions += t0;
    }
    dr.nnz = d.nnz > t0 ? d.nnz - t0 : 0;
    hipLaunchKernelGGL((rope_append_seg_kernel<DT, NEOX>), dim3(gx, (unsigned)rem, 1), dim3(64), 0,
                       st, reinterpret_cast<char*>(a.query) + t0 * qsb,
                       reinterpret_cast<char*>(a.key) + t0 * ksb,
                       reinterpret_cast<const char*>(value) + t0 * vsb, (uint32_t)qsb,
                       (uint32_t)ksb, (uint32_t)vsb, geom, heads, (uint32_t)write_key,
                       a.positions + t0, a.cache, dr);
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
  if (num_tokens > 0 && (!positions || !query || !key || !cos_sin_cache))
    return SARATHI_ERR_INVALID_ARG;  // empty tensors have no data
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

extern "C" int sarathi_rotary_embedding_append_paged_kv(
    const int64_t* positions, void* query, void* key, const void* value, const void* cos_sin_cache,
    const int32_t* batch_indices, const int32_t* append_positions, void* k_cache, void* v_cache,
    const int32_t* kv_indices, const int32_t* kv_indptr, const int32_t* slot_mapping,
    int64_t num_tokens, int64_t num_append_tokens, int num_heads, int num_kv_heads, int head_size,
    int rot_dim, int64_t query_stride, int64_t key_stride, int64_t value_stride, int page_size,
    int64_t page_stride, int64_t entry_stride, int is_neox, int write_key, int dtype,
    void* stream) {
  using namespace sarathi_hip;
  if (num_tokens > 0 && (!positions || !query || !key || !value || !cos_sin_cache))
    return SARATHI_ERR_INVALID_ARG;
  if (num_append_tokens > 0 &&
      (!k_cache || !v_cache ||
       (!slot_mapping && (!batch_indices || !append_positions || !kv_indices || !kv_indptr))))
    return SARATHI_ERR_INVALID_ARG;
  if (num_tokens < 0 || num_append_tokens < 0 || num_append_tokens > num_tokens ||
      num_heads <= 0 || num_kv_heads <= 0 || head_size <= 0 || rot_dim <= 0 || (rot_dim & 1) ||
      rot_dim > head_size || page_size <= 0)
    return SARATHI_ERR_INVALID_ARG;
  const int64_t kv_row = (int64_t)num_kv_heads * head_size;
  if (query_stride < (int64_t)num_heads * head_size || key_stride < kv_row ||
      value_stride < kv_row || entry_stride < kv_row ||
      page_stride < (int64_t)page_size * entry_stride)
    return SARATHI_ERR_INVALID_ARG;
  if (num_tokens == 0) return SARATHI_OK;
  const int eb = dtype == kF32 ? 4 : 2;
  RopeArgs a{positions, query,     key,          cos_sin_cache, num_tokens, query_stride,
             key_stride, num_heads, num_kv_heads, head_size,     rot_dim};
  KvDest d{batch_indices, append_positions, kv_indices,       kv_indptr,         slot_mapping,
           k_cache,       v_cache,          page_stride * eb, entry_stride * eb, num_append_tokens,
           (int32_t)page_size};
  hipStream_t st = (hipStream_t)stream;
#define SK_ROPE_APPEND(DT)                                                              \
  (is_neox ? launch_rope_append<DT, true>(a, value, value_stride, write_key, d, st)     \
           : launch_rope_append<DT, false>(a, value, value_stride, write_key, d, st))
  switch (dtype) {
    case kBF16: return SK_ROPE_APPEND(kBF16);
    case kF16: return SK_ROPE_APPEND(kF16);
    case kF32: return SK_ROPE_APPEND(kF32);
    default: return SARATHI_ERR_UNSUPPORTED;
  }
#undef SK_ROPE_APPEND
}
