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
// 64 consecutive slots of a token's list of heads (the q heads, then the k heads;
// 8 heads of 128 at bf16) form a segment.  A workgroup is ONE wave that takes up
// to five NeoX (ten GPT-J) consecutive segments of one token:
// at Llama-3-8B's 32 + 8 heads that is the whole token, so its position and its
// cos/sin row are fetched once, all of its loads are in flight before the first
// result is needed, and the launch has one workgroup per token.  (Measured on
// MI355X at 2304 tokens: one wave per segment 9.3 us, one wave per token 8.1 us;
// a launch of N one-wave workgroups costs about 0.2 ns per workgroup in the
// dispatcher alone, 3.5 us for the 11520 of the per-segment layout, and
// multi-wave workgroups lose more to uneven compute-unit load than they gain.)
// Tokens with more segments than that are dealt to two or three waves at mid-size batches
// (plan_rope_chunks), and NeoX heads of 128 bytes are read in memory order with the x and y
// vectors traded between lanes (trade_pairs).
// The token's q row, k row and cos/sin cache row are scalar buffer resources
// (the position is a scalar load issued first and consumed after the data loads
// have been issued); lanes past the last head are clipped by the hardware range
// check, so the kernel has no divergent branches.  Elements at or beyond rot_dim
// inside a head are not touched.
//
// Arithmetic is the reference's scalar_t arithmetic: each product and the final
// sum round to the tensor dtype (csrc/pos_encoding_kernels.cu:32-35):
//   x' = T( T(x*cos) - T(y*sin) ),  y' = T( T(y*cos) + T(x*sin) ).
// The two products of a sum are rounded by one packed conversion.  bf16 on the vector path: a
// result that is exactly zero is stored as +0 also where the reference's arithmetic yields -0;
// everything else is bit-identical to it.
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

// One rotation with the reference's rounding points.  For 16-bit dtypes the two products of each
// sum go through ONE packed conversion (v_cvt_pk_*) and come back as floats.
template <int DT> SK_DEV void rotate(float x, float y, float c, float s, float& ox, float& oy) {
  if constexpr (DT == kBF16) {
    // The two rounded products of a sum stay packed in one register and v_dot2_f32_bf16 forms
    // lo * 1 -/+ hi * 1 + (-0) from it: one instruction instead of two unpacks and an add (a
    // quarter of the kernel's VALU work; 8.4 -> 8.2 us at 2304 tokens).  The products by +-1 are
    // exact.  The instruction truncates its fp32 sum where an fp32 add rounds to nearest; the sum
    // of two bf16 values is either exact in fp32 (exponents at most 16 apart) or within one fp32
    // ulp of the larger term, which the rounding to bf16 that follows maps to the same value, so
    // the stored result is the reference's bit for bit (subnormals included; checked on the GPU
    // over 7e7 operand pairs).  One exception: a sum that is exactly zero comes out as +0 where
    // the reference's arithmetic yields -0.
    const bf16x2 a = __builtin_bit_cast(bf16x2, pack2<kBF16>(x * c, y * s));
    const bf16x2 b = __builtin_bit_cast(bf16x2, pack2<kBF16>(y * c, x * s));
    ox = __builtin_amdgcn_fdot2_f32_bf16(a, __builtin_bit_cast(bf16x2, 0xbf803f80u), -0.0f, false);
    oy = __builtin_amdgcn_fdot2_f32_bf16(b, __builtin_bit_cast(bf16x2, 0x3f803f80u), -0.0f, false);
  } else {
    const f32x2 a = rnd2<DT>(x * c, y * s);
    const f32x2 b = rnd2<DT>(y * c, x * s);
    ox = a.x - a.y;
    oy = b.x + b.y;
  }
}

// Rotates the 16-byte slot(s) of one lane: NeoX x vector `xr` and y vector `yr`; GPT-J only `xr`
// (interleaved pairs).  `cr`/`sr` hold the matching cos / sin values (GPT-J: in the low half).
template <int DT, bool NEOX>
SK_DEV void rotate_slot(u32x4& xr, u32x4& yr, const Vec<DT>& c, const Vec<DT>& s) {
  constexpr int N = VecElems<DT>::value;
  Vec<DT> x;
  x.unpack(xr);
  if constexpr (NEOX) {
    Vec<DT> y, ox, oy;
    y.unpack(yr);
#pragma unroll
    for (int i = 0; i < N; ++i) rotate<DT>(x.f[i], y.f[i], c.f[i], s.f[i], ox.f[i], oy.f[i]);
    xr = ox.pack();
    yr = oy.pack();
  } else {
    Vec<DT> o;
#pragma unroll
    for (int i = 0; i < N / 2; ++i)
      rotate<DT>(x.f[2 * i], x.f[2 * i + 1], c.f[i], s.f[i], o.f[2 * i], o.f[2 * i + 1]);
    xr = o.pack();
  }
}

// Heads of 128 bytes (NeoX, head_size 64 in a 16-bit type, fully rotated): the x half and the y
// half of a head share one 128-byte line, and a load that takes the x vectors of 16 heads touches
// half of each of 16 lines, the y load the other halves.  The paired layout reads memory in order
// instead: eight consecutive lanes take the eight 16-byte pieces of one head (x x x x y y y y),
// the wave's first load the first eight heads of the segment and the second load the next eight,
// each 1 KiB of consecutive bytes.  A lane then holds the same piece of two heads; the lanes of a
// head's x pieces trade their second register for the first register of the lane four up, after
// which every lane holds an x vector and the matching y vector of ONE head (lanes 0-3 of a group
// of eight the first load's head, lanes 4-7 the second load's), exactly what rotate_slot() takes.
// The same trade after the rotation puts the results back in memory order.  Two DPP moves per
// dword, bank-masked so that each direction writes only its receivers.
SK_DEV void trade_pairs(u32x4& lo, u32x4& hi) {
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int a = (int)lo[i], b = (int)hi[i];
    // lanes 0-3 and 8-11 of each row of 16: hi <- lo of the lane four up (row_shl:4)
    const int nb = __builtin_amdgcn_update_dpp(b, a, 0x104, 0xf, 0x5, false);
    // lanes 4-7 and 12-15: lo <- hi of the lane four down (row_shr:4)
    const int na = __builtin_amdgcn_update_dpp(a, b, 0x114, 0xf, 0xa, false);
    lo[i] = (uint32_t)na;
    hi[i] = (uint32_t)nb;
  }
}

// Store policy of the in-place results.  With a wave per token the rows it rewrites are still in
// L2 from its own loads; a non-temporal write-back store measured 2 % faster there than the
// write-through store that wins for out-of-place streams and for the one-segment shape.
constexpr int kNtStore = 2;

// What a launch works on.  The two row arrays are called A and B: A is whichever of query / key
// starts lower in memory, and B is reached THROUGH A's per-token buffer resource at byte offset
// delta0 + token * delta_step (callers pass views of one packed qkv buffer, so this is a small
// constant), which leaves one resource and no per-segment selects in the kernel.  A token's
// list of heads is A's heads, then B's, cut into segments of 64 slots.
//   geom  = head_bytes | embed_bytes << 16          (bytes of one head / of rot_dim/2)
//   heads = heads of A | heads of B << 12 | slot_shift << 24 | log2 gcd(chunks, 8) << 28 |
//           (A is the key array) << 31     (the gcd field is filled in at launch)
// slot_shift = log2(16-byte slots per head), at most 6; NeoX counts the slots of the x half,
// GPT-J those of the whole rotated span.
// Everything the first loads need sits in the first 56 bytes of the kernel arguments, which the
// hardware preloads into scalar registers at wave launch.
struct RopeLaunch {
  const int64_t* positions;
  void* a;
  const void* cache;
  int64_t a_stride_bytes;
  int64_t delta0;
  int64_t delta_step;
  uint32_t geom;
  uint32_t heads;
};
constexpr uint32_t kRopeAIsKey = 0x80000000u;

// One wave: SPW consecutive segments of one token.  FLAT: the launch is one-dimensional with one
// wave per token (a (1, tokens) grid dispatches measurably slower than a (tokens) grid);
// otherwise grid = (chunks, tokens) and chunk c is segments [c * SPW, (c + 1) * SPW).
// The position is a scalar load that the compiler places behind the data loads; moving it, or the
// cos/sin loads that depend on it, ahead of them measured 5-10 % slower.
//
// APPEND: the rotary embedding fused with the paged KV-cache append.  The reference rotates q and
// k in place (models/llama.py:178) and then copies k and v into the paged cache with flashinfer's
// append_paged_kv_cache (attention/flashinfer_attention_wrapper.py:262-273).  Fused, the rotated k
// goes straight from registers to its cache entry (k is read once and, unless the caller asks for
// the in-place result too, written once), and the v row is copied by the same wave: with
// rot_dim == head_size, which this path requires, the x and y vectors of a k segment cover its
// heads completely, so the v vectors at the same two offsets cover the same heads of the v row.
// The entry address is resolved with scalar loads while the data loads are in flight.
template <int DT, bool NEOX, int SPW, bool FLAT, bool APPEND, bool PAIRED>
SK_DEV void rope_wave(const int64_t* __restrict__ positions, void* a,
                      const void* __restrict__ cache, int64_t a_stride_bytes, int64_t delta0,
                      int64_t delta_step, uint32_t geom, uint32_t heads,
                      const void* __restrict__ value, int64_t v_stride_bytes, uint32_t write_key,
                      const KvDest* d) {
  constexpr int SP = SPW == 1 ? kStreamStore : kNtStore;
  // Cache-entry stores: non-temporal from the waves that hold several segments, the default
  // write-back policy from one-segment waves (32 + 32 heads at 4608 tokens 43.6 -> 37.8 us,
  // 32 + 8 heads 20.4 -> 19.2; the other way round a whole-token wave loses 9 % at 2304 tokens).
  constexpr int KSP = SPW == 1 ? kKvStore : kKvStoreFused;
  const uint32_t head_bytes = geom & 0xffffu, embed_bytes = geom >> 16;
  const uint32_t heads_a = heads & 0xfffu, heads_b = (heads >> 12) & 0xfffu;
  const uint32_t sh = (heads >> 24) & 0x7u;
  const bool a_is_key = (heads & kRopeAIsKey) != 0;
  const int64_t tok = FLAT ? (int64_t)blockIdx.x : (int64_t)blockIdx.z * kMaxGridY + blockIdx.y;
  uint32_t chunk = FLAT ? 0u : blockIdx.x;
  if constexpr (APPEND && !FLAT) {
    // Workgroup ids go round the eight XCDs, and a token's key segments (twice the loads and
    // stores of a query segment) sit at fixed places in its list: when the list length shares a
    // factor g with 8 they would always land on the same 8 / g XCDs.  Exchanging chunks inside
    // aligned groups of g, by an amount that steps every 8 / g tokens, spreads them over all eight.
    const uint32_t lg = (heads >> 28) & 3u;  // log2 g, from the host
    chunk ^= ((uint32_t)tok >> (3u - lg)) & ((1u << lg) - 1u);
  }
  const uint32_t delta = (uint32_t)(delta0 + tok * delta_step);
  // A's row and, beyond it, B's: per-access validity is decided below (kClipped), the resource
  // only has to reach past B's row
  const rsrc_t r = make_rsrc(reinterpret_cast<char*>(a) + tok * a_stride_bytes, 0x7fffffffu);
  // B's heads follow A's in the token's list.  With the append fused in, A's span is padded to
  // whole segments, so that a segment is all key heads or none (the append decisions are then
  // uniform over the wave); without it B's first head takes the lane after A's last.
  const uint32_t a_pad = APPEND ? (((heads_a << sh) + 63u) >> 6) << (6 - sh) : heads_a;
  const uint32_t slot = threadIdx.x & ((1u << sh) - 1u);
  // PAIRED (sh == 2): the lane's piece of its head in memory order, see trade_pairs()
  const uint32_t h0 = chunk * (uint32_t)(SPW << (6 - sh)) + (threadIdx.x >> (PAIRED ? 3 : sh));
  const uint32_t piece = (threadIdx.x & 7u) * 16u;  // PAIRED only

  const uint32_t kv_row_bytes = (a_is_key ? heads_a : heads_b) * head_bytes;

  u32x4 xr[SPW], yr[SPW], vx[SPW], vy[SPW];
  uint32_t xoff[SPW];   // offset of the lane's first vector (x) from A's row
  uint32_t koff[SPW];   // APPEND: the same offset inside the k / v row
  // The second vector of a lane: the y vector of the same head, embed_bytes on; PAIRED: the same
  // piece of the head eight heads on, at offsets of its own.
  uint32_t yoff2[PAIRED ? SPW : 1], kyoff2[PAIRED ? SPW : 1];
  auto yoff = [&](int j) -> uint32_t {
    if constexpr (PAIRED) return yoff2[j];
    else return xoff[j] + embed_bytes;
  };
  auto kyoff = [&](int j) -> uint32_t {
    if constexpr (PAIRED) return kyoff2[j];
    else return koff[j] + embed_bytes;
  };
  // where a head's piece lies: from A's row (query / key traffic) and inside its own row
  auto locate = [&](uint32_t h, uint32_t& from_a, uint32_t& in_row) {
    const uint32_t hb = h - a_pad;  // wraps to a huge value while h is inside A's padded span
    const bool in_a = h < heads_a, in_b = hb < heads_b;
    const uint32_t row_off = (in_a ? h : hb) * head_bytes + piece;
    from_a = (in_a || in_b) ? row_off + (in_a ? 0u : delta) : kClipped;
    in_row = (in_a || in_b) ? row_off : kClipped;
  };
  // The query / key loads need nothing beyond the kernel arguments that the hardware preloads into
  // scalar registers (the first 14 dwords), so they leave before the wave has waited for anything;
  // the value loads and the append bookkeeping read later arguments and follow them.
#pragma unroll
  for (int j = 0; j < SPW; ++j) {
    const uint32_t h = h0 + (uint32_t)(j << (6 - sh));
    if constexpr (PAIRED) {
      locate(h, xoff[j], koff[j]);
      locate(h + 8u, yoff2[j], kyoff2[j]);
    } else {
      const uint32_t hb = h - a_pad;  // wraps to a huge value while h is inside A's padded span
      const bool in_a = h < heads_a, in_b = hb < heads_b;
      const uint32_t row_off = (in_a ? h : hb) * head_bytes + slot * 16u;
      xoff[j] = (in_a || in_b) ? row_off + (in_a ? 0u : delta) : kClipped;
      koff[j] = (in_a || in_b) ? row_off : kClipped;
    }
    xr[j] = buf_load16<kStreamLoad>(r, xoff[j]);
    if constexpr (NEOX) yr[j] = buf_load16<kStreamLoad>(r, yoff(j));
  }
  bool appended = false;
  if constexpr (APPEND) {
    __builtin_amdgcn_sched_barrier(0);
    appended = tok < d->nnz;  // uniform over the wave
#pragma unroll
    for (int j = 0; j < SPW; ++j) {
      // a segment lies wholly in A's padded span or wholly in B's: uniform
      const bool seg_in_a = (chunk * SPW + j) < (a_pad >> (6 - sh));
      const bool is_k = seg_in_a == a_is_key;
      if (is_k && appended) {
        const rsrc_t rv = make_rsrc(
            reinterpret_cast<const char*>(value) + tok * v_stride_bytes, kv_row_bytes);
        vx[j] = buf_load16<kStreamLoad>(rv, koff[j]);
        if constexpr (NEOX) vy[j] = buf_load16<kStreamLoad>(rv, kyoff(j));
      }
    }
  }
  // everything above is issued before the first wait (the position's)
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
  // destination of the k and v rows: resolved while the data loads are in flight
  int64_t entry = 0;
  if constexpr (APPEND) {
    if (appended) entry = kv_entry_offset(*d, tok);
  }
  __builtin_amdgcn_sched_barrier(0);

  Vec<DT> c, s;
  c.unpack(cr);
  s.unpack(sr);
  // Rotate every segment first and issue the stores afterwards, back to back: a wave that starts
  // writing while its other segments (and its neighbours' rows) are still being read slows those
  // reads down.  2048-2560 tokens of 32 + 8 heads: 7-9 % faster (2304: 8.2 -> 7.6 us); within 4 %
  // either way at 1536 and 3072 tokens.
#pragma unroll
  for (int j = 0; j < SPW; ++j) {
    if constexpr (PAIRED) trade_pairs(xr[j], yr[j]);
    rotate_slot<DT, NEOX>(xr[j], yr[j], c, s);
    if constexpr (PAIRED) trade_pairs(xr[j], yr[j]);
  }
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int j = 0; j < SPW; ++j) {
    bool in_place = true;
    if constexpr (APPEND) {
      const bool seg_in_a = (chunk * SPW + j) < (a_pad >> (6 - sh));
      const bool is_k = seg_in_a == a_is_key;
      in_place = !is_k || write_key != 0 || !appended;
      if (is_k && appended) {  // uniform
        const rsrc_t rkc = make_rsrc(reinterpret_cast<char*>(d->k_cache) + entry, kv_row_bytes);
        const rsrc_t rvc = make_rsrc(reinterpret_cast<char*>(d->v_cache) + entry, kv_row_bytes);
        buf_store16<KSP>(rkc, koff[j], xr[j]);
        if constexpr (NEOX) buf_store16<KSP>(rkc, kyoff(j), yr[j]);
        buf_store16<KSP>(rvc, koff[j], vx[j]);
        if constexpr (NEOX) buf_store16<KSP>(rvc, kyoff(j), vy[j]);
      }
    }
    if (in_place) {
      buf_store16<SP>(r, xoff[j], xr[j]);
      if constexpr (NEOX) buf_store16<SP>(r, yoff(j), yr[j]);
    }
  }
}

template <int DT, bool NEOX, int SPW, bool FLAT, bool PAIRED>
__global__ __launch_bounds__(64) void rope_tok_kernel(
    const int64_t* __restrict__ positions, void* a, const void* __restrict__ cache,
    int64_t a_stride_bytes, int64_t delta0, int64_t delta_step, uint32_t geom, uint32_t heads) {
  rope_wave<DT, NEOX, SPW, FLAT, false, PAIRED>(positions, a, cache, a_stride_bytes, delta0,
                                                delta_step, geom, heads, nullptr, 0, 0, nullptr);
}

template <int DT, bool NEOX, int SPW, bool FLAT, bool PAIRED>
__global__ __launch_bounds__(64) void rope_append_tok_kernel(
    const int64_t* __restrict__ positions, void* a, const void* __restrict__ cache,
    int64_t a_stride_bytes, int64_t delta0, int64_t delta_step, uint32_t geom, uint32_t heads,
    const void* __restrict__ value, int64_t v_stride_bytes, uint32_t write_key, KvDest d) {
  rope_wave<DT, NEOX, SPW, FLAT, true, PAIRED>(positions, a, cache, a_stride_bytes, delta0,
                                               delta_step, geom, heads, value, v_stride_bytes,
                                               write_key, &d);
}

// Segments a wave takes.  One wave per segment (a grid of segments x tokens) is the general
// shape.  A whole token per wave (a flat grid of tokens, all of the token's loads in flight at
// once, position and cache row fetched once, every store behind the last rotation) wins where that
// grid is five to ten waves per compute unit, which is where a 2048-token chunk plus its
// decode tokens falls.  Measured on separately allocated tensors, bf16, 32 query + 8 key heads of
// 128, cold, whole token / one segment per wave: 1024 tokens 5.2 / 5.0 us, 1280 5.8 / 5.8, 1536
// 6.4 / 6.8, 2048 7.2 / 8.4, 2304 8.1 / 9.3, 2560 9.9 / 10.2, 2688 10.7 / 10.5, 2816 11.3 / 10.9,
// 3072 12.2 / 11.6, 4096 16.0 / 14.9 (on inputs still in the memory-side cache the whole token
// wins throughout).
// With 64 query heads (nine segments, i.e. two chunks of five against nine waves of one) 4608
// tokens take 31.5 against 27.3 us.
// Per token the whole-token shape costs 3.3 ns at nine waves per compute unit, 3.6 at ten and 3.9
// from eleven on, whatever the positions are: up to about ten such waves per unit the loads of the
// whole batch are in flight at once, so the launch is one read phase followed by one write phase;
// beyond that the later waves' loads queue behind the first ones and meet their stores.
// A wave's loads in flight, not its segment count, are what the limit is about: a NeoX segment is
// two 16-byte loads per lane, a GPT-J segment one.
constexpr int kMaxSegsPerWave = 5;       // NeoX
constexpr int kMaxSegsPerWaveGptj = 10;
struct RopeChunks {
  int chunks, spw;
};
// With the cache append fused in (the value row's loads and the cache stores ride along), the
// whole-token shape wins over a wider range, same harness: 1024 tokens 5.5 / 6.5 us, 1536 6.8 / 8.2,
// 2048 8.3 / 10.2, 2304 9.7 / 11.2, 2560 11.4 / 12.3, 3072 13.5 / 14.3, 4096 17.8 / 18.3; equal at
// 512 (5.5), behind at 4608 (21.1 / 20.4).
//
// Tokens of more than max_segs segments (64 query heads of 128, or as many key heads as query
// heads) can be dealt to a few waves of up to max_segs segments each, in equal parts where the
// count allows (nine segments as 3 x 3, eight as 2 x 4).  That wins in the same place, four to
// eight such waves per compute unit, i.e. at 500-1000 tokens; bf16, cold, one wave per segment ->
// dealt: 32 + 32 heads, 768 tokens 5.9 -> 5.1 us, 1024 7.2 -> 6.4 (1280 equal); 40 + 40 heads, 640
// tokens 6.0 -> 5.4, 1024 8.5 -> 8.0 (1152: 9.4 against 9.9); 64 + 8 heads, 512 tokens 4.8 -> 4.5,
// 768 6.1 -> 5.7 (896: 7.0 against 7.2); 64 + 64 heads, 512 tokens 7.2 -> 6.4 (640 equal).  With
// the append fused in the gain ends earlier, at five waves per unit (40 + 40 heads, 640 tokens
// 8.9 -> 8.6, 768 10.4 against 10.5; 32 + 32 heads, 768 tokens 9.4 -> 8.1, 1024 equal), unless
// the key heads are a small part of the token, where it lasts to twelve waves per unit: 56 + 8
// heads at 1024 tokens 9.4 -> 6.8 us, 1536 12.5 -> 11.2 (2304 equal, behind from there); 64 + 8
// heads at 1024 tokens 8.8 -> 7.5 (1280 equal); 40 + 8 heads at 1280 tokens 8.3 -> 6.8, 1536
// 9.4 -> 8.8 (2048 behind).
static RopeChunks plan_rope_chunks(int64_t segs, int64_t key_segs, int64_t tokens, int max_segs,
                                   bool append) {
  const int64_t units = compute_units();
  RopeChunks p;
  p.chunks = (int)(segs < 1 ? 1 : segs);
  p.spw = 1;
  if (segs <= max_segs) {
    // tokens of one or two segments (tensor-parallel shards: 8 + 1 heads): the whole token at
    // every size measured, 3072 tokens 4.8 -> 4.5 us, 4608 6.3 -> 5.5, 8192 9.3 -> 8.4
    const bool in_range = segs <= 2 ? tokens >= 5 * units
                          : append  ? tokens >= 4 * units && tokens <= 16 * units
                                    : tokens >= 5 * units && 4 * tokens <= 41 * units;
    if (in_range) {
      p.chunks = 1;
      p.spw = (int)(segs < 1 ? 1 : segs);
    }
    return p;
  }
  int64_t parts = (segs + max_segs - 1) / max_segs;
  if (segs % parts != 0 && segs % (parts + 1) == 0) ++parts;
  const int64_t waves = parts * tokens;
  const int64_t lo = append ? 3 : 4, hi = !append ? 8 : 4 * key_segs > segs ? 5 : 12;
  if (waves >= lo * units && waves <= hi * units) {
    p.chunks = (int)parts;
    p.spw = (int)((segs + parts - 1) / parts);
  }
  return p;
}

// How query and key rows map onto the A / B arrays of a launch.  `pieces` is 1 when B can be
// reached through A's resource for every token, else 2 (query alone, then key alone).
struct RopeAnchor {
  int pieces;
  RopeLaunch l[2];
  int64_t segs[2];
};
static RopeAnchor plan_rope_anchor(const RopeArgs& a, int eb, int slots, int slot_shift,
                                   uint32_t geom, bool append) {
  const int64_t qsb = a.q_stride * eb, ksb = a.k_stride * eb;
  const int64_t q_row = (int64_t)a.num_heads * a.head_size * eb;
  const int64_t k_row = (int64_t)a.num_kv_heads * a.head_size * eb;
  char* q = reinterpret_cast<char*>(a.query);
  char* k = reinterpret_cast<char*>(a.key);
  const int64_t last = a.num_tokens - 1;
  const int64_t d_first = k - q, d_last = d_first + last * (ksb - qsb);  // key row - query row
  const int64_t q_blocks = ((int64_t)a.num_heads * slots + 63) / 64;
  const int64_t k_blocks = ((int64_t)a.num_kv_heads * slots + 63) / 64;
  // segments of a token whose two rows go out in one launch: see a_pad in rope_wave()
  const int64_t joined =
      append ? q_blocks + k_blocks : ((int64_t)(a.num_heads + a.num_kv_heads) * slots + 63) / 64;
  const int64_t reach = (int64_t)kClipped - 64;  // offsets, + embed_bytes, must stay below kClipped
  const uint32_t sh = (uint32_t)slot_shift << 24;
  RopeAnchor p;
  if (a.num_kv_heads == 0 || (d_first >= 0 && d_last >= 0 && d_first + k_row < reach &&
                              d_last + k_row < reach)) {
    p.pieces = 1;  // A = query, B = key
    p.l[0] = {a.positions, q, a.cache, qsb, d_first, ksb - qsb, geom,
              (uint32_t)a.num_heads | ((uint32_t)a.num_kv_heads << 12) | sh};
    p.segs[0] = joined;
  } else if (d_first <= 0 && d_last <= 0 && -d_first + q_row < reach && -d_last + q_row < reach) {
    p.pieces = 1;  // A = key, B = query
    p.l[0] = {a.positions, k, a.cache, ksb, -d_first, qsb - ksb, geom,
              (uint32_t)a.num_kv_heads | ((uint32_t)a.num_heads << 12) | sh | kRopeAIsKey};
    p.segs[0] = joined;
  } else {
    p.pieces = 2;  // too far apart (or crossing): each array on its own
    p.l[0] = {a.positions, q, a.cache, qsb, 0, 0, geom, (uint32_t)a.num_heads | sh};
    p.segs[0] = q_blocks;
    p.l[1] = {a.positions, k, a.cache, ksb, 0, 0, geom,
              (uint32_t)a.num_kv_heads | sh | kRopeAIsKey};
    p.segs[1] = k_blocks;
  }
  return p;
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

// Launches the wave kernels for one piece of an anchor plan.  One wave per token goes out as a
// one-dimensional grid; chunked tokens as (chunks, tokens), with tokens above 65535 spilling into
// grid.z and the ragged remainder launched apart.
template <int DT, bool NEOX, bool APPEND>
static int launch_rope_piece(const RopeLaunch& l, int64_t segs, int64_t num_tokens,
                             const void* value, int64_t vsb, int write_key, const KvDest* d,
                             hipStream_t st) {
  if (segs <= 0) return SARATHI_OK;
  const uint32_t sh = (l.heads >> 24) & 0x7u;
  const int64_t key_heads = (l.heads & kRopeAIsKey) ? (l.heads & 0xfffu) : ((l.heads >> 12) & 0xfffu);
  const RopeChunks plan =
      plan_rope_chunks(segs, ((key_heads << sh) + 63) >> 6, num_tokens,
                       NEOX ? kMaxSegsPerWave : kMaxSegsPerWaveGptj, APPEND);
  const bool flat = plan.chunks == 1;
  const int64_t full_z = flat ? 0 : num_tokens / kMaxGridY;
  const int64_t rem = flat ? num_tokens : num_tokens % kMaxGridY;
  const int64_t t0 = full_z * kMaxGridY;
  // arguments of the remainder launch: everything indexed by token moves on by t0
  RopeLaunch lr = l;
  lr.positions += t0;
  lr.a = reinterpret_cast<char*>(l.a) + t0 * l.a_stride_bytes;
  lr.delta0 += t0 * l.delta_step;
  KvDest d0{}, dr{};
  const void* value_r = value;
  if constexpr (APPEND) {
    d0 = *d;
    dr = *d;
    if (dr.slot_mapping) {
      dr.slot_mapping += t0;
    } else {
      dr.batch_indices += t0;
      dr.positions += t0;
    }
    dr.nnz = d->nnz > t0 ? d->nnz - t0 : 0;
    value_r = reinterpret_cast<const char*>(value) + t0 * vsb;
  }
  // see the chunk exchange in rope_wave()
  uint32_t lg = 0;
  while (lg < 3 && (plan.chunks & (1 << lg)) == 0) ++lg;
  const uint32_t heads_arg = l.heads | (lg << 28);
  const dim3 block(64);
  const dim3 grid_full((unsigned)plan.chunks, kMaxGridY, (unsigned)full_z);
  const dim3 grid_rem = flat ? dim3((unsigned)rem) : dim3((unsigned)plan.chunks, (unsigned)rem, 1);
  // heads of 128 bytes, fully rotated: memory-order loads (trade_pairs)
  const bool paired = NEOX && (l.geom & 0xffffu) == 128u && (l.geom >> 16) == 64u;
#define SK_ROPE_GO1(SPW, FLAT, PAIRED, GRID, L, VALUE, DEST)                                     \
  do {                                                                                           \
    if constexpr (APPEND)                                                                        \
      hipLaunchKernelGGL((rope_append_tok_kernel<DT, NEOX, SPW, FLAT, PAIRED>), GRID, block, 0,  \
                         st, L.positions, L.a, L.cache, L.a_stride_bytes, L.delta0,              \
                         L.delta_step, L.geom, heads_arg, VALUE, vsb, (uint32_t)write_key,       \
                         DEST);                                                                  \
    else                                                                                         \
      hipLaunchKernelGGL((rope_tok_kernel<DT, NEOX, SPW, FLAT, PAIRED>), GRID, block, 0, st,     \
                         L.positions, L.a, L.cache, L.a_stride_bytes, L.delta0, L.delta_step,    \
                         L.geom, heads_arg);                                                     \
  } while (0)
#define SK_ROPE_GO(SPW, FLAT, GRID, L, VALUE, DEST)                                              \
  do {                                                                                           \
    if constexpr (NEOX) {                                                                        \
      if (paired) {                                                                              \
        SK_ROPE_GO1(SPW, FLAT, true, GRID, L, VALUE, DEST);                                      \
        break;                                                                                   \
      }                                                                                          \
    }                                                                                            \
    SK_ROPE_GO1(SPW, FLAT, false, GRID, L, VALUE, DEST);                                         \
  } while (0)
#define SK_ROPE_LAUNCH(SPW)                                                \
  case SPW:                                                                \
    if (flat) {                                                            \
      SK_ROPE_GO(SPW, true, grid_rem, lr, value_r, dr);                    \
    } else {                                                               \
      if (full_z > 0) SK_ROPE_GO(SPW, false, grid_full, l, value, d0);     \
      if (rem > 0) SK_ROPE_GO(SPW, false, grid_rem, lr, value_r, dr);      \
    }                                                                      \
    break;
  switch (plan.spw) {
    SK_ROPE_LAUNCH(1) SK_ROPE_LAUNCH(2) SK_ROPE_LAUNCH(3) SK_ROPE_LAUNCH(4) SK_ROPE_LAUNCH(5)
    default:
      if constexpr (!NEOX) {
        switch (plan.spw) {
          SK_ROPE_LAUNCH(6) SK_ROPE_LAUNCH(7) SK_ROPE_LAUNCH(8) SK_ROPE_LAUNCH(9) SK_ROPE_LAUNCH(10)
          default: return SARATHI_ERR_UNSUPPORTED;
        }
      } else {
        return SARATHI_ERR_UNSUPPORTED;
      }
  }
#undef SK_ROPE_LAUNCH
#undef SK_ROPE_GO
#undef SK_ROPE_GO1
  return launch_status();
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
  // the packed-argument kernel needs a power-of-two number of slots per head, at most a wave's
  // worth (so a lane keeps its slot, hence its cos/sin vectors, across segments), and fields that
  // fit their bit widths
  const bool packable = (1 << slot_shift) == slots && slots <= 64 && head_bytes < 65536 &&
                        embed * EB < 65536 &&
                        a.num_heads < 4096 && a.num_kv_heads < 4096;
  if (!packable) {
    hipLaunchKernelGGL((rope_generic_kernel<DT, NEOX>), dim3((unsigned)a.num_tokens), dim3(256),
                       0, st, a);
    return launch_status();
  }
  const uint32_t geom = (uint32_t)head_bytes | ((uint32_t)(embed * EB) << 16);
  const RopeAnchor plan = plan_rope_anchor(a, EB, slots, slot_shift, geom, false);
  for (int i = 0; i < plan.pieces; ++i) {
    const int rc = launch_rope_piece<DT, NEOX, false>(plan.l[i], plan.segs[i], a.num_tokens,
                                                      nullptr, 0, 0, nullptr, st);
    if (rc != SARATHI_OK) return rc;
  }
  return SARATHI_OK;
}

// ---- rotary embedding fused with the paged KV-cache append: element-wise fallback ------------
//
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
      k_row_bytes < (int64_t)kClipped && (1 << slot_shift) == slots && slots <= 64 &&
      head_bytes < 65536 &&
      embed * EB < 65536 && a.num_heads < 4096 && a.num_kv_heads < 4096;
  if (!vec_ok) {
    hipLaunchKernelGGL((rope_append_generic_kernel<DT, NEOX>), dim3((unsigned)a.num_tokens),
                       dim3(256), 0, st, a, value, v_stride, write_key, d);
    return launch_status();
  }
  const uint32_t geom = (uint32_t)head_bytes | ((uint32_t)(embed * EB) << 16);
  const RopeAnchor plan = plan_rope_anchor(a, EB, slots, slot_shift, geom, true);
  for (int i = 0; i < plan.pieces; ++i) {
    const int rc = launch_rope_piece<DT, NEOX, true>(plan.l[i], plan.segs[i], a.num_tokens, value,
                                                     vsb, write_key, &d, st);
    if (rc != SARATHI_OK) return rc;
  }
  return SARATHI_OK;
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
