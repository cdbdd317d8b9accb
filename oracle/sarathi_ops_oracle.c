/*
 * TEST INFRASTRUCTURE ONLY.  CPU restatement, in plain C, of the arithmetic of
 * Sarathi-Serve's csrc op library.  Nothing the product ships may include,
 * link, import or call this file; it exists so tests, the smoke check and the
 * benchmark's cpu_baseline leg have something to compare the HIP kernels with.
 *
 * Every function simulates the reference kernel it cites: the same element to
 * thread assignment, the same accumulation order, and a rounding to the tensor
 * dtype at every point where the reference's `scalar_t` arithmetic rounds.
 * Build with contraction off (gcc -O2 -ffp-contract=off, no fast-math) so the
 * only fused multiply-adds are the explicit fmaf() calls below.
 *
 * What cannot be pinned from a CPU: the last-ulp behaviour of CUDA's expf,
 * rsqrtf and tanhf.  This file uses correctly rounded rsqrt (via double) and
 * the C library's expf/tanhf instead.
 *
 * Parity unpinned: the non-power-of-two / >256 expert branch of
 * oracle_topk_softmax follows the published algorithm of cub::BlockReduce
 * (CUDA toolkit, version unpinned by the reference), which no reference test
 * or fixture covers.
 *
 * dtype codes: 0 = float32, 1 = float16, 2 = bfloat16.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define DT_F32 0
#define DT_F16 1
#define DT_BF16 2

/* ------------------------------------------------------------------ scalars */

static inline uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

/* float -> bfloat16, round to nearest even; NaN stays a quiet NaN. */
static inline uint16_t f32_to_bf16(float f) {
  uint32_t u = f2u(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}
static inline float bf16_to_f32(uint16_t h) { return u2f((uint32_t)h << 16); }

/* float -> IEEE binary16, round to nearest even, with subnormals. */
static inline uint16_t f32_to_f16(float f) {
  uint32_t u = f2u(f);
  uint32_t sign = (u >> 16) & 0x8000u;
  uint32_t a = u & 0x7fffffffu;
  if (a > 0x7f800000u) return (uint16_t)(sign | 0x7e00u);  /* NaN */
  if (a >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u); /* >= 65520 -> inf */
  if (a < 0x33000001u) return (uint16_t)sign;              /* <= 2^-25 -> 0 */
  int32_t e = (int32_t)(a >> 23) - 127;
  uint32_t m = (a & 0x7fffffu) | 0x800000u;
  if (e < -14) { /* subnormal result: shift so that the ulp is 2^-24 */
    int shift = 13 + (-14 - e);
    uint32_t q = m >> shift;
    uint32_t rem = m & ((1u << shift) - 1u);
    uint32_t half = 1u << (shift - 1);
    if (rem > half || (rem == half && (q & 1u))) q++;
    return (uint16_t)(sign | q);
  }
  uint32_t q = ((uint32_t)(e + 15) << 10) | ((m >> 13) & 0x3ffu);
  uint32_t rem = m & 0x1fffu;
  if (rem > 0x1000u || (rem == 0x1000u && (q & 1u))) q++; /* may carry into exp */
  return (uint16_t)(sign | q);
}
static inline float f16_to_f32(uint16_t h) {
  uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
  uint32_t e = (h >> 10) & 0x1fu;
  uint32_t m = h & 0x3ffu;
  if (e == 0) {
    if (m == 0) return u2f(sign);
    float v = (float)m * 5.9604644775390625e-8f; /* m * 2^-24, exact */
    return sign ? -v : v;
  }
  if (e == 31) return u2f(sign | 0x7f800000u | (m << 13));
  return u2f(sign | ((e + 112u) << 23) | (m << 13));
}

/* Round a float to the tensor dtype and widen it again: what a cast to
 * `scalar_t` followed by a use in float arithmetic does in the reference. */
static inline float rnd(float f, int dt) {
  if (dt == DT_BF16) return bf16_to_f32(f32_to_bf16(f));
  if (dt == DT_F16) return f16_to_f32(f32_to_f16(f));
  return f;
}
static inline float ld(const void* p, int64_t i, int dt) {
  if (dt == DT_BF16) return bf16_to_f32(((const uint16_t*)p)[i]);
  if (dt == DT_F16) return f16_to_f32(((const uint16_t*)p)[i]);
  return ((const float*)p)[i];
}
static inline void st(void* p, int64_t i, int dt, float v) {
  if (dt == DT_BF16) ((uint16_t*)p)[i] = f32_to_bf16(v);
  else if (dt == DT_F16) ((uint16_t*)p)[i] = f32_to_f16(v);
  else ((float*)p)[i] = v;
}

/* exported for tests of the conversions themselves */
uint16_t oracle_f32_to_bf16(float f) { return f32_to_bf16(f); }
uint16_t oracle_f32_to_f16(float f) { return f32_to_f16(f); }
float oracle_f16_to_f32(uint16_t h) { return f16_to_f32(h); }

/* ------------------------------------------------------------ block reduce */

/* csrc/reduction_utils.cuh:50-59: xor butterfly over the 32 lanes of a warp.
 * After it every lane holds the same sum; lanes are simulated together. */
static void warp_butterfly_sum(float* v /*[32]*/) {
  float t[32];
  for (int mask = 16; mask > 0; mask >>= 1) {
    for (int l = 0; l < 32; ++l) t[l] = v[l] + v[l ^ mask];
    memcpy(v, t, sizeof t);
  }
}

/* csrc/reduction_utils.cuh:62-85 with maxBlockSize = 1024: per-warp butterfly,
 * lane 0 of each warp stores to shared[wid], then threads below
 * blockDim/32.0 reload shared[lane] (others 0) and run a second butterfly.
 * `val` has one entry per thread, nthreads <= 1024; lanes of a partial last
 * warp that do not exist contribute 0.  Returns thread 0's value. */
static float block_reduce_sum_thread0(const float* val, int nthreads) {
  float shared[32];
  int nwarps = (nthreads + 31) / 32;
  for (int w = 0; w < 32; ++w) shared[w] = 0.0f;
  for (int w = 0; w < nwarps; ++w) {
    float lanes[32];
    for (int l = 0; l < 32; ++l) {
      int t = w * 32 + l;
      lanes[l] = t < nthreads ? val[t] : 0.0f;
    }
    warp_butterfly_sum(lanes);
    shared[w] = lanes[0];
  }
  float lanes[32];
  float lim = (float)nthreads / 32.0f;
  for (int l = 0; l < 32; ++l) lanes[l] = ((float)l < lim) ? shared[l] : 0.0f;
  warp_butterfly_sum(lanes);
  return lanes[0];
}

/* ---------------------------------------------------------------- rms_norm */

/* One row of csrc/layernorm_kernels.cu:18-34.  `src` is the row the variance
 * is taken over, `dst` receives T(x * s) * w. */
static void rms_norm_row(void* dst, int64_t dst_off, const void* src, int64_t src_off,
                         const void* w, float eps, int H, int dt) {
  int nthreads = H < 1024 ? H : 1024;
  float part[1024];
  for (int t = 0; t < nthreads; ++t) {
    float acc = 0.0f;
    /* `variance += x * x` (:22-23); nvcc's default -fmad contracts it */
    for (int idx = t; idx < H; idx += nthreads) {
      float x = ld(src, src_off + idx, dt);
      acc = fmaf(x, x, acc);
    }
    part[t] = acc;
  }
  float variance = block_reduce_sum_thread0(part, nthreads);
  /* :27  rsqrtf(variance / hidden_size + epsilon) */
  float arg = variance / (float)H + eps;
  float s = (float)(1.0 / sqrt((double)arg));
  for (int idx = 0; idx < H; ++idx) {
    float x = ld(src, src_off + idx, dt);
    float n = rnd(x * s, dt);                 /* (scalar_t)(x * s_variance) */
    st(dst, dst_off + idx, dt, n * ld(w, idx, dt)); /* ... * weight[idx] in scalar_t */
  }
}

/* csrc/layernorm_kernels.cu:11-35, host :39-62.  Contiguous rows. */
void oracle_rms_norm(void* out, const void* in, const void* w, float eps,
                     int64_t T, int H, int dt) {
  for (int64_t r = 0; r < T; ++r) rms_norm_row(out, r * H, in, r * H, w, eps, H, dt);
}

/* Not a reference op: the exact fusion of the two steps the reference's
 * decoder layer performs, sarathi/model_executor/models/llama.py:248-252:
 * hidden = residual + hidden (one rounding to scalar_t), residual = hidden,
 * hidden = rms_norm(hidden).  Both tensors are updated in place. */
void oracle_fused_add_rms_norm(void* x, void* res, const void* w, float eps,
                               int64_t T, int H, int dt) {
  for (int64_t r = 0; r < T; ++r) {
    for (int i = 0; i < H; ++i) {
      float z = ld(x, r * H + i, dt) + ld(res, r * H + i, dt);
      st(res, r * H + i, dt, z);
    }
    rms_norm_row(x, r * H, res, r * H, w, eps, H, dt);
  }
}

/* -------------------------------------------------------------- activation */

/* csrc/activation_kernels.cu:9-12,19-24: silu in float, cast to scalar_t, then
 * a scalar_t multiply by y. */
void oracle_silu_and_mul(void* out, const void* in, int64_t T, int64_t d, int dt) {
  for (int64_t t = 0; t < T; ++t)
    for (int64_t i = 0; i < d; ++i) {
      float x = ld(in, t * 2 * d + i, dt);
      float y = ld(in, t * 2 * d + d + i, dt);
      float s = rnd(x / (1.0f + expf(-x)), dt);
      st(out, t * d + i, dt, s * y);
    }
}

/* csrc/activation_kernels.cu:86-91 */
void oracle_gelu_new(void* out, const void* in, int64_t T, int64_t d, int dt) {
  for (int64_t n = 0; n < T * d; ++n) {
    float x = ld(in, n, dt);
    float x3 = rnd(rnd(x * x, dt) * x, dt);            /* (float)(x * x * x) in T */
    float a = rnd(0.044715f * x3, dt);                 /* (T)(0.044715f * x3) */
    float b = rnd(x + a, dt);                          /* x + ... in T */
    float c = rnd(0.79788456f * b, dt);                /* (T)(0.79788456f * (float)...) */
    float t = rnd(tanhf(c), dt);
    float h = rnd(rnd(0.5f, dt) * x, dt);              /* ((T)0.5) * x */
    float g = rnd(rnd(1.0f, dt) + t, dt);              /* ((T)1.0) + t */
    st(out, n, dt, h * g);
  }
}

/* csrc/activation_kernels.cu:93-98 */
void oracle_gelu_fast(void* out, const void* in, int64_t T, int64_t d, int dt) {
  for (int64_t n = 0; n < T * d; ++n) {
    float x = ld(in, n, dt);
    float a = rnd(x * 0.79788456f, dt);                /* (T)(f * 0.79788456f) */
    float b = rnd(0.044715f * x, dt);                  /* (T)(0.044715f * f) */
    float c = rnd(b * x, dt);
    float e = rnd(rnd(1.0f, dt) + c, dt);
    float u = rnd(a * e, dt);
    float t = rnd(tanhf(u), dt);
    float h = rnd(rnd(0.5f, dt) * x, dt);
    float g = rnd(rnd(1.0f, dt) + t, dt);
    st(out, n, dt, h * g);
  }
}

/* ------------------------------------------------------------------ rotary */

/* csrc/pos_encoding_kernels.cu:8-36: every operator acts on scalar_t, so each
 * product and the final sum/difference round to the tensor dtype. */
static void rope_pair(void* arr, int64_t base, const void* cache, int64_t crow,
                      int rot_offset, int embed_dim, int is_neox, int dt) {
  int64_t xi, yi;
  if (is_neox) { xi = rot_offset; yi = embed_dim + rot_offset; }
  else { xi = 2 * rot_offset; yi = 2 * rot_offset + 1; }
  float c = ld(cache, crow + rot_offset, dt);
  float s = ld(cache, crow + embed_dim + rot_offset, dt);
  float x = ld(arr, base + xi, dt);
  float y = ld(arr, base + yi, dt);
  st(arr, base + xi, dt, rnd(x * c, dt) - rnd(y * s, dt));
  st(arr, base + yi, dt, rnd(y * c, dt) + rnd(x * s, dt));
}

/* csrc/pos_encoding_kernels.cu:38-76, host :80-127.  q and k are rows of
 * q_stride / k_stride elements (views into a packed qkv buffer are allowed);
 * the cache row of a token is cos[0:rot/2] || sin[0:rot/2]. */
void oracle_rotary_embedding(const int64_t* positions, void* q, void* k, const void* cache,
                             int64_t T, int nq, int nkv, int head_size, int rot_dim,
                             int64_t q_stride, int64_t k_stride, int is_neox, int dt) {
  int embed = rot_dim / 2;
  for (int64_t t = 0; t < T; ++t) {
    int64_t crow = positions[t] * rot_dim;
    for (int i = 0; i < nq * embed; ++i)
      rope_pair(q, t * q_stride + (int64_t)(i / embed) * head_size, cache, crow,
                i % embed, embed, is_neox, dt);
    for (int i = 0; i < nkv * embed; ++i)
      rope_pair(k, t * k_stride + (int64_t)(i / embed) * head_size, cache, crow,
                i % embed, embed, is_neox, dt);
  }
}

/* ------------------------------------------------------------ topk_softmax */

/* Fast path, csrc/moe_topk_softmax_kernels.cu:182-380, for E a power of two
 * up to 256.  A row is shared by TPR = E / VPT threads; thread g holds, for
 * each of its LDG loads l, the ELTS consecutive columns starting at
 * l * ELTS * TPR + g * ELTS (:236-248).  Sums: per thread in register order
 * (:270-275), then an xor butterfly over the TPR threads (:278-282). */
static void topk_row_pow2(const float* x, int E, int k, int64_t row, int64_t T,
                          float* w, int32_t* idx, int32_t* src) {
  int bytes = E * 4 < 16 ? E * 4 : 16;               /* BYTES_PER_LDG :391 */
  int elts = bytes / 4;                              /* ELTS_PER_LDG */
  int vecs = E / (elts * 32) > 1 ? E / (elts * 32) : 1; /* :385 */
  int vpt = vecs * elts;
  int tpr = E / vpt;
  int cols_per_ldg = elts * tpr;
  float chunk[32][8];                                /* [thread][register] */
  int col_of[32][8];
  for (int g = 0; g < tpr; ++g)
    for (int l = 0; l < vecs; ++l)
      for (int ii = 0; ii < elts; ++ii) {
        int c = l * cols_per_ldg + g * elts + ii;
        chunk[g][l * elts + ii] = x[c];
        col_of[g][l * elts + ii] = c;
      }
  /* max: per thread, then butterfly (:253-264); max is order independent */
  float m = chunk[0][0];
  for (int g = 0; g < tpr; ++g)
    for (int r = 0; r < vpt; ++r) m = chunk[g][r] > m ? chunk[g][r] : m;
  float part[32];
  for (int g = 0; g < tpr; ++g) {
    float s = 0.0f;
    for (int r = 0; r < vpt; ++r) {
      chunk[g][r] = expf(chunk[g][r] - m);
      s += chunk[g][r];
    }
    part[g] = s;
  }
  for (int mask = tpr / 2; mask > 0; mask /= 2) {
    float t[32];
    for (int g = 0; g < tpr; ++g) t[g] = part[g] + part[g ^ mask];
    memcpy(part, t, sizeof(float) * tpr);
  }
  float recip = 1.0f / part[0];                       /* :289 */
  for (int g = 0; g < tpr; ++g)
    for (int r = 0; r < vpt; ++r) chunk[g][r] = chunk[g][r] * recip;

  for (int j = 0; j < k; ++j) {
    /* per-thread argmax with strict > (:311-329), then the cross-thread rule
     * "larger value, or equal value and lower expert" (:334-346).  That rule
     * is a total order, so a plain scan applying it gives the butterfly's
     * consensus. */
    float best = 0.0f; int be = -1, bg = 0, br = 0;
    for (int g = 0; g < tpr; ++g) {
      float tv = chunk[g][0]; int te = col_of[g][0], tr = 0;
      for (int r = 1; r < vpt; ++r)
        if (chunk[g][r] > tv) { tv = chunk[g][r]; te = col_of[g][r]; tr = r; }
      if (be < 0 || tv > best || (tv == best && te < be)) { best = tv; be = te; bg = g; br = tr; }
    }
    w[j] = best;
    idx[j] = be;                                      /* start_expert = 0 (:415-419) */
    src[j] = (int32_t)(j * T + row);                  /* :362 */
    if (j + 1 < k) {
      /* :366-377 the owner of column `be` blanks it.  (bg, br) is that
       * owner unless the per-thread winner was a tie at a lower register. */
      int og = (be / elts) % tpr, orr = (be / cols_per_ldg) * elts + be % elts;
      (void)bg; (void)br;
      chunk[og][orr] = -10000.f;
    }
  }
}

/* cub::BlockReduce<float,256> default algorithm (BLOCK_REDUCE_WARP_REDUCTIONS):
 * inside each warp, steps offset = 1,2,4,8,16 with v[l] += v[l+offset] when
 * l+offset <= 31; then thread 0 adds the other warps' aggregates in order. */
static float cub_block_sum_256(const float* val) {
  float agg[8];
  for (int w = 0; w < 8; ++w) {
    float v[32];
    memcpy(v, val + 32 * w, sizeof v);
    for (int off = 1; off < 32; off <<= 1) {
      float t[32];
      for (int l = 0; l < 32; ++l) t[l] = (l + off <= 31) ? v[l] + v[l + off] : v[l];
      memcpy(v, t, sizeof v);
    }
    agg[w] = v[0];
  }
  float s = agg[0];
  for (int w = 1; w < 8; ++w) s = s + agg[w];
  return s;
}

/* Fallback, csrc/moe_topk_softmax_kernels.cu:50-166 with TPB = 256. */
static void topk_row_generic(const float* x, int E, int k, int64_t row, int64_t T,
                             float* w, int32_t* idx, int32_t* src, float* prob) {
  float m = -3.402823466e+38f;
  for (int c = 0; c < E; ++c) m = x[c] > m ? x[c] : m;
  float part[256];
  for (int t = 0; t < 256; ++t) {
    float s = 0.0f;
    for (int c = t; c < E; c += 256) s += expf(x[c] - m);
    part[t] = s;
  }
  float Z = cub_block_sum_256(part);
  float nf = 1.f / Z;
  for (int c = 0; c < E; ++c) prob[c] = expf(x[c] - m) * nf;
  for (int j = 0; j < k; ++j) {
    int bk = 0; float bv = -1.f;                      /* :129-130 */
    for (int c = 0; c < E; ++c) {
      int taken = 0;
      for (int p = 0; p < j; ++p) taken |= (idx[p] == c);
      if (taken) continue;
      /* cub::ArgMax: larger value, or equal value and smaller key */
      if (prob[c] > bv || (prob[c] == bv && c < bk)) { bv = prob[c]; bk = c; }
    }
    w[j] = bv; idx[j] = bk; src[j] = (int32_t)(j * T + row);
  }
}

/* csrc/moe_topk_softmax_kernels.cu:476-503 and the switch at :423-471. */
void oracle_topk_softmax(float* w, int32_t* idx, int32_t* src, const float* gating,
                         int64_t T, int E, int k) {
  int pow2 = E > 0 && (E & (E - 1)) == 0 && E <= 256;
  float* prob = (float*)malloc(sizeof(float) * (size_t)(E > 0 ? E : 1));
  for (int64_t r = 0; r < T; ++r) {
    if (pow2) topk_row_pow2(gating + r * E, E, k, r, T, w + r * k, idx + r * k, src + r * k);
    else topk_row_generic(gating + r * E, E, k, r, T, w + r * k, idx + r * k, src + r * k, prob);
  }
  free(prob);
}

/* ---------------------------------------------------- moe_align_block_size */

static inline int64_t ld_id(const void* p, int64_t i, int id_dt) {
  switch (id_dt) {
    case 0: return ((const uint8_t*)p)[i];
    case 1: return ((const int8_t*)p)[i];
    case 2: return ((const int16_t*)p)[i];
    case 3: return ((const int32_t*)p)[i];
    default: return ((const int64_t*)p)[i];
  }
}

/* csrc/moe_align_block_size_kernels.cu:23-109: E threads, thread t owns the
 * contiguous shard [t*tpt, (t+1)*tpt) of the flat ids.  id_dt: 0 u8, 1 i8,
 * 2 i16, 3 i32, 4 i64.  `sorted` keeps whatever the caller pre-filled in its
 * padding slots and `expert_ids` is written only for blocks below
 * post_pad / block_size, as in the reference. */
void oracle_moe_align_block_size(const void* ids, int id_dt, int64_t numel, int E, int B,
                                 int32_t* sorted, int32_t* expert_ids, int32_t* post_pad) {
  int64_t tpt = (numel + E - 1) / E;                  /* :30 */
  int32_t* cnts = (int32_t*)calloc((size_t)(E + 1) * (size_t)E, 4);
  int32_t* cumsum = (int32_t*)calloc((size_t)E + 1, 4);
  for (int t = 0; t < E; ++t)                         /* :50-52 */
    for (int64_t i = t * tpt; i < numel && i < (t + 1) * tpt; ++i)
      ++cnts[(int64_t)(t + 1) * E + ld_id(ids, i, id_dt)];
  for (int e = 0; e < E; ++e)                         /* :57-61 */
    for (int t = 1; t <= E; ++t) cnts[(int64_t)t * E + e] += cnts[(int64_t)(t - 1) * E + e];
  for (int e = 1; e <= E; ++e)                        /* :66-75 */
    cumsum[e] = cumsum[e - 1] + (cnts[(int64_t)E * E + e - 1] + B - 1) / B * B;
  *post_pad = cumsum[E];
  for (int e = 0; e < E; ++e)                         /* :83-86 */
    for (int i = cumsum[e]; i < cumsum[e + 1]; i += B) expert_ids[i / B] = e;
  for (int t = 0; t < E; ++t)                         /* :95-108 */
    for (int64_t i = t * tpt; i < numel && i < (t + 1) * tpt; ++i) {
      int64_t e = ld_id(ids, i, id_dt);
      int32_t rank = cnts[(int64_t)t * E + e] + cumsum[e];
      sorted[rank] = (int32_t)i;
      ++cnts[(int64_t)t * E + e];
    }
  free(cnts);
  free(cumsum);
}
