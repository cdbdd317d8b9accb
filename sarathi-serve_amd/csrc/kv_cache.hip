// Paged KV-cache append and its index helpers for gfx950.
//
// Stand in for the three flashinfer calls on the reference's attention path
// (sarathi/model_executor/attention/flashinfer_attention_wrapper.py:213-226 and :262-273;
// flashinfer-python==0.4.1 per requirements.txt): get_seq_lens, get_batch_indices_positions and
// append_paged_kv_cache with kv_layout="NHD".  The rotary-embedding + append fusion lives next to
// the rotary kernel (rope.hip); this file holds the plain copy.
//
// append: a workgroup is one wave that moves the key row and the value row of one to four
// consecutive tokens (rows of up to 4 KiB, every lane 16 bytes of up to four 1 KiB pieces).  The
// index loads of all its tokens go out first, then all the row loads, and only then are the cache
// entries resolved and written: the dependent page-table lookups run under the row loads instead
// of in front of them.  Source rows are read with the streaming policy (they are not needed
// again), cache entries are written with the default policy (attention reads them next).  Rows
// longer than 4 KiB go through the older kernel of one wave per 1 KiB piece.
#include "kv_dest.h"
#include "launch.h"

namespace sarathi_hip {

// PPL pieces of 1 KiB per row (one 16-byte load per lane each), TPW tokens per wave; SLOTS says
// whether a slot mapping is given (a kernel of its own each way keeps the order below free of
// branches).  What the row loads need comes first in the argument list, where the kernel
// arguments are preloaded into registers; the cache geometry is fetched under the row loads.
// Tokens past the end of the batch get empty buffer resources: their loads return nothing and
// their stores are dropped.
template <int PPL, int TPW, bool SLOTS>
__global__ __launch_bounds__(64) void kv_append_tok_kernel(
    const void* __restrict__ key, const void* __restrict__ value, int64_t k_stride_bytes,
    int64_t v_stride_bytes, uint32_t row_bytes, uint32_t nnz, const int32_t* __restrict__ index_a,
    const int32_t* __restrict__ index_b, KvDest d) {
  const uint32_t tok0 = blockIdx.x * TPW;
  const uint32_t off = threadIdx.x * 16u;
  KvEntryKey keys[TPW];
  u32x4 kk[TPW][PPL], vv[TPW][PPL];
  uint32_t recs[TPW];
#pragma unroll
  for (int t = 0; t < TPW; ++t) {
    const bool live = tok0 + t < nnz;
    const uint32_t tok = live ? tok0 + t : nnz - 1;
    recs[t] = live ? row_bytes : 0u;
    keys[t].a = index_a[tok];  // slot, or request
    keys[t].b = SLOTS ? 0 : index_b[tok];
  }
#pragma unroll
  for (int t = 0; t < TPW; ++t) {
    const rsrc_t rk = make_rsrc(
        reinterpret_cast<const char*>(key) + (int64_t)(tok0 + t) * k_stride_bytes, recs[t]);
    const rsrc_t rv = make_rsrc(
        reinterpret_cast<const char*>(value) + (int64_t)(tok0 + t) * v_stride_bytes, recs[t]);
#pragma unroll
    for (int p = 0; p < PPL; ++p) kk[t][p] = buf_load16<kStreamLoad>(rk, off + p * 1024u);
#pragma unroll
    for (int p = 0; p < PPL; ++p) vv[t][p] = buf_load16<kStreamLoad>(rv, off + p * 1024u);
  }
  __builtin_amdgcn_sched_barrier(0);  // every load is issued before anything waits
#pragma unroll
  for (int t = 0; t < TPW; ++t) {
    const int64_t e = kv_entry_resolve<SLOTS>(d, keys[t]);
    const rsrc_t dk = make_rsrc(reinterpret_cast<char*>(d.k_cache) + e, recs[t]);
    const rsrc_t dv = make_rsrc(reinterpret_cast<char*>(d.v_cache) + e, recs[t]);
#pragma unroll
    for (int p = 0; p < PPL; ++p) buf_store16<kKvStore>(dk, off + p * 1024u, kk[t][p]);
#pragma unroll
    for (int p = 0; p < PPL; ++p) buf_store16<kKvStore>(dv, off + p * 1024u, vv[t][p]);
  }
}

template <int PPL>
static void launch_kv_tok(hipStream_t st, const void* key, const void* value, int64_t ksb,
                          int64_t vsb, uint32_t row_bytes, const KvDest& d) {
  const int tpw = pick_rows_per_workgroup(d.nnz, 4 / PPL);
  const unsigned grid = (unsigned)((d.nnz + tpw - 1) / tpw);
  const uint32_t nnz = (uint32_t)d.nnz;
#define SARATHI_KV_TOK(T)                                                                        \
  do {                                                                                           \
    if (d.slot_mapping)                                                                          \
      hipLaunchKernelGGL((kv_append_tok_kernel<PPL, T, true>), dim3(grid), dim3(64), 0, st, key, \
                         value, ksb, vsb, row_bytes, nnz, d.slot_mapping, nullptr, d);           \
    else                                                                                         \
      hipLaunchKernelGGL((kv_append_tok_kernel<PPL, T, false>), dim3(grid), dim3(64), 0, st,     \
                         key, value, ksb, vsb, row_bytes, nnz, d.batch_indices, d.positions, d); \
  } while (0)
  if constexpr (PPL == 1) {
    if (tpw == 4) { SARATHI_KV_TOK(4); return; }
    if (tpw == 3) { SARATHI_KV_TOK(3); return; }
  }
  if constexpr (PPL <= 2) {
    if (tpw == 2) { SARATHI_KV_TOK(2); return; }
  }
  SARATHI_KV_TOK(1);
#undef SARATHI_KV_TOK
}

// Rows of any length: a workgroup is one wave that moves 64 consecutive 16-byte pieces of one
// token's key row or value row.  Workgroup ids run over the key pieces, then the value pieces,
// then the tokens.
__global__ __launch_bounds__(64) void kv_append_seg_kernel(
    const void* __restrict__ key, const void* __restrict__ value, int64_t k_stride_bytes,
    int64_t v_stride_bytes, uint32_t row_bytes, uint32_t blocks_per_row, KvDest d) {
  const int64_t tok = (int64_t)blockIdx.z * kMaxGridY + blockIdx.y;
  const bool is_k = blockIdx.x < blocks_per_row;  // uniform over the wave
  const uint32_t seg = blockIdx.x - (is_k ? 0u : blocks_per_row);
  const uint32_t off = (seg * 64u + threadIdx.x) * 16u;
  const char* src = reinterpret_cast<const char*>(is_k ? key : value) +
                    tok * (is_k ? k_stride_bytes : v_stride_bytes);
  const u32x4 v = buf_load16<kStreamLoad>(make_rsrc(src, row_bytes), off);
  char* dst = reinterpret_cast<char*>(is_k ? d.k_cache : d.v_cache) + kv_entry_offset(d, tok);
  buf_store16<kKvStore>(make_rsrc(dst, row_bytes), off, v);  // pieces past the row are dropped
}

// Any alignment: one workgroup per token, 2-byte units (every supported dtype is a multiple).
__global__ __launch_bounds__(256) void kv_append_generic_kernel(
    const void* __restrict__ key, const void* __restrict__ value, int64_t k_stride_bytes,
    int64_t v_stride_bytes, uint32_t row_bytes, KvDest d) {
  const int64_t tok = blockIdx.x;
  const int64_t e = kv_entry_offset(d, tok);
  const uint16_t* ks =
      reinterpret_cast<const uint16_t*>(reinterpret_cast<const char*>(key) + tok * k_stride_bytes);
  const uint16_t* vs = reinterpret_cast<const uint16_t*>(reinterpret_cast<const char*>(value) +
                                                         tok * v_stride_bytes);
  uint16_t* kd = reinterpret_cast<uint16_t*>(reinterpret_cast<char*>(d.k_cache) + e);
  uint16_t* vd = reinterpret_cast<uint16_t*>(reinterpret_cast<char*>(d.v_cache) + e);
  for (uint32_t i = threadIdx.x; i < row_bytes / 2; i += 256) {
    kd[i] = ks[i];
    vd[i] = vs[i];
  }
}

__global__ __launch_bounds__(256) void kv_seq_lens_kernel(const int32_t* __restrict__ kv_indptr,
                                                          const int32_t* __restrict__ last_page_len,
                                                          int32_t* __restrict__ seq_lens,
                                                          int64_t num_seqs, int32_t page_size) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= num_seqs) return;
  const int32_t full = kv_indptr[i + 1] - kv_indptr[i] - 1;
  seq_lens[i] = (full > 0 ? full : 0) * page_size + last_page_len[i];
}

// One thread per appended token: binary search for the request whose range of append_indptr
// holds the token (empty requests, i.e. repeated indptr values, are stepped over).
__global__ __launch_bounds__(256) void kv_batch_positions_kernel(
    const int32_t* __restrict__ append_indptr, const int32_t* __restrict__ seq_lens,
    int32_t* __restrict__ batch_indices, int32_t* __restrict__ positions, int64_t num_seqs,
    int64_t nnz) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= nnz || i < append_indptr[0] || i >= append_indptr[num_seqs]) return;
  int64_t lo = 0, hi = num_seqs;  // invariant: indptr[lo] <= i < indptr[hi]
  while (hi - lo > 1) {
    const int64_t mid = (lo + hi) >> 1;
    if (append_indptr[mid] <= i) lo = mid; else hi = mid;
  }
  batch_indices[i] = (int32_t)lo;
  positions[i] = (int32_t)(i + seq_lens[lo] - append_indptr[lo + 1]);
}

// slot_mapping[i] = page * page_size + entry of appended token i
__global__ __launch_bounds__(256) void kv_slot_mapping_kernel(
    const int32_t* __restrict__ batch_indices, const int32_t* __restrict__ positions,
    const int32_t* __restrict__ kv_indices, const int32_t* __restrict__ kv_indptr,
    int32_t* __restrict__ slot_mapping, int64_t nnz, int32_t page_size) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= nnz) return;
  const uint32_t pos = (uint32_t)positions[i];
  const uint32_t pg = pos / (uint32_t)page_size;
  const int32_t page = kv_indices[(int64_t)kv_indptr[batch_indices[i]] + pg];
  slot_mapping[i] = page * page_size + (int32_t)(pos - pg * (uint32_t)page_size);
}

}  // namespace sarathi_hip

using namespace sarathi_hip;

static int elem_bytes_of(int dtype) {
  return dtype == kF32 ? 4 : (dtype == kF16 || dtype == kBF16) ? 2 : 0;
}

extern "C" int sarathi_append_paged_kv_cache(
    const void* append_key, const void* append_value, const int32_t* batch_indices,
    const int32_t* positions, void* k_cache, void* v_cache, const int32_t* kv_indices,
    const int32_t* kv_indptr, const int32_t* slot_mapping, int64_t nnz, int num_kv_heads,
    int head_size, int page_size, int64_t key_stride, int64_t value_stride, int64_t page_stride,
    int64_t entry_stride, int dtype, void* stream) {
  if (nnz > 0 && (!append_key || !append_value || !k_cache || !v_cache ||
                  (!slot_mapping && (!batch_indices || !positions || !kv_indices || !kv_indptr))))
    return SARATHI_ERR_INVALID_ARG;  // empty tensors have no data
  const int64_t row = (int64_t)num_kv_heads * head_size;
  if (nnz < 0 || num_kv_heads <= 0 || head_size <= 0 || page_size <= 0 || key_stride < row ||
      value_stride < row || entry_stride < row || page_stride < (int64_t)page_size * entry_stride)
    return SARATHI_ERR_INVALID_ARG;
  const int eb = elem_bytes_of(dtype);
  if (eb == 0 || row * eb >= 0x80000000LL || nnz > 0x7fffffffLL) return SARATHI_ERR_UNSUPPORTED;
  if (nnz == 0) return SARATHI_OK;
  hipStream_t st = (hipStream_t)stream;
  KvDest d{batch_indices, positions, kv_indices,       kv_indptr,         slot_mapping,
           k_cache,       v_cache,   page_stride * eb, entry_stride * eb, nnz,
           (int32_t)page_size};
  const uint32_t row_bytes = (uint32_t)(row * eb);
  const int64_t ksb = key_stride * eb, vsb = value_stride * eb;
  const bool vec_ok = row_bytes % 16 == 0 && ksb % 16 == 0 && vsb % 16 == 0 &&
                      d.page_stride_bytes % 16 == 0 && d.entry_stride_bytes % 16 == 0 &&
                      aligned16(append_key) && aligned16(append_value) && aligned16(k_cache) &&
                      aligned16(v_cache);
  if (!vec_ok) {
    hipLaunchKernelGGL(kv_append_generic_kernel, dim3((unsigned)nnz), dim3(256), 0, st, append_key,
                       append_value, ksb, vsb, row_bytes, d);
    return launch_status();
  }
  if (row_bytes <= 4096) {
    if (row_bytes <= 1024) launch_kv_tok<1>(st, append_key, append_value, ksb, vsb, row_bytes, d);
    else if (row_bytes <= 2048) launch_kv_tok<2>(st, append_key, append_value, ksb, vsb, row_bytes, d);
    else launch_kv_tok<4>(st, append_key, append_value, ksb, vsb, row_bytes, d);
    return launch_status();
  }
  const uint32_t bpr = (row_bytes / 16 + 63) / 64;
  const int64_t full_z = nnz / kMaxGridY, rem = nnz % kMaxGridY;
  if (full_z > 0)
    hipLaunchKernelGGL(kv_append_seg_kernel, dim3(2 * bpr, kMaxGridY, (unsigned)full_z), dim3(64),
                       0, st, append_key, append_value, ksb, vsb, row_bytes, bpr, d);
  if (rem > 0) {
    const int64_t t0 = full_z * kMaxGridY;
    KvDest dr = d;
    if (dr.slot_mapping) {
      dr.slot_mapping += t0;
    } else {
      dr.batch_indices += t0;
      dr.positions += t0;
    }
    hipLaunchKernelGGL(kv_append_seg_kernel, dim3(2 * bpr, (unsigned)rem, 1), dim3(64), 0, st,
                       reinterpret_cast<const char*>(append_key) + t0 * ksb,
                       reinterpret_cast<const char*>(append_value) + t0 * vsb, ksb, vsb, row_bytes,
                       bpr, dr);
  }
  return launch_status();
}

extern "C" int sarathi_get_seq_lens(const int32_t* kv_indptr, const int32_t* kv_last_page_len,
                                    int32_t* seq_lens, int64_t num_seqs, int page_size,
                                    void* stream) {
  if (num_seqs < 0 || page_size <= 0) return SARATHI_ERR_INVALID_ARG;
  if (num_seqs == 0) return SARATHI_OK;  // empty tensors have no data: pointers may be null
  if (!kv_indptr || !kv_last_page_len || !seq_lens) return SARATHI_ERR_INVALID_ARG;
  if (num_seqs > 0x7fffffffLL) return SARATHI_ERR_UNSUPPORTED;
  hipLaunchKernelGGL(kv_seq_lens_kernel, dim3((unsigned)((num_seqs + 255) / 256)), dim3(256), 0,
                     (hipStream_t)stream, kv_indptr, kv_last_page_len, seq_lens, num_seqs,
                     (int32_t)page_size);
  return launch_status();
}

extern "C" int sarathi_get_batch_indices_positions(const int32_t* append_indptr,
                                                   const int32_t* seq_lens, int32_t* batch_indices,
                                                   int32_t* positions, int64_t num_seqs,
                                                   int64_t nnz, void* stream) {
  if (num_seqs < 0 || nnz < 0) return SARATHI_ERR_INVALID_ARG;
  if (num_seqs == 0 || nnz == 0) return SARATHI_OK;
  if (!append_indptr || !seq_lens || !batch_indices || !positions) return SARATHI_ERR_INVALID_ARG;
  if (nnz > 0x7fffffffLL) return SARATHI_ERR_UNSUPPORTED;
  hipLaunchKernelGGL(kv_batch_positions_kernel, dim3((unsigned)((nnz + 255) / 256)), dim3(256), 0,
                     (hipStream_t)stream, append_indptr, seq_lens, batch_indices, positions,
                     num_seqs, nnz);
  return launch_status();
}

extern "C" int sarathi_get_kv_slot_mapping(const int32_t* batch_indices, const int32_t* positions,
                                           const int32_t* kv_indices, const int32_t* kv_indptr,
                                           int32_t* slot_mapping, int64_t nnz, int page_size,
                                           void* stream) {
  if (nnz < 0 || page_size <= 0) return SARATHI_ERR_INVALID_ARG;
  if (nnz == 0) return SARATHI_OK;
  if (!batch_indices || !positions || !kv_indices || !kv_indptr || !slot_mapping)
    return SARATHI_ERR_INVALID_ARG;
  if (nnz > 0x7fffffffLL) return SARATHI_ERR_UNSUPPORTED;
  hipLaunchKernelGGL(kv_slot_mapping_kernel, dim3((unsigned)((nnz + 255) / 256)), dim3(256), 0,
                     (hipStream_t)stream, batch_indices, positions, kv_indices, kv_indptr,
                     slot_mapping, nnz, (int32_t)page_size);
  return launch_status();
}
