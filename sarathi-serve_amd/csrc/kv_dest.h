// Where an appended token lands in a paged KV cache (NHD page layout).
//
// Follows the published algorithm of flashinfer's append_paged_kv_cache (the reference pins
// flashinfer-python==0.4.1 in requirements.txt and calls it at
// sarathi/model_executor/attention/flashinfer_attention_wrapper.py:262-273): token i belongs to
// request b = batch_indices[i] and is the positions[i]-th entry of that request's key/value
// sequence; the request's pages are kv_indices[kv_indptr[b] .. kv_indptr[b+1]), page_size entries
// each, so the token goes to entry positions[i] % page_size of page
// kv_indices[kv_indptr[b] + positions[i] / page_size].
#pragma once

#include <stdint.h>

#include "vec16.h"

namespace sarathi_hip {

// Cache policy of the stores into cache entries (overridable for tuning runs).
#ifndef SARATHI_KV_STORE_POLICY
#define SARATHI_KV_STORE_POLICY 0
#endif
constexpr int kKvStore = SARATHI_KV_STORE_POLICY;
// The same for the rotary embedding fused with the append, in the waves that take several
// segments of a token: there the cache stores leave the wave together with eight in-place query
// stores per lane, and a non-temporal hint (2) keeps them from displacing the rows other waves are
// still reading (2304 tokens: 10.5 -> 9.7 us; the stand-alone append and the fused kernel's
// one-segment waves are fastest with the default policy).
#ifndef SARATHI_KV_STORE_POLICY_FUSED
#define SARATHI_KV_STORE_POLICY_FUSED 2
#endif
constexpr int kKvStoreFused = SARATHI_KV_STORE_POLICY_FUSED;

struct KvDest {
  const int32_t* batch_indices;  // [nnz]
  const int32_t* positions;      // [nnz] index of the token inside its request's kv sequence
  const int32_t* kv_indices;     // page numbers, ragged over requests
  const int32_t* kv_indptr;      // [requests + 1]
  const int32_t* slot_mapping;   // optional [nnz]: page * page_size + entry, precomputed once per
                                 // batch; replaces the three dependent lookups above
  void* k_cache;                 // entry (page, e) of K starts at page*page_stride + e*entry_stride
  void* v_cache;                 // same geometry for V
  int64_t page_stride_bytes;
  int64_t entry_stride_bytes;
  int64_t nnz;                   // tokens to append (tokens at or above it are not appended)
  int32_t page_size;
};

// Byte offset of token `tok`'s entry from k_cache / v_cache, in two steps so that a kernel can
// put other work between them: kv_entry_key() issues the scalar loads that depend on nothing but
// the token index, kv_entry_resolve() the dependent page-table lookups.  `tok` is uniform over
// the wave, so all of these are scalar loads.
struct KvEntryKey {
  int32_t a;  // slot (with a slot mapping) or request index
  int32_t b;  // position of the token inside its request's kv sequence (unused with a mapping)
};
SK_DEV KvEntryKey kv_entry_key(const KvDest& d, int64_t tok) {
  KvEntryKey k;
  if (d.slot_mapping != nullptr) {
    k.a = d.slot_mapping[tok];
    k.b = 0;
  } else {
    k.a = d.batch_indices[tok];
    k.b = d.positions[tok];
  }
  return k;
}
// SLOTS: whether k.a is a slot (known at compile time where a kernel is specialised on it).
template <bool SLOTS>
SK_DEV int64_t kv_entry_resolve(const KvDest& d, KvEntryKey k) {
  if (SLOTS) {
    const uint32_t slot = (uint32_t)k.a;
    const uint32_t page = slot / (uint32_t)d.page_size;
    const uint32_t entry = slot - page * (uint32_t)d.page_size;
    return (int64_t)page * d.page_stride_bytes + (int64_t)entry * d.entry_stride_bytes;
  }
  const uint32_t pos = (uint32_t)k.b;
  const uint32_t pg = pos / (uint32_t)d.page_size;
  const uint32_t entry = pos - pg * (uint32_t)d.page_size;
  const int64_t page = d.kv_indices[(int64_t)d.kv_indptr[k.a] + pg];
  return page * d.page_stride_bytes + (int64_t)entry * d.entry_stride_bytes;
}
SK_DEV int64_t kv_entry_resolve(const KvDest& d, KvEntryKey k) {
  return d.slot_mapping != nullptr ? kv_entry_resolve<true>(d, k) : kv_entry_resolve<false>(d, k);
}
SK_DEV int64_t kv_entry_offset(const KvDest& d, int64_t tok) {
  return kv_entry_resolve(d, kv_entry_key(d, tok));
}

}  // namespace sarathi_hip
