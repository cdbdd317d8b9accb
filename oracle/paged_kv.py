"""Paged KV-cache append, restated on the CPU with numpy.  TEST INFRASTRUCTURE ONLY: imported by
tests/, the smoke check and the benchmark's CPU baseline, never by the shipped package.

The algorithm lives in a third-party dependency that is not part of the reference tree:
flashinfer-python==0.4.1 (requirements.txt:18).  Its published behaviour, as used at the
reference's call sites (sarathi/model_executor/attention/flashinfer_attention_wrapper.py:213-226
for the two index helpers and :262-273 for the append, cache layout "NHD" from :70-78), is:

  get_seq_lens(kv_indptr, kv_last_page_len, page_size)
      = max(kv_indptr[1:] - kv_indptr[:-1] - 1, 0) * page_size + kv_last_page_len
  get_batch_indices_positions(append_indptr, seq_lens, nnz)
      for request b, token i in [append_indptr[b], append_indptr[b+1]):
          batch_indices[i] = b;  positions[i] = i + seq_lens[b] - append_indptr[b+1]
  append_paged_kv_cache(k, v, batch_indices, positions, cache, kv_indices, kv_indptr, ...)
      for token i:  page = kv_indices[kv_indptr[batch_indices[i]] + positions[i] // page_size]
                    cache[page, 0, positions[i] % page_size] = k[i]
                    cache[page, 1, positions[i] % page_size] = v[i]

Pinned (tests/test_oracle_pinning.py) by what the call sites require rather than by the absent
library: gathering a request's pages in page-table order returns exactly its tokens in order
(round trip), untouched entries keep their contents, the last appended token is the last entry
of its sequence, and a hand-worked example.  No fixture of flashinfer's own exists in the
reference, so agreement with the library itself is parity unpinned.
"""
import numpy as np


def get_seq_lens(kv_indptr, kv_last_page_len, page_size):
    kv_indptr = np.asarray(kv_indptr, dtype=np.int64)
    full = np.maximum(kv_indptr[1:] - kv_indptr[:-1] - 1, 0)
    return (full * page_size + np.asarray(kv_last_page_len, dtype=np.int64)).astype(np.int32)


def get_batch_indices_positions(append_indptr, seq_lens, nnz, fill=-1):
    """Entries of tokens no request covers keep ``fill`` (the library leaves them undefined)."""
    batch_indices = np.full((nnz,), fill, dtype=np.int32)
    positions = np.full((nnz,), fill, dtype=np.int32)
    for b in range(len(seq_lens)):
        lo, hi = int(append_indptr[b]), int(append_indptr[b + 1])
        for i in range(lo, min(hi, nnz)):
            batch_indices[i] = b
            positions[i] = i + int(seq_lens[b]) - hi
    return batch_indices, positions


def append_paged_kv_cache(append_key, append_value, batch_indices, positions, k_cache, v_cache,
                          kv_indices, kv_indptr):
    """k_cache / v_cache: numpy views [num_pages, page_size, heads, head_size], written in place.
    append_key / append_value: [nnz, heads, head_size] arrays of the same item size."""
    page_size = k_cache.shape[1]
    for i in range(len(batch_indices)):
        b, pos = int(batch_indices[i]), int(positions[i])
        page = int(kv_indices[int(kv_indptr[b]) + pos // page_size])
        k_cache[page, pos % page_size] = append_key[i]
        v_cache[page, pos % page_size] = append_value[i]


def gather_sequence(cache_plane, kv_indices, kv_indptr, seq_lens, b):
    """The first seq_lens[b] entries of request b, in order (what attention reads)."""
    page_size = cache_plane.shape[1]
    pages = [int(p) for p in kv_indices[int(kv_indptr[b]):int(kv_indptr[b + 1])]]
    rows = [cache_plane[pages[j // page_size], j % page_size] for j in range(int(seq_lens[b]))]
    return np.stack(rows) if rows else np.zeros((0,) + cache_plane.shape[2:], cache_plane.dtype)
