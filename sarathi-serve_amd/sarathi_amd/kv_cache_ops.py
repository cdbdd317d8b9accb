"""Paged KV-cache append ops with the signatures of the flashinfer functions the reference's
attention wrapper calls (sarathi/model_executor/attention/flashinfer_attention_wrapper.py:213-226
and :262-273; flashinfer-python==0.4.1), plus the rotary-embedding + append fusion.

The cache is flashinfer's NHD layout: one tensor ``[num_pages, 2, page_size, num_kv_heads,
head_size]`` (K plane, V plane) or a ``(k_cache, v_cache)`` pair of
``[num_pages, page_size, num_kv_heads, head_size]`` tensors.
"""
from typing import Optional, Tuple, Union

import torch

from ._ext import C as _C

PagedCache = Union[torch.Tensor, Tuple[torch.Tensor, torch.Tensor]]


def _split_cache(paged_kv_cache: PagedCache, kv_layout: str):
    if kv_layout != "NHD":
        raise ValueError("only the NHD page layout is supported, got %r" % (kv_layout,))
    if isinstance(paged_kv_cache, (tuple, list)):
        k_cache, v_cache = paged_kv_cache
        return k_cache, v_cache
    if paged_kv_cache.dim() != 5 or paged_kv_cache.shape[1] != 2:
        raise ValueError("paged_kv_cache must be [num_pages, 2, page_size, num_kv_heads, head_size]")
    return paged_kv_cache[:, 0], paged_kv_cache[:, 1]


def get_seq_lens(kv_indptr: torch.Tensor, kv_last_page_len: torch.Tensor,
                 page_size: int) -> torch.Tensor:
    """Length of every request's kv sequence: full pages * page_size + entries of the last page."""
    seq_lens = torch.empty_like(kv_last_page_len)
    _C.get_seq_lens(kv_indptr, kv_last_page_len, seq_lens, page_size)
    return seq_lens


def get_batch_indices_positions(append_indptr: torch.Tensor, seq_lens: torch.Tensor,
                                nnz: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """For each of the ``nnz`` appended tokens: the request it belongs to and its index in that
    request's kv sequence (the request's last appended token is the sequence's last entry)."""
    batch_indices = torch.empty((nnz,), dtype=torch.int32, device=append_indptr.device)
    positions = torch.empty((nnz,), dtype=torch.int32, device=append_indptr.device)
    _C.get_batch_indices_positions(append_indptr, seq_lens, batch_indices, positions)
    return batch_indices, positions


def get_kv_slot_mapping(batch_indices: torch.Tensor, positions: torch.Tensor,
                        kv_indices: torch.Tensor, kv_indptr: torch.Tensor,
                        page_size: int) -> torch.Tensor:
    """``page * page_size + entry`` of every appended token.  The page table of a batch is the
    same for all layers: compute this once per batch and pass it as ``slot_mapping`` to the append
    ops, which then resolve a token's destination with one index load instead of three."""
    slot_mapping = torch.empty_like(batch_indices)
    _C.get_kv_slot_mapping(batch_indices, positions, kv_indices, kv_indptr, slot_mapping, page_size)
    return slot_mapping


def append_paged_kv_cache(append_key: torch.Tensor, append_value: torch.Tensor,
                          batch_indices: torch.Tensor, positions: torch.Tensor,
                          paged_kv_cache: PagedCache, kv_indices: torch.Tensor,
                          kv_indptr: torch.Tensor, kv_last_page_len: Optional[torch.Tensor] = None,
                          kv_layout: str = "NHD",
                          slot_mapping: Optional[torch.Tensor] = None) -> None:
    """Copy ``append_key`` / ``append_value`` ``[nnz, num_kv_heads, head_size]`` into the cache.
    ``kv_last_page_len`` is accepted for signature compatibility; the destination of a token
    follows from ``positions`` alone."""
    k_cache, v_cache = _split_cache(paged_kv_cache, kv_layout)
    _C.append_paged_kv_cache(append_key, append_value, batch_indices, positions, k_cache, v_cache,
                             kv_indices, kv_indptr, slot_mapping)


def rotary_embedding_append_paged_kv(positions: torch.Tensor, query: torch.Tensor,
                                     key: torch.Tensor, value: torch.Tensor, head_size: int,
                                     cos_sin_cache: torch.Tensor, is_neox: bool,
                                     batch_indices: torch.Tensor, append_positions: torch.Tensor,
                                     paged_kv_cache: PagedCache, kv_indices: torch.Tensor,
                                     kv_indptr: torch.Tensor,
                                     num_append_tokens: Optional[int] = None,
                                     write_key: bool = False, kv_layout: str = "NHD",
                                     slot_mapping: Optional[torch.Tensor] = None) -> None:
    """``pos_encoding_ops.rotary_embedding(positions, query, key, ...)`` followed by
    ``append_paged_kv_cache(key[:n], value[:n], ...)`` in one launch (n = ``num_append_tokens``,
    default all tokens).  ``query`` is rotated in place; the rotated keys go to the cache and, only
    with ``write_key=True``, also back into ``key``."""
    k_cache, v_cache = _split_cache(paged_kv_cache, kv_layout)
    n = positions.shape[0] if num_append_tokens is None else int(num_append_tokens)
    _C.rotary_embedding_append_paged_kv(positions, query, key, value, head_size, cos_sin_cache,
                                        is_neox, batch_indices, append_positions, k_cache, v_cache,
                                        kv_indices, kv_indptr, n, write_key, slot_mapping)


__all__ = ["get_seq_lens", "get_batch_indices_positions", "get_kv_slot_mapping", "append_paged_kv_cache",
           "rotary_embedding_append_paged_kv"]
