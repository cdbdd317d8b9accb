"""Host-side index bookkeeping for the paged KV-cache append of a hybrid batch (reference:
FlashinferAttentionWrapper.begin_forward,
sarathi/model_executor/attention/flashinfer_attention_wrapper.py:84-229).

A batch is prefill chunks first, then one decode token per running request.  For every request
the page table prefix in use, the fill of its last page and the start of its tokens in the
flattened batch are collected into the four int32 vectors the append needs; the two derived
vectors (request index and kv position of every token) come from the device helpers, and so does
the slot of every token (page * block_size + entry), which is the same for all layers of the
model: it is computed once here and every append of the batch (``AppendMetadata.append``,
``AppendMetadata.rotary_embedding_append``) passes it on, so that the per-layer kernels do one
index load per token instead of three dependent ones.
"""
from dataclasses import dataclass
from typing import List, Sequence

import torch

from .. import kv_cache_ops


@dataclass
class SequenceSlice:
    """What begin_forward reads from a SequenceMetadata: ``num_new_tokens`` tokens of this request
    are in the batch (a prompt chunk, or 1 for a decode step), after which the request holds
    ``total_len`` tokens in the cache; ``block_table`` lists its pages."""
    is_prompt: bool
    num_new_tokens: int
    total_len: int
    block_table: Sequence[int]


@dataclass
class AppendMetadata:
    append_qo_indptr: torch.Tensor          # [requests + 1] start of each request's tokens
    append_kv_page_indices: torch.Tensor    # pages of all requests, concatenated
    append_kv_page_indptr: torch.Tensor     # [requests + 1]
    append_kv_last_page_len: torch.Tensor   # [requests]
    append_batch_indices: torch.Tensor      # [num_total_tokens]
    append_positions: torch.Tensor          # [num_total_tokens]
    slot_mapping: torch.Tensor              # [num_total_tokens] page * block_size + entry
    num_prefill_tokens: int
    num_total_tokens: int

    def append(self, key: torch.Tensor, value: torch.Tensor, kv_cache, kv_layout: str = "NHD") -> None:
        """The append of FlashinferAttentionWrapper.forward
        (sarathi/model_executor/attention/flashinfer_attention_wrapper.py:262-273) for this batch:
        ``key`` / ``value`` ``[num_total_tokens, num_kv_heads, head_size]`` go into ``kv_cache``."""
        kv_cache_ops.append_paged_kv_cache(
            key, value, self.append_batch_indices, self.append_positions, kv_cache,
            self.append_kv_page_indices, self.append_kv_page_indptr, self.append_kv_last_page_len,
            kv_layout=kv_layout, slot_mapping=self.slot_mapping)

    def rotary_embedding_append(self, positions: torch.Tensor, query: torch.Tensor,
                                key: torch.Tensor, value: torch.Tensor, head_size: int,
                                cos_sin_cache: torch.Tensor, is_neox: bool, kv_cache,
                                write_key: bool = False, kv_layout: str = "NHD") -> None:
        """Rotary embedding of ``query`` / ``key`` and the append above in one launch."""
        kv_cache_ops.rotary_embedding_append_paged_kv(
            positions, query, key, value, head_size, cos_sin_cache, is_neox,
            self.append_batch_indices, self.append_positions, kv_cache,
            self.append_kv_page_indices, self.append_kv_page_indptr, self.num_total_tokens,
            write_key, kv_layout, slot_mapping=self.slot_mapping)


def build_append_metadata(seqs: Sequence[SequenceSlice], block_size: int,
                          device: torch.device) -> AppendMetadata:
    qo_indptr: List[int] = [0]
    page_indices: List[int] = []
    page_indptr: List[int] = [0]
    last_page_len: List[int] = []
    num_prefill_tokens = 0
    # prompts first, then decodes, each group in batch order (flashinfer_attention_wrapper.py:113-168)
    for want_prompt in (True, False):
        for s in seqs:
            if s.is_prompt != want_prompt:
                continue
            new = s.num_new_tokens if s.is_prompt else 1
            blocks = (s.total_len + block_size - 1) // block_size
            if len(s.block_table) < blocks:
                raise ValueError("block_table holds %d pages, %d tokens need %d"
                                 % (len(s.block_table), s.total_len, blocks))
            qo_indptr.append(qo_indptr[-1] + new)
            page_indices.extend(s.block_table[:blocks])
            page_indptr.append(page_indptr[-1] + blocks)
            last_page_len.append(s.total_len % block_size or block_size)
            if s.is_prompt:
                num_prefill_tokens += new

    def to_int_tensor(data: List[int]) -> torch.Tensor:
        return torch.tensor(data, dtype=torch.int32, device=device)

    num_total_tokens = qo_indptr[-1]
    m_qo, m_idx = to_int_tensor(qo_indptr), to_int_tensor(page_indices)
    m_indptr, m_last = to_int_tensor(page_indptr), to_int_tensor(last_page_len)
    seq_lens = kv_cache_ops.get_seq_lens(m_indptr, m_last, block_size)
    batch_indices, positions = kv_cache_ops.get_batch_indices_positions(m_qo, seq_lens,
                                                                        num_total_tokens)
    slot_mapping = kv_cache_ops.get_kv_slot_mapping(batch_indices, positions, m_idx, m_indptr,
                                                    block_size)
    return AppendMetadata(m_qo, m_idx, m_indptr, m_last, batch_indices, positions, slot_mapping,
                          num_prefill_tokens, num_total_tokens)
