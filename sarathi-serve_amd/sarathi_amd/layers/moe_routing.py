"""MoE routing helpers (reference: layers/fused_moe/fused_moe.py:151-204 and :346-373)."""
from typing import Tuple

import torch

from .. import moe_ops


def fused_topk(hidden_states: torch.Tensor, gating_output: torch.Tensor, topk: int,
               renormalize: bool) -> Tuple[torch.Tensor, torch.Tensor]:
    """Softmax over the experts and top-k per token.  Returns (topk_weights f32 [M, topk],
    topk_ids i32 [M, topk]).  With ``renormalize`` the weights of a token are divided by their sum,
    inside the same kernel (the reference does it with a separate tensor divide)."""
    assert hidden_states.shape[0] == gating_output.shape[0], "Number of tokens mismatch"
    M = hidden_states.shape[0]
    dev = hidden_states.device
    topk_weights = torch.empty((M, topk), dtype=torch.float32, device=dev)
    topk_ids = torch.empty((M, topk), dtype=torch.int32, device=dev)
    token_expert_indices = torch.empty((M, topk), dtype=torch.int32, device=dev)
    logits = gating_output if gating_output.dtype == torch.float32 else gating_output.float()
    op = moe_ops.topk_softmax_renorm if renormalize else moe_ops.topk_softmax
    op(topk_weights, topk_ids, token_expert_indices, logits.contiguous())
    return topk_weights, topk_ids


def grouped_topk(hidden_states: torch.Tensor, gating_output: torch.Tensor, topk: int,
                 renormalize: bool, num_expert_group: int = 0,
                 topk_group: int = 0) -> Tuple[torch.Tensor, torch.Tensor]:
    """Group-limited routing (DeepSeek-V2): only experts of the ``topk_group`` best of
    ``num_expert_group`` expert groups can be selected.  Returns (topk_weights f32, topk_ids i32),
    in descending weight order (the reference's torch.topk(sorted=False) leaves the order open)."""
    assert hidden_states.shape[0] == gating_output.shape[0], "Number of tokens mismatch"
    M = hidden_states.shape[0]
    dev = hidden_states.device
    topk_weights = torch.empty((M, topk), dtype=torch.float32, device=dev)
    topk_ids = torch.empty((M, topk), dtype=torch.int32, device=dev)
    logits = gating_output if gating_output.dtype == torch.float32 else gating_output.float()
    moe_ops.grouped_topk(topk_weights, topk_ids, logits.contiguous(), num_expert_group, topk_group,
                         renormalize)
    return topk_weights, topk_ids


def moe_align_block_size(topk_ids: torch.Tensor, block_size: int,
                         num_experts: int) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """Sorts the flat (token, k) slots by expert and pads every expert's run to a multiple of
    ``block_size``.  Returns (sorted_token_ids, expert_ids, num_tokens_post_padded) with the buffer
    sizes of the reference wrapper; padding slots hold ``topk_ids.numel()`` (written by the kernel
    itself, so there is no separate fill)."""
    numel = topk_ids.numel()
    max_padded = numel + num_experts * (block_size - 1)
    dev = topk_ids.device
    sorted_ids = torch.empty((max_padded,), dtype=torch.int32, device=dev)
    expert_ids = torch.empty(((max_padded + block_size - 1) // block_size,), dtype=torch.int32,
                             device=dev)
    num_tokens_post_pad = torch.empty((1,), dtype=torch.int32, device=dev)
    moe_ops.moe_align_block_size_filled(topk_ids.contiguous(), num_experts, block_size, sorted_ids,
                                        expert_ids, num_tokens_post_pad)
    return sorted_ids, expert_ids, num_tokens_post_pad


GEMM_TILE_SLOTS = 32   # slots of one matrix-core tile of the grouped GEMM kernels


def balance_blocks(sorted_token_ids: torch.Tensor, expert_ids: torch.Tensor,
                   num_tokens_post_padded: torch.Tensor, block_size: int, num_experts: int,
                   numel: int, packed: bool = False) -> torch.Tensor:
    """``moe_align_block_size``'s ``sorted_token_ids`` with every expert's slots spread evenly over
    its blocks instead of filling them one after the other (no counterpart in the reference; the
    grouped GEMM runs 8-10 % faster on it when experts have a nearly empty last block, with
    bit-identical results).  ``expert_ids`` and ``num_tokens_post_padded`` stay valid for the
    returned tensor; ``numel`` is the padding value (``topk_ids.numel()``).  ``packed`` names the
    weight layout of the GEMM that will read the result: the kernels differ in how their waves
    split a block's slots, and the deal follows that split."""
    out = torch.empty_like(sorted_token_ids)
    rows = moe_ops.moe_gemm_slot_rows(block_size, packed)
    moe_ops.moe_balance_blocks(sorted_token_ids, out, expert_ids, num_tokens_post_padded,
                               num_experts, block_size, numel,
                               min(GEMM_TILE_SLOTS, block_size // rows), rows)
    return out


def fused_topk_and_align(hidden_states: torch.Tensor, gating_output: torch.Tensor, topk: int,
                         renormalize: bool, block_size: int):
    """``fused_topk`` followed by ``moe_align_block_size`` in one call: ONE kernel launch up to
    1024 (token, k) slots and a power-of-two expert count up to 16; other shapes run the two kernels.
    Returns (topk_weights, topk_ids, sorted_token_ids, expert_ids, num_tokens_post_padded), the
    same tensors the two separate calls return."""
    assert hidden_states.shape[0] == gating_output.shape[0], "Number of tokens mismatch"
    M, E = gating_output.shape
    dev = hidden_states.device
    topk_weights = torch.empty((M, topk), dtype=torch.float32, device=dev)
    topk_ids = torch.empty((M, topk), dtype=torch.int32, device=dev)
    token_expert_indices = torch.empty((M, topk), dtype=torch.int32, device=dev)
    max_padded = M * topk + E * (block_size - 1)
    sorted_ids = torch.empty((max_padded,), dtype=torch.int32, device=dev)
    expert_ids = torch.empty(((max_padded + block_size - 1) // block_size,), dtype=torch.int32,
                             device=dev)
    num_tokens_post_pad = torch.empty((1,), dtype=torch.int32, device=dev)
    logits = gating_output if gating_output.dtype == torch.float32 else gating_output.float()
    moe_ops.fused_topk_align(topk_weights, topk_ids, token_expert_indices, logits.contiguous(),
                             renormalize, block_size, sorted_ids, expert_ids, num_tokens_post_pad,
                             True)
    return topk_weights, topk_ids, sorted_ids, expert_ids, num_tokens_post_pad
