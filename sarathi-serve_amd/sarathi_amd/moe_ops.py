"""Counterpart of the reference's ``sarathi.moe_ops`` (csrc/moe.cpp:19-28).

``topk_softmax_renorm`` and ``moe_align_block_size_filled`` are fused variants:
the first also performs the caller-side renormalisation of
sarathi/model_executor/layers/fused_moe/fused_moe.py:371-372, the second the
caller-side ``sorted_ids.fill_(numel)`` of fused_moe.py:195.
"""
from ._ext import C as _C

topk_softmax = _C.topk_softmax
moe_align_block_size = _C.moe_align_block_size
topk_softmax_renorm = _C.topk_softmax_renorm
moe_align_block_size_filled = _C.moe_align_block_size_filled
# grouped expert GEMM over moe_align_block_size's layout: what the reference launches as a Triton
# kernel from invoke_fused_moe_kernel (layers/fused_moe/fused_moe.py:207-260)
moe_grouped_gemm = _C.moe_grouped_gemm
# fused_topk_align(topk_weights, topk_ids, token_expert_indices, gating_output, renormalize,
#                  block_size, sorted_token_ids, experts_ids, num_tokens_post_pad, fill_pad):
# topk_softmax(_renorm) and moe_align_block_size(_filled) in one launch, same outputs
fused_topk_align = _C.fused_topk_align
# grouped_topk(topk_weights, topk_ids, gating_output, num_expert_group, topk_group, renormalize):
# the group-limited routing the reference writes with tensor ops (fused_moe.py:377-408)
grouped_topk = _C.grouped_topk

# moe_balance_blocks(sorted_in, sorted_out, expert_ids, num_tokens_post_pad, num_experts, block_size,
#                    pad_value, granule, rows_per_block=1): moe_align_block_size's sort with every
# expert's slots spread evenly over its blocks, or over the rows_per_block equal ranges of each block
# (no counterpart in the reference; what fused_experts feeds its GEMMs)
moe_balance_blocks = _C.moe_balance_blocks
# moe_gemm_slot_rows(block_m, b_packed): the rows_per_block that suits moe_grouped_gemm's kernel
moe_gemm_slot_rows = _C.moe_gemm_slot_rows

# moe_plan_riders(sorted_token_ids, expert_ids, num_tokens_post_padded, num_valid_tokens, block_m,
#                 riders): fills `riders` (int32, one entry per slot block) for
# moe_grouped_gemm(..., riders=riders): the few slots of an expert's partly filled last block are
# multiplied by the workgroups of its full blocks instead of by workgroups of their own (row-major
# 16-bit weights, block_m = 256; no counterpart in the reference)
moe_plan_riders = _C.moe_plan_riders
# moe_plan_blocks(sorted_in, sorted_out, expert_ids, num_tokens_post_pad, num_experts, block_m,
#                 pad_value, riders): moe_plan_riders and moe_balance_blocks in one launch, chosen per
# expert: riders where the last block's tiles fit onto the expert's full blocks (layout kept), an
# even fill of the expert's blocks otherwise (block_m = 256)
moe_plan_blocks = _C.moe_plan_blocks

# moe_sum(input[tokens, top_k, hidden], out[tokens, hidden]): the torch.sum over the top-k expert
# outputs that ends fused_experts (fused_moe.py:539-543)
moe_sum = _C.moe_sum

__all__ = ["moe_sum", "moe_plan_riders", "moe_plan_blocks", "moe_balance_blocks", "moe_gemm_slot_rows", "topk_softmax", "moe_align_block_size", "topk_softmax_renorm",
           "moe_align_block_size_filled", "moe_grouped_gemm", "fused_topk_align", "grouped_topk"]
