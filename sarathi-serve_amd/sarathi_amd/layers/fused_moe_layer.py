"""FusedMoE layer module (reference: sarathi/model_executor/layers/fused_moe/layer.py:12-134):
owns the fused gate/up projection weights ``w13_weight [E, 2*I, H]`` and the down projection
weights ``w2_weight [E, H, I]`` of all experts and applies ``fused_moe`` to a batch.

This library runs one process on one GPU, so the tensor-parallel degree is 1: the intermediate
size is not partitioned and ``reduce_results`` has nothing to reduce.  The reference's per-layer
timers (``linear_metric_name`` etc.) belong to its metrics subsystem; the arguments are accepted and
ignored.
"""
from typing import Optional

import torch

from .fused_moe import fused_moe, pack_expert_weights


class FusedMoE(torch.nn.Module):

    def __init__(self, num_experts: int, top_k: int, hidden_size: int, intermediate_size: int,
                 params_dtype: Optional[torch.dtype] = None, reduce_results: bool = False,
                 renormalize: bool = True, use_grouped_topk: bool = False,
                 num_expert_group: Optional[int] = None, topk_group: Optional[int] = None,
                 linear_metric_name: Optional[str] = None,
                 communication_metric_name: Optional[str] = None,
                 world_size: Optional[int] = None, layer_id: Optional[int] = None):
        super().__init__()
        if params_dtype is None:
            params_dtype = torch.get_default_dtype()
        self.params_dtype = params_dtype
        self.tp_size = 1
        self.top_k = top_k
        self.num_experts = num_experts
        self.hidden_size = hidden_size
        self.intermediate_size_per_partition = intermediate_size // self.tp_size
        self.reduce_results = reduce_results
        self.renormalize = renormalize
        self.use_grouped_topk = use_grouped_topk
        if self.use_grouped_topk:
            assert num_expert_group is not None and topk_group is not None
        self.num_expert_group = num_expert_group
        self.topk_group = topk_group
        self.world_size = 1 if world_size is None else world_size
        if self.reduce_results and self.world_size > 1:
            raise NotImplementedError("this library runs on one GPU: there is no tensor-parallel "
                                      "group to reduce over")
        self._packed = None
        self.create_weights()

    def create_weights(self):
        dev = torch.device("cuda") if torch.cuda.is_available() else None
        self.w13_weight = torch.nn.Parameter(
            torch.empty(self.num_experts, 2 * self.intermediate_size_per_partition,
                        self.hidden_size, dtype=self.params_dtype, device=dev),
            requires_grad=False)
        self.w2_weight = torch.nn.Parameter(
            torch.empty(self.num_experts, self.hidden_size, self.intermediate_size_per_partition,
                        dtype=self.params_dtype, device=dev),
            requires_grad=False)

    def pack_weights(self, inplace: bool = False) -> None:
        """Re-tile both weight tensors once, after loading, into the order the grouped GEMM's
        matrix-core loads consume (same results; within a few per cent of the row-major path at every
        batch size, so this is optional).  By default this keeps a
        second copy of the weights; ``inplace=True`` re-tiles inside the parameters' own storage
        (no extra memory; the parameters then hold the packed values).  Call again after changing
        the weights."""
        self._packed = (pack_expert_weights(self.w13_weight.data, inplace=inplace),
                        pack_expert_weights(self.w2_weight.data, inplace=inplace))

    def apply_weights(self, x: torch.Tensor, router_logits: torch.Tensor) -> torch.Tensor:
        w13, w2 = self._packed if self._packed is not None else (self.w13_weight, self.w2_weight)
        return fused_moe(x, w13, w2, router_logits, self.top_k, renormalize=self.renormalize,
                         inplace=True, use_grouped_topk=self.use_grouped_topk,
                         num_expert_group=self.num_expert_group, topk_group=self.topk_group)

    def forward(self, hidden_states: torch.Tensor, router_logits: torch.Tensor) -> torch.Tensor:
        return self.apply_weights(x=hidden_states, router_logits=router_logits)
