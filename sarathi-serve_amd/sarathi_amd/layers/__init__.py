"""Counterparts of the reference's Python layer classes that sit directly on the ops
(sarathi/model_executor/layers/{layernorm,activation,rotary_embedding}.py and the routing helpers of
layers/fused_moe/fused_moe.py).  Same class / function names and call signatures, so model code written
against the reference's layers runs unchanged; the bodies call this package's HIP ops."""
from .activation import FastGELU, NewGELU, SiluAndMul, get_act_fn
from .fused_moe import (PackedExpertWeights, fused_experts, fused_moe, get_default_config,
                        get_moe_configs, invoke_fused_moe_kernel, pack_expert_weights,
                        try_get_optimal_moe_config)
from .fused_moe_layer import FusedMoE
from .kv_append import AppendMetadata, SequenceSlice, build_append_metadata
from .moe_routing import (balance_blocks, fused_topk, fused_topk_and_align, grouped_topk,
                          moe_align_block_size)
from .norm import RMSNorm
from .op_timer import op_timer, set_op_timer_factory
from .rotary import (DynamicNTKScalingRotaryEmbedding, LinearScalingRotaryEmbedding,
                     RotaryEmbedding, YaRNScalingRotaryEmbedding, get_rope)

__all__ = ["RMSNorm", "SiluAndMul", "NewGELU", "FastGELU", "get_act_fn", "RotaryEmbedding",
           "LinearScalingRotaryEmbedding", "DynamicNTKScalingRotaryEmbedding",
           "YaRNScalingRotaryEmbedding", "get_rope", "fused_topk", "fused_topk_and_align", "grouped_topk", "moe_align_block_size",
           "invoke_fused_moe_kernel", "fused_experts", "fused_moe", "FusedMoE", "get_default_config",
           "get_moe_configs", "try_get_optimal_moe_config", "pack_expert_weights",
           "PackedExpertWeights", "SequenceSlice", "AppendMetadata", "build_append_metadata",
           "op_timer", "set_op_timer_factory", "balance_blocks"]
