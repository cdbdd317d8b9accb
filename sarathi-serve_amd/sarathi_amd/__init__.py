"""MI355X (gfx950) implementation of the op library that Sarathi-Serve's csrc/
provides to sarathi.model_executor.layers.

The four op namespaces keep the reference's module names and positional
signatures (the reference builds them as four pybind11 modules, setup.py:95-136):

    from sarathi_amd import layernorm_ops, activation_ops, pos_encoding_ops, moe_ops

    layernorm_ops.rms_norm(out, input, weight, epsilon)
    layernorm_ops.fused_add_rms_norm(input, residual, weight, epsilon)   # new
    activation_ops.silu_and_mul(out, input) / gelu_new / gelu_fast
    pos_encoding_ops.rotary_embedding(positions, query, key, head_size, cos_sin_cache, is_neox)
    moe_ops.topk_softmax(topk_weights, topk_indices, token_expert_indices, gating_output)
    moe_ops.moe_align_block_size(topk_ids, num_experts, block_size, sorted_token_ids,
                                 experts_ids, num_tokens_post_pad)

``kv_cache_ops`` adds the paged KV-cache append that follows the rotary embedding on the
reference's attention path (flashinfer's get_seq_lens / get_batch_indices_positions /
append_paged_kv_cache signatures) and its fusion with rotary_embedding.

All ops return None, write through out-parameters or in place, and launch
asynchronously on torch's current stream.  There is no CPU or PyTorch fallback:
importing this package raises ImportError when the compiled HIP extension is
missing.  ``sarathi_amd.layers`` holds counterparts of the reference's Python
layer classes that call these ops.
"""
from . import _ext  # noqa: F401  (raises ImportError if the HIP extension is not built)
from . import activation_ops, kv_cache_ops, layernorm_ops, moe_ops, pos_encoding_ops  # noqa: F401

__all__ = ["layernorm_ops", "activation_ops", "pos_encoding_ops", "moe_ops", "kv_cache_ops"]
