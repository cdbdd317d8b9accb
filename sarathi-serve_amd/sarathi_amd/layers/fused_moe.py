"""Fused MoE forward on this package's ops (reference:
sarathi/model_executor/layers/fused_moe/fused_moe.py:207-260 and :411-622).

``fused_moe`` = top-k routing -> slot sort (moe_align_block_size) -> grouped GEMM with w1 ->
silu_and_mul -> grouped GEMM with w2 (times the routing weight) -> sum over the k slots of a token.
The two GEMMs are hand-written MFMA kernels (csrc/moe_gemm.hip, csrc/moe_gemm_wide.hip) instead of
the reference's Triton kernel.  Their only free parameter is the slot-block size, which comes from
the tuned tables under ``configs/`` (the reference's JSON format, written by tune_fused_moe.py)
when one matches (E, N, device, weight layout), else from ``get_default_config``.
float16 and bfloat16 run the tuned kernels; float32 tensors (which the reference admits,
fused_moe.py:430) run a plain float32 matrix-core kernel (csrc/moe_gemm_f32.hip) on row-major
weights, with the reference's rounding of every GEMM output through float16 (fused_moe.py:142, 466);
fp8 weights / scales raise.
"""
import functools
import json
import os
from typing import Any, Dict, Optional, Tuple

import torch

from .. import activation_ops, moe_ops
from .moe_routing import (balance_blocks, fused_topk, fused_topk_and_align, grouped_topk,
                          moe_align_block_size)

_BLOCK_SIZES = (32, 64, 128, 256)


class PackedExpertWeights:
    """Expert weights [E, N, K] re-tiled once into the order the matrix cores consume them
    (see ``pack_expert_weights``).  Pass it wherever ``fused_moe`` / ``fused_experts`` /
    ``invoke_fused_moe_kernel`` take ``w1`` / ``w2`` / ``B``; results are the same as with the
    row-major tensor and the grouped GEMM runs within a few per cent of the row-major path
    (faster or slower, by batch size), so packing is optional."""

    def __init__(self, data: torch.Tensor, shape):
        self.data = data                      # [E, ceil(N/32), K/16, 2, 32, 8]
        self.shape = torch.Size(shape)        # logical (E, N, K)
        self.dtype = data.dtype
        self.device = data.device

    def is_contiguous(self) -> bool:
        return True


def pack_expert_weights(w: torch.Tensor, inplace: bool = False) -> PackedExpertWeights:
    """[E, N, K] -> tiles of 32 rows x 16 columns stored as 64 lanes x 8 elements, lane =
    (n mod 32) + 32 * ((k mod 16) // 8).  K must be a multiple of 16; N is padded with zero rows
    to a multiple of 32.  Do this once when the weights are loaded.

    ``inplace=True`` re-tiles expert by expert inside ``w``'s own storage (one expert's matrix of
    temporary memory instead of a second copy of all weights); ``w`` then no longer holds the
    row-major values and must only be used through the returned object.  Needs N % 32 == 0 and a
    contiguous ``w``."""
    E, N, K = w.shape
    assert K % 16 == 0, "K must be a multiple of 16"
    n_pad = (N + 31) // 32 * 32

    def tile(m: torch.Tensor) -> torch.Tensor:      # [n_pad, K] -> [n_pad/32, K/16, 2, 32, 8]
        return m.reshape(n_pad // 32, 32, K // 16, 2, 8).permute(0, 2, 3, 1, 4).contiguous()

    if inplace:
        assert n_pad == N and w.is_contiguous(), "in-place packing needs N % 32 == 0, contiguous w"
        for e in range(E):
            w[e].view(-1).copy_(tile(w[e]).view(-1))
        return PackedExpertWeights(w.view(E, N // 32, K // 16, 2, 32, 8), (E, N, K))
    if n_pad != N:
        w = torch.cat((w, w.new_zeros((E, n_pad - N, K))), dim=1)
    tiles = torch.stack([tile(w[e]) for e in range(E)])
    return PackedExpertWeights(tiles, (E, N, K))


# fused_moe asks for routing and slot sort in one call (fused_topk_align) up to this many
# (token, k) slots and experts; the op itself runs them as one launch up to 1024 slots and as the
# two stand-alone kernels above that.  Measured on MI355X, launches issued back to back from
# Python, E = 8, top-2:
#   tokens      16     256    512    1024   2048   4096
#   two ops     6.8    6.9    6.7    7.1    7.7    8.9   us
#   one launch  5.7    6.1    6.7    7.3    9.0    12.5  us
FUSED_ROUTING_MAX_SLOTS = 1024
FUSED_ROUTING_MAX_EXPERTS = 16
# silu_and_mul inside the gate/up GEMM's epilogue (same bits as the separate kernel)
FUSE_SILU_AND_MUL = True
# Spread every expert's slots evenly over its blocks before the GEMMs (moe_routing.balance_blocks)
# whenever some expert can have more than one block.  Off: on the Mixtral layer at 4096 tokens it
# cuts the bytes the GEMMs pull over the fabric by 8-15 % and leaves the time where it was (row-major
# forward 2.69 ms greedy, 2.73 ms even; packed 2.66 / 2.67): a workgroup's time is mostly a fixed
# cost per slot block, and an even fill has as many blocks as a greedy one.
BALANCE_BLOCKS = False
# Riders (moe_ops.moe_plan_riders): the few slots of an expert's partly filled last block are taken
# along by the workgroups of its full blocks.  Row-major 16-bit weights at 256-slot blocks.
RIDERS = True
# ... and the experts whose last block cannot ride (more 32-slot tiles in it than the expert has
# full blocks) get their slots spread evenly over the two 128-slot halves of each of their blocks:
# a block costs the GEMM as much as its fuller half (moe_ops.moe_plan_blocks: both in one launch).
# Planned from a mean load of half a block per expert: below that the even fill wakes the second
# pair of waves of every workgroup for a tile or two and costs 2-10 %.  Same bits either way.
# Mixtral layer forward, N(0, 1) router logits, MI355X, ms (off: neither; on: both, the default;
# riders: RIDERS_EVEN_REST = False):
#   tokens   512    640    1024   1280   1536   2048   2560   3072   4096   6144
#   off      0.651  0.680  0.934  1.130  1.183  1.558  1.860  2.097  2.731  3.959
#   on       0.631  0.664  0.907  1.035  1.112  1.421  1.810  2.065  2.569  3.777
#   riders   0.651  0.685  0.911  1.121  1.181  1.415  1.843  2.069  2.568  3.772
RIDERS_EVEN_REST = True
CHUNK_SIZE = 64 * 1024     # tokens per pass, as in the reference (fused_moe.py:437)


def get_default_config(M: int, E: int, N: int, K: int, topk: int, dtype: Optional[str] = None,
                       packed: bool = True) -> Dict[str, int]:
    """Slot-block size for M tokens: the more slots an expert receives, the taller the tile (a
    taller tile re-uses each weight fragment for more tokens).  Thresholds from sweeps of the
    Mixtral-8x7B, Mixtral-8x22B and a 64-expert shape on MI355X (tune_fused_moe.py): with packed
    weights 128 and 256 are within a few per cent of each other at large batches (the tuned
    tables pick per batch size); row-major weights run the four-wave kernel, with 64-slot blocks
    (small tiles, several workgroups per compute unit: weight streaming) up to ~64 slots per expert
    and 256-slot blocks (128 x 128 wave tiles) beyond, a little later with many experts.
    BLOCK_SIZE_N / BLOCK_SIZE_K are fixed properties of the kernels, reported for information."""
    per_expert = M * topk / max(E, 1)
    if not packed:
        block_m = 256 if per_expert >= (64 if E <= 16 else 128) else 64
    else:
        block_m = 128 if per_expert >= 48 else 64 if per_expert >= 10 else 32
    return {"BLOCK_SIZE_M": block_m, "BLOCK_SIZE_N": 256, "BLOCK_SIZE_K": 64, "GROUP_SIZE_M": 1}


def get_config_file_name(E: int, N: int, dtype: Optional[str], packed: bool = True) -> str:
    """The reference's naming rule (fused_moe.py:262-265), plus a ``,layout=row_major`` selector
    for tables tuned on un-packed weights."""
    device_name = torch.cuda.get_device_name().replace(" ", "_")
    return f"E={E},N={N},device_name={device_name}{_selectors(dtype, packed)}.json"


def _selectors(dtype: Optional[str], packed: bool) -> str:
    return ("" if not dtype else f",dtype={dtype}") + ("" if packed else ",layout=row_major")


CONFIG_DIR = os.path.join(os.path.dirname(os.path.realpath(__file__)), "configs")


@functools.lru_cache
def get_moe_configs(E: int, N: int, dtype: Optional[str],
                    packed: bool = True) -> Optional[Dict[int, Any]]:
    """Tuned slot-block sizes for this (E, N) on this device, as a map batch size -> config, or
    None (reference: fused_moe.py:268-294).  Files are written by ``tune_fused_moe.py``.  MI355X
    boards report different marketing names depending on the driver, so a file named for the
    architecture (``device_name=gfx950``) is tried after the one named for the device."""
    names = [get_config_file_name(E, N, dtype, packed)]
    arch = getattr(torch.cuda.get_device_properties(torch.cuda.current_device()), "gcnArchName", "")
    if arch:
        names.append(f"E={E},N={N},device_name={arch.split(':')[0]}{_selectors(dtype, packed)}.json")
    for name in names:
        path = os.path.join(CONFIG_DIR, name)
        if os.path.exists(path):
            with open(path) as f:
                return {int(key): val for key, val in json.load(f).items()}
    return None


def try_get_optimal_moe_config(w1_shape: Tuple[int, ...], w2_shape: Tuple[int, ...], top_k: int,
                               M: int, dtype: Optional[str] = None,
                               override_config: Optional[Dict[str, Any]] = None,
                               packed: bool = True) -> Dict[str, Any]:
    """override_config, else the tuned entry closest to M, else the default rule
    (reference: fused_moe.py:321-343).  An override written for the reference's Triton kernel may
    name a slot-block size this library's kernels do not have (the reference's default for tiny
    batches is 16): it is raised to the next size that exists, the other keys pass through."""
    if override_config:
        block_m = int(override_config["BLOCK_SIZE_M"])
        if block_m in _BLOCK_SIZES:
            return override_config
        config = dict(override_config)
        config["BLOCK_SIZE_M"] = min((b for b in _BLOCK_SIZES if b >= block_m),
                                     default=max(_BLOCK_SIZES))
        return config
    E, _, N = w2_shape
    configs = get_moe_configs(E, N, dtype, packed)
    if configs:
        return configs[min(configs.keys(), key=lambda x: abs(x - M))]
    return get_default_config(M, E, N, w1_shape[2], top_k, dtype, packed)


def invoke_fused_moe_kernel(A: torch.Tensor, B: torch.Tensor, C: torch.Tensor,
                            A_scale: Optional[torch.Tensor], B_scale: Optional[torch.Tensor],
                            topk_weights: torch.Tensor, topk_ids: torch.Tensor,
                            sorted_token_ids: torch.Tensor, expert_ids: torch.Tensor,
                            num_tokens_post_padded: torch.Tensor, mul_routed_weight: bool,
                            top_k: int, config: Dict[str, Any], compute_type=None,
                            silu_and_mul: bool = False,
                            riders: Optional[torch.Tensor] = None) -> None:
    """Same argument list as the reference's launcher.  ``config["BLOCK_SIZE_M"]`` must be the block
    size ``sorted_token_ids`` was aligned with.  ``silu_and_mul=True`` (not in the reference):
    ``B`` is a gate/up projection ``[E, 2I, K]`` and ``C [.., I]`` receives
    ``silu_and_mul(A @ B^T)`` directly, bit-identical to running the two ops separately."""
    assert A_scale is None and B_scale is None, "fp8 scales are not supported"
    assert topk_weights.stride(1) == 1 and sorted_token_ids.stride(0) == 1
    block_m = int(config["BLOCK_SIZE_M"])
    if block_m not in _BLOCK_SIZES:
        raise ValueError(f"BLOCK_SIZE_M must be one of {_BLOCK_SIZES}, got {block_m}")
    packed = isinstance(B, PackedExpertWeights)
    moe_ops.moe_grouped_gemm(A, B.data if packed else B, C, topk_weights, sorted_token_ids,
                             expert_ids, num_tokens_post_padded, topk_ids.numel(), block_m, top_k,
                             bool(mul_routed_weight), packed, B.shape[1], bool(silu_and_mul),
                             riders)


def fused_experts(hidden_states: torch.Tensor, w1: torch.Tensor, w2: torch.Tensor,
                  topk_weights: torch.Tensor, topk_ids: torch.Tensor, inplace: bool = False,
                  override_config: Optional[Dict[str, Any]] = None,
                  w1_scale: Optional[torch.Tensor] = None, w2_scale: Optional[torch.Tensor] = None,
                  a1_scale: Optional[torch.Tensor] = None,
                  a2_scale: Optional[torch.Tensor] = None, _alignment=None) -> torch.Tensor:
    """``_alignment``: (sorted_token_ids, expert_ids, num_tokens_post_padded, block_size) already
    computed for the whole batch by the fused routing launch (single-chunk batches only)."""
    assert hidden_states.shape[1] == w1.shape[2], "Hidden size mismatch"
    assert topk_weights.shape == topk_ids.shape, "topk shape mismatch"
    assert hidden_states.is_contiguous(), "Hidden_states must be contiguous"
    assert w1.is_contiguous() and w2.is_contiguous(), "Expert weights must be contiguous"
    if hidden_states.dtype not in (torch.float32, torch.float16, torch.bfloat16) \
            or w1.dtype != hidden_states.dtype or w2.dtype != hidden_states.dtype:
        raise TypeError("fused_experts needs float32, float16 or bfloat16 activations and expert weights "
                        f"of the same dtype: got hidden_states {hidden_states.dtype}, w1 {w1.dtype}, "
                        f"w2 {w2.dtype}")
    is_f32 = hidden_states.dtype == torch.float32
    if is_f32 and (isinstance(w1, PackedExpertWeights) or isinstance(w2, PackedExpertWeights)):
        raise TypeError("packed expert weights are a 16-bit layout; float32 runs on the [E, N, K] tensors")
    assert w1_scale is None and w2_scale is None and a1_scale is None and a2_scale is None, \
        "fp8 scales are not supported"
    num_tokens, K = hidden_states.shape
    E, N, _ = w1.shape
    topk = topk_ids.shape[1]
    dev, dt = hidden_states.device, hidden_states.dtype
    # the GEMM addresses its activations with 32-bit byte offsets: keep both inputs below 4 GiB
    chunk = CHUNK_SIZE
    eb = hidden_states.element_size()
    while chunk > 1 and max(chunk * K, chunk * topk * (N // 2)) * eb + 4 * max(K, N) >= 1 << 32:
        chunk //= 2
    M = min(num_tokens, chunk)
    # gate/up GEMM with the activation fused into its epilogue: no [M, topk, N] intermediate
    fuse_act = FUSE_SILU_AND_MUL and (N // 2) % 32 == 0 and not is_f32
    cache1 = None if fuse_act else torch.empty((M, topk, N), device=dev, dtype=dt)
    cache2 = torch.empty((M * topk, N // 2), device=dev, dtype=dt)
    cache3 = torch.empty((M, topk, w2.shape[1]), device=dev, dtype=dt)
    out = hidden_states if inplace else torch.empty_like(hidden_states)
    topk_weights = topk_weights.contiguous()
    for begin in range(0, num_tokens, chunk):
        end = min(begin + chunk, num_tokens)
        n = end - begin
        cur_hidden = hidden_states[begin:end]
        cur_ids, cur_w = topk_ids[begin:end], topk_weights[begin:end]
        config = try_get_optimal_moe_config(tuple(w1.shape), tuple(w2.shape), topk, n,
                                            override_config=override_config,
                                            packed=isinstance(w1, PackedExpertWeights))
        c2, c3 = cache2[:n * topk], cache3[:n]
        if _alignment is not None and n == num_tokens and _alignment[3] == config["BLOCK_SIZE_M"]:
            sorted_ids, expert_ids, post_padded = _alignment[:3]
        else:
            sorted_ids, expert_ids, post_padded = moe_align_block_size(
                cur_ids, config["BLOCK_SIZE_M"], E)
        if BALANCE_BLOCKS and config["BLOCK_SIZE_M"] >= 64 and n * topk > config["BLOCK_SIZE_M"]:
            sorted_ids = balance_blocks(sorted_ids, expert_ids, post_padded,
                                        config["BLOCK_SIZE_M"], E, n * topk,
                                        packed=isinstance(w1, PackedExpertWeights))
        riders = None
        if (RIDERS and config["BLOCK_SIZE_M"] == 256 and not is_f32 and 2 * n * topk >= 256 * E
                and not isinstance(w1, PackedExpertWeights)
                and not isinstance(w2, PackedExpertWeights)
                and not (BALANCE_BLOCKS and config["BLOCK_SIZE_M"] >= 64)):
            riders = torch.empty((expert_ids.numel(),), dtype=torch.int32, device=dev)
            if RIDERS_EVEN_REST:
                planned = torch.empty_like(sorted_ids)
                moe_ops.moe_plan_blocks(sorted_ids, planned, expert_ids, post_padded, E, 256,
                                        n * topk, riders)
                sorted_ids = planned
            else:
                moe_ops.moe_plan_riders(sorted_ids, expert_ids, post_padded, n * topk, 256, riders)
        if fuse_act:
            invoke_fused_moe_kernel(cur_hidden, w1, c2, None, None, cur_w, cur_ids, sorted_ids,
                                    expert_ids, post_padded, False, topk, config,
                                    silu_and_mul=True, riders=riders)
        else:
            c1 = cache1[:n]
            invoke_fused_moe_kernel(cur_hidden, w1, c1, None, None, cur_w, cur_ids, sorted_ids,
                                    expert_ids, post_padded, False, topk, config, riders=riders)
            activation_ops.silu_and_mul(c2, c1.view(-1, N))
        invoke_fused_moe_kernel(c2, w2, c3, None, None, cur_w, cur_ids, sorted_ids, expert_ids,
                                post_padded, True, 1, config, riders=riders)
        moe_ops.moe_sum(c3, out[begin:end])   # the reference's torch.sum(c3, dim=1, out=...)
    return out


def fused_moe(hidden_states: torch.Tensor, w1: torch.Tensor, w2: torch.Tensor,
              gating_output: torch.Tensor, topk: int, renormalize: bool, inplace: bool = False,
              override_config: Optional[Dict[str, Any]] = None, use_grouped_topk: bool = False,
              num_expert_group: Optional[int] = None, topk_group: Optional[int] = None,
              w1_scale: Optional[torch.Tensor] = None, w2_scale: Optional[torch.Tensor] = None,
              a1_scale: Optional[torch.Tensor] = None,
              a2_scale: Optional[torch.Tensor] = None) -> torch.Tensor:
    """MoE layer forward: ``hidden_states [T, H]``, ``w1 [E, 2I, H]``, ``w2 [E, H, I]``,
    ``gating_output [T, E]`` (logits)."""
    assert gating_output.shape[1] == w1.shape[0], "Number of experts mismatch"
    num_tokens, E = gating_output.shape
    alignment = None
    if use_grouped_topk:
        assert num_expert_group is not None and topk_group is not None
        topk_weights, topk_ids = grouped_topk(hidden_states, gating_output, topk, renormalize,
                                              num_expert_group, topk_group)
    elif 0 < num_tokens * topk <= FUSED_ROUTING_MAX_SLOTS and E <= FUSED_ROUTING_MAX_EXPERTS:
        # small batches are launch-latency bound: routing and slot sort in one launch
        config = try_get_optimal_moe_config(tuple(w1.shape), tuple(w2.shape), topk, num_tokens,
                                            override_config=override_config,
                                            packed=isinstance(w1, PackedExpertWeights))
        block_m = config["BLOCK_SIZE_M"]
        topk_weights, topk_ids, sorted_ids, expert_ids, post_padded = fused_topk_and_align(
            hidden_states, gating_output, topk, renormalize, block_m)
        alignment = (sorted_ids, expert_ids, post_padded, block_m)
    else:
        topk_weights, topk_ids = fused_topk(hidden_states, gating_output, topk, renormalize)
    return fused_experts(hidden_states, w1, w2, topk_weights, topk_ids, inplace=inplace,
                         override_config=override_config, w1_scale=w1_scale, w2_scale=w2_scale,
                         a1_scale=a1_scale, a2_scale=a2_scale, _alignment=alignment)
