"""ctypes front end of ``sarathi_ops_oracle.c``.  TEST INFRASTRUCTURE ONLY.

All functions take CPU torch tensors, follow the positional signatures of the
reference's pybind modules (csrc/layernorm.cpp:9, csrc/activation.cpp:15,
csrc/pos_encoding.cpp:11, csrc/moe.cpp:19) and write through out-parameters or
in place, returning ``None``.
"""
import ctypes
import os
import subprocess

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "_build", "libsarathi_ops_oracle.so")

_DT = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}
_ID_DT = {torch.uint8: 0, torch.int8: 1, torch.int16: 2, torch.int32: 3, torch.int64: 4}


def build(force: bool = False) -> str:
    """Compile the C oracle with gcc (seconds).  Returns the library path."""
    src = os.path.join(_HERE, "sarathi_ops_oracle.c")
    stale = (not os.path.exists(_SO)) or (
        os.path.exists(src) and os.path.getmtime(src) > os.path.getmtime(_SO)
    )
    if force or stale:
        if not os.path.exists(src):
            raise RuntimeError("oracle source missing and no prebuilt library")
        subprocess.check_call(["make", "-C", _HERE] + (["-B"] if force else []),
                              stdout=subprocess.DEVNULL)
    return _SO


_lib = None


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        _lib = ctypes.CDLL(build())
        _lib.oracle_f16_to_f32.restype = ctypes.c_float
        _lib.oracle_f16_to_f32.argtypes = [ctypes.c_uint16]
        _lib.oracle_f32_to_f16.restype = ctypes.c_uint16
        _lib.oracle_f32_to_f16.argtypes = [ctypes.c_float]
        _lib.oracle_f32_to_bf16.restype = ctypes.c_uint16
        _lib.oracle_f32_to_bf16.argtypes = [ctypes.c_float]
    return _lib


def _p(t: torch.Tensor) -> ctypes.c_void_p:
    assert t.device.type == "cpu", "the oracle runs on CPU tensors only"
    return ctypes.c_void_p(t.data_ptr())


def _i64(v) -> ctypes.c_int64:
    return ctypes.c_int64(int(v))


def rms_norm(out, input, weight, epsilon):
    assert input.is_contiguous() and out.is_contiguous() and input.dim() == 2
    T, H = input.shape
    lib().oracle_rms_norm(_p(out), _p(input), _p(weight), ctypes.c_float(epsilon),
                          _i64(T), ctypes.c_int(H), ctypes.c_int(_DT[input.dtype]))


def fused_add_rms_norm(input, residual, weight, epsilon):
    assert input.is_contiguous() and residual.is_contiguous() and input.dim() == 2
    T, H = input.shape
    lib().oracle_fused_add_rms_norm(_p(input), _p(residual), _p(weight),
                                    ctypes.c_float(epsilon), _i64(T), ctypes.c_int(H),
                                    ctypes.c_int(_DT[input.dtype]))


def _act(name, out, input, halve):
    assert input.is_contiguous() and out.is_contiguous()
    d = input.shape[-1] // 2 if halve else input.shape[-1]
    T = input.numel() // input.shape[-1]
    getattr(lib(), name)(_p(out), _p(input), _i64(T), _i64(d), ctypes.c_int(_DT[input.dtype]))


def silu_and_mul(out, input):
    _act("oracle_silu_and_mul", out, input, True)


def gelu_new(out, input):
    _act("oracle_gelu_new", out, input, False)


def gelu_fast(out, input):
    _act("oracle_gelu_fast", out, input, False)


def rotary_embedding(positions, query, key, head_size, cos_sin_cache, is_neox):
    assert positions.dtype == torch.int64 and positions.is_contiguous()
    assert query.stride(-1) == 1 and key.stride(-1) == 1 and cos_sin_cache.is_contiguous()
    T = query.shape[0]
    lib().oracle_rotary_embedding(
        _p(positions), _p(query), _p(key), _p(cos_sin_cache), _i64(T),
        ctypes.c_int(query.shape[1] // head_size), ctypes.c_int(key.shape[1] // head_size),
        ctypes.c_int(head_size), ctypes.c_int(cos_sin_cache.shape[1]),
        _i64(query.stride(0)), _i64(key.stride(0)), ctypes.c_int(bool(is_neox)),
        ctypes.c_int(_DT[query.dtype]))


def topk_softmax(topk_weights, topk_indices, token_expert_indices, gating_output):
    assert gating_output.dtype == torch.float32 and gating_output.is_contiguous()
    E = gating_output.shape[-1]
    T = gating_output.numel() // E
    k = topk_weights.shape[-1]
    lib().oracle_topk_softmax(_p(topk_weights), _p(topk_indices), _p(token_expert_indices),
                              _p(gating_output), _i64(T), ctypes.c_int(E), ctypes.c_int(k))


def moe_align_block_size(topk_ids, num_experts, block_size, sorted_token_ids, experts_ids,
                         num_tokens_post_pad):
    assert topk_ids.is_contiguous()
    lib().oracle_moe_align_block_size(
        _p(topk_ids), ctypes.c_int(_ID_DT[topk_ids.dtype]), _i64(topk_ids.numel()),
        ctypes.c_int(num_experts), ctypes.c_int(block_size), _p(sorted_token_ids),
        _p(experts_ids), _p(num_tokens_post_pad))
