"""ctypes view of the C ABI (include/sarathi_ops.h) for the GPU tests that bypass the torch
binding: device pointers from ``tensor.data_ptr()``, torch's current stream as the
``hipStream_t``.  This is the stub a non-torch host would write; torch is used here only to
own the device memory.
"""
import ctypes
import os

import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB = os.path.join(ROOT, "sarathi-serve_amd", "sarathi_amd", "lib", "libsarathi_ops_hip.so")

DT = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}
ID_DT = {torch.uint8: 0, torch.int8: 1, torch.int16: 2, torch.int32: 3, torch.int64: 4}

vp, i64, ci, cf = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_float

_SIGNATURES = {
    "sarathi_rms_norm": [vp, vp, vp, cf, i64, i64, i64, i64, ci, vp],
    "sarathi_fused_add_rms_norm": [vp, vp, vp, cf, i64, i64, i64, i64, ci, vp],
    "sarathi_silu_and_mul": [vp, vp, i64, i64, i64, i64, ci, vp],
    "sarathi_gelu_new": [vp, vp, i64, i64, ci, vp],
    "sarathi_gelu_fast": [vp, vp, i64, i64, ci, vp],
    "sarathi_rotary_embedding": [vp, vp, vp, vp, i64, ci, ci, ci, ci, i64, i64, ci, ci, vp],
    "sarathi_topk_softmax": [vp, vp, vp, vp, i64, ci, ci, ci, vp],
    "sarathi_moe_align_block_size": [vp, ci, i64, ci, ci, vp, i64, vp, i64, vp, ci, vp, i64, vp],
    "sarathi_moe_align_block_size_static": [vp, ci, i64, ci, ci, vp, i64, vp, i64, vp, ci, vp],
    "sarathi_moe_sum": [vp, vp, i64, i64, i64, i64, i64, i64, ci, vp],
}


def load():
    """The C-ABI library, loaded after torch so that it binds to the HIP runtime torch loaded."""
    assert os.path.exists(LIB), "build the library first: python sarathi-serve_amd/build.py"
    lib = ctypes.CDLL(LIB)
    for name, argtypes in _SIGNATURES.items():
        fn = getattr(lib, name)
        fn.argtypes = argtypes
        fn.restype = ci
    lib.sarathi_moe_align_workspace_bytes.argtypes = [i64, ci]
    lib.sarathi_moe_align_workspace_bytes.restype = i64
    lib.sarathi_ops_strerror.restype = ctypes.c_char_p
    return lib


def ptr(t):
    assert t is None or t.is_cuda
    return vp(None) if t is None else vp(t.data_ptr())


def stream():
    return vp(torch.cuda.current_stream().cuda_stream)


def check(lib, rc):
    assert rc == 0, "C ABI returned %d: %s" % (rc, lib.sarathi_ops_strerror(rc).decode())


def align_buffers(numel, num_experts, block_size, device, fill=None):
    """Output buffers of moe_align_block_size sized as the reference's caller sizes them
    (sarathi/model_executor/layers/fused_moe/fused_moe.py:191-200)."""
    sorted_len = numel + num_experts * (block_size - 1)
    blocks = (sorted_len + block_size - 1) // block_size
    sorted_ids = torch.full((sorted_len,), numel if fill is None else fill, dtype=torch.int32,
                            device=device)
    expert_ids = torch.full((blocks,), -7, dtype=torch.int32, device=device)
    post_pad = torch.full((1,), -7, dtype=torch.int32, device=device)
    return sorted_ids, expert_ids, post_pad
