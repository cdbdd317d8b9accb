"""The C-ABI shared library loads and exports every entry point that include/sarathi_ops.h
declares; argument validation that happens before any GPU work returns the documented codes;
the PyTorch front end refuses CPU tensors.  No kernel is launched here."""
import ctypes
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "sarathi_ops.h")
LIB = os.path.join(ROOT, "sarathi-serve_amd", "sarathi_amd", "lib", "libsarathi_ops_hip.so")


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(sarathi_[a-z0-9_]+)\s*\(", text)))


@pytest.fixture(scope="module")
def lib():
    import sarathi_amd  # noqa: F401  loads torch (and with it the HIP runtime the library links to)
    assert os.path.exists(LIB), "build the library first: python sarathi-serve_amd/build.py"
    return ctypes.CDLL(LIB)


def test_header_declares_the_expected_entry_points():
    names = declared_functions()
    for n in ["sarathi_rms_norm", "sarathi_fused_add_rms_norm", "sarathi_silu_and_mul",
              "sarathi_gelu_new", "sarathi_gelu_fast", "sarathi_rotary_embedding",
              "sarathi_topk_softmax", "sarathi_moe_align_block_size",
              "sarathi_moe_align_workspace_bytes", "sarathi_ops_abi_version",
              "sarathi_ops_strerror"]:
        assert n in names


def test_library_exports_every_declared_symbol(lib):
    for name in declared_functions():
        assert hasattr(lib, name), "missing symbol " + name


def test_version_and_error_strings(lib):
    assert lib.sarathi_ops_abi_version() == 1
    lib.sarathi_ops_strerror.restype = ctypes.c_char_p
    assert lib.sarathi_ops_strerror(0) == b"ok"
    for code in (-1, -2, -3, -99):
        assert len(lib.sarathi_ops_strerror(code)) > 0


def test_argument_validation_without_gpu(lib):
    """Null pointers, negative sizes, bad strides and unknown dtype codes are rejected on the
    host before anything is launched; zero tokens is a successful no-op."""
    i64, f32, ci, vp = ctypes.c_int64, ctypes.c_float, ctypes.c_int, ctypes.c_void_p
    buf = ctypes.create_string_buffer(256)
    p = ctypes.cast(buf, vp)
    null = vp(None)
    INVALID, UNSUPPORTED, OK = -1, -2, 0
    rms = lib.sarathi_rms_norm
    assert rms(null, p, p, f32(1e-5), i64(1), i64(8), i64(8), i64(8), ci(2), null) == INVALID
    assert rms(p, p, p, f32(1e-5), i64(-1), i64(8), i64(8), i64(8), ci(2), null) == INVALID
    assert rms(p, p, p, f32(1e-5), i64(1), i64(8), i64(4), i64(8), ci(2), null) == INVALID  # stride < H
    assert rms(p, p, p, f32(1e-5), i64(1), i64(8), i64(8), i64(8), ci(7), null) == UNSUPPORTED
    assert rms(p, p, p, f32(1e-5), i64(0), i64(8), i64(8), i64(8), ci(2), null) == OK
    # an empty batch comes with null data pointers (an empty tensor owns no memory): still a no-op
    assert rms(null, null, p, f32(1e-5), i64(0), i64(8), i64(8), i64(8), ci(2), null) == OK
    fused = lib.sarathi_fused_add_rms_norm
    assert fused(p, null, p, f32(1e-5), i64(1), i64(8), i64(8), i64(8), ci(2), null) == INVALID
    assert fused(p, p, p, f32(1e-5), i64(0), i64(8), i64(8), i64(8), ci(2), null) == OK
    silu = lib.sarathi_silu_and_mul
    assert silu(p, null, i64(1), i64(8), i64(16), i64(8), ci(2), null) == INVALID
    assert silu(p, p, i64(1), i64(8), i64(8), i64(8), ci(2), null) == INVALID      # stride < 2d
    assert silu(p, p, i64(1), i64(8), i64(16), i64(8), ci(9), null) == UNSUPPORTED
    assert silu(p, p, i64(0), i64(8), i64(16), i64(8), ci(2), null) == OK
    assert silu(null, null, i64(0), i64(8), i64(16), i64(8), ci(2), null) == OK
    for gelu in (lib.sarathi_gelu_new, lib.sarathi_gelu_fast):
        assert gelu(null, p, i64(1), i64(8), ci(2), null) == INVALID
        assert gelu(p, p, i64(1), i64(0), ci(2), null) == INVALID
        assert gelu(p, p, i64(0), i64(8), ci(2), null) == OK
    rope = lib.sarathi_rotary_embedding
    args = lambda **kw: [kw.get("pos", p), p, p, kw.get("cache", p), i64(kw.get("T", 1)), ci(2), ci(1),  # noqa: E731
                         ci(kw.get("hs", 16)), ci(kw.get("rot", 16)), i64(kw.get("qs", 32)), i64(16),
                         ci(1), ci(kw.get("dt", 2)), null]
    assert rope(*args(pos=null)) == INVALID
    assert rope(*args(rot=15)) == INVALID            # odd rot_dim
    assert rope(*args(rot=32)) == INVALID            # rot_dim > head_size
    assert rope(*args(qs=16)) == INVALID             # stride < num_heads * head_size
    assert rope(*args(dt=5)) == UNSUPPORTED
    assert rope(*args(T=0)) == OK
    topk = lib.sarathi_topk_softmax
    assert topk(null, p, p, p, i64(1), ci(8), ci(2), ci(0), null) == INVALID
    assert topk(p, p, p, p, i64(1), ci(8), ci(9), ci(0), null) == INVALID   # topk > experts
    assert topk(p, p, p, p, i64(1), ci(0), ci(1), ci(0), null) == INVALID
    assert topk(p, p, p, p, i64(1), ci(2048), ci(1), ci(0), null) == UNSUPPORTED
    assert topk(p, p, p, p, i64(0), ci(8), ci(2), ci(0), null) == OK
    assert topk(null, null, null, null, i64(0), ci(8), ci(2), ci(0), null) == OK
    align = lib.sarathi_moe_align_block_size
    ws = (null, i64(0), null)      # workspace, workspace_bytes, stream
    assert align(p, ci(3), i64(4), ci(8), ci(4), null, i64(64), p, i64(16), p, ci(0), *ws) == INVALID
    assert align(p, ci(3), i64(4), ci(0), ci(4), p, i64(64), p, i64(16), p, ci(0), *ws) == INVALID
    assert align(p, ci(3), i64(4), ci(8), ci(4), p, i64(8), p, i64(16), p, ci(0), *ws) == INVALID  # sorted too short
    assert align(p, ci(3), i64(4), ci(8), ci(4), p, i64(64), p, i64(1), p, ci(0), *ws) == INVALID  # expert_ids too short
    assert align(p, ci(3), i64(4), ci(4096), ci(4), p, i64(64), p, i64(16), p, ci(0), *ws) == UNSUPPORTED
    assert align(p, ci(11), i64(4), ci(8), ci(4), p, i64(64), p, i64(16), p, ci(0), *ws) == UNSUPPORTED
    # no ids and block_size 1: the output buffers are empty and may be null; post_pad is written
    assert align(null, ci(3), i64(0), ci(8), ci(1), null, i64(0), null, i64(0), null, ci(0), *ws) == INVALID
    wsb = lib.sarathi_moe_align_workspace_bytes
    wsb.restype = ctypes.c_int64
    assert wsb(i64(8192), ci(8)) == 0                       # small inputs: single workgroup
    big = wsb(i64(131072), ci(8))
    assert big > 0 and big % 4 == 0 and wsb(i64(131072), ci(256)) > big
    assert wsb(i64(1 << 20), ci(1024)) <= (1024 * 1024 + 1025) * 4


def test_front_end_refuses_cpu_tensors_and_bad_shapes(ops):
    x = torch.zeros((2, 8), dtype=torch.bfloat16)
    w = torch.ones(8, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="must live on the GPU"):
        ops.layernorm_ops.rms_norm(torch.empty_like(x), x, w, 1e-5)
    with pytest.raises(RuntimeError, match="must live on the GPU"):
        ops.layernorm_ops.fused_add_rms_norm(x, x.clone(), w, 1e-5)
    with pytest.raises(RuntimeError, match="must live on the GPU"):
        ops.activation_ops.silu_and_mul(torch.empty((2, 4), dtype=torch.bfloat16), x)
    with pytest.raises(RuntimeError, match="must live on the GPU"):
        ops.pos_encoding_ops.rotary_embedding(torch.zeros(2, dtype=torch.int64), x, x.clone(), 8,
                                              torch.zeros((4, 8), dtype=torch.bfloat16), True)
    with pytest.raises(RuntimeError, match="must live on the GPU"):
        ops.moe_ops.topk_softmax(torch.empty((2, 2)), torch.empty((2, 2), dtype=torch.int32),
                                 torch.empty((2, 2), dtype=torch.int32), torch.zeros((2, 8)))
    with pytest.raises(RuntimeError, match="must live on the GPU"):
        ops.moe_ops.moe_align_block_size(torch.zeros((2, 2), dtype=torch.int32), 8, 4,
                                         torch.empty(36, dtype=torch.int32),
                                         torch.empty(9, dtype=torch.int32),
                                         torch.empty(1, dtype=torch.int32))


def test_op_namespaces_match_the_reference_module_surface(ops):
    """Attribute names of the four pybind modules the reference builds (setup.py:95-136)."""
    assert {"rms_norm", "fused_add_rms_norm"} <= set(dir(ops.layernorm_ops))
    assert {"silu_and_mul", "gelu_new", "gelu_fast"} <= set(dir(ops.activation_ops))
    assert {"rotary_embedding"} <= set(dir(ops.pos_encoding_ops))
    assert {"topk_softmax", "moe_align_block_size"} <= set(dir(ops.moe_ops))


def test_kv_cache_and_gemm_argument_validation_without_gpu(lib):
    i64, ci, vp = ctypes.c_int64, ctypes.c_int, ctypes.c_void_p
    buf = ctypes.create_string_buffer(256)
    p = ctypes.cast(buf, vp)
    null = vp(None)
    INVALID, UNSUPPORTED, OK = -1, -2, 0

    def append(**kw):
        return lib.sarathi_append_paged_kv_cache(
            kw.get("key", p), p, kw.get("bi", p), p, p, kw.get("vc", p), p, p, kw.get("slots", null),
            i64(kw.get("nnz", 1)), ci(2),
            ci(8), ci(kw.get("page", 4)), i64(kw.get("ks", 16)), i64(16),
            i64(kw.get("ps", 64)), i64(kw.get("es", 16)), ci(kw.get("dt", 2)), null)
    assert append(key=null) == INVALID
    assert append(vc=null) == INVALID
    assert append(bi=null) == INVALID     # neither index arrays nor a slot mapping
    assert append(bi=null, slots=p, nnz=0) == OK
    assert append(ks=8) == INVALID        # key rows narrower than heads * head_size
    assert append(es=8) == INVALID        # cache entries narrower than a row
    assert append(ps=32) == INVALID       # page stride < page_size * entry stride
    assert append(page=0) == INVALID
    assert append(dt=6) == UNSUPPORTED
    assert append(nnz=0) == OK

    assert lib.sarathi_get_seq_lens(null, p, p, i64(1), ci(4), null) == INVALID
    assert lib.sarathi_get_seq_lens(p, p, p, i64(1), ci(0), null) == INVALID
    assert lib.sarathi_get_seq_lens(p, p, p, i64(0), ci(4), null) == OK
    assert lib.sarathi_get_batch_indices_positions(p, p, null, p, i64(1), i64(1), null) == INVALID
    assert lib.sarathi_get_batch_indices_positions(p, p, p, p, i64(0), i64(0), null) == OK
    assert lib.sarathi_get_kv_slot_mapping(p, p, p, p, null, i64(1), ci(4), null) == INVALID
    assert lib.sarathi_get_kv_slot_mapping(null, null, p, p, null, i64(0), ci(4), null) == OK
    assert lib.sarathi_get_batch_indices_positions(p, p, null, null, i64(1), i64(0), null) == OK
    assert lib.sarathi_get_kv_slot_mapping(p, p, p, p, p, i64(0), ci(4), null) == OK

    def fused(**kw):
        return lib.sarathi_rotary_embedding_append_paged_kv(
            kw.get("pos", p), p, p, kw.get("value", p), p, p, p, p, p, p, p, null,
            i64(kw.get("T", 1)),
            i64(kw.get("n", 1)), ci(2), ci(1), ci(16), ci(kw.get("rot", 16)), i64(32),
            i64(kw.get("ks", 16)), i64(16), ci(4), i64(64), i64(16), ci(1), ci(0),
            ci(kw.get("dt", 2)), null)
    assert fused(pos=null) == INVALID
    assert fused(value=null) == INVALID
    assert fused(n=2) == INVALID          # more appended tokens than tokens
    assert fused(rot=18) == INVALID       # rot_dim > head_size
    assert fused(ks=8) == INVALID
    assert fused(dt=9) == UNSUPPORTED
    assert fused(T=0, n=0) == OK

    def gemm(**kw):
        return lib.sarathi_moe_grouped_gemm(
            kw.get("a", p), p, p, kw.get("w", p), p, p, p, i64(kw.get("valid", 4)), i64(64),
            i64(kw.get("n", 64)), i64(kw.get("k", 64)), i64(kw.get("astride", 64)),
            i64(64 * 128), i64(64), ci(kw.get("bm", 64)), ci(2), ci(kw.get("mul", 0)),
            ci(kw.get("layout", 0)), ci(kw.get("dt", 2)), null)
    assert gemm(a=null) == INVALID
    assert gemm(w=null, mul=1) == INVALID           # routing weights required when multiplying
    assert gemm(astride=32) == INVALID              # rows of A narrower than K
    assert gemm(layout=5) == INVALID
    assert gemm(mul=7) == INVALID                   # unknown epilogue code
    assert gemm(mul=2, n=66) == UNSUPPORTED         # gated: N/2 = 33 is not a multiple of 4
    assert gemm(bm=48) == UNSUPPORTED
    assert gemm(dt=0, layout=1) == UNSUPPORTED      # fp32: row-major weights only,
    assert gemm(dt=0, mul=2) == UNSUPPORTED         # no gated epilogue,
    assert gemm(dt=0, bm=48) == UNSUPPORTED         # blocks in multiples of its 32-slot tile
    assert gemm(dt=7) == UNSUPPORTED
    assert gemm(k=72, astride=72) == UNSUPPORTED    # K must be whole 64-wide steps
    assert gemm(valid=0) == OK


def test_new_entry_points_validate_arguments_without_gpu(lib):
    """sarathi_moe_gemm_slot_rows is a host-side table; sarathi_moe_balance_blocks and
    sarathi_stream_copy reject bad sizes before anything is launched."""
    i64, ci, vp = ctypes.c_int64, ctypes.c_int, ctypes.c_void_p
    buf = ctypes.create_string_buffer(256)
    p = ctypes.cast(buf, vp)
    q = vp(p.value + 128)
    null = vp(None)
    INVALID, UNSUPPORTED, OK = -1, -2, 0
    rows = lib.sarathi_moe_gemm_slot_rows
    assert [rows(ci(b), ci(0)) for b in (32, 64, 128, 256)] == [1, 2, 2, 2]     # row-major weights
    assert [rows(ci(b), ci(1)) for b in (32, 64, 128, 256)] == [1, 1, 1, 2]     # packed weights
    assert rows(ci(48), ci(0)) == UNSUPPORTED and rows(ci(64), ci(7)) == INVALID

    def balance(**kw):
        return lib.sarathi_moe_balance_blocks(
            kw.get("src", p), kw.get("dst", q), p, p, i64(kw.get("n", 64)), ci(kw.get("e", 8)),
            ci(kw.get("b", 64)), ci(64), ci(kw.get("g", 32)), ci(kw.get("r", 1)), null)
    assert balance(src=null) == INVALID
    assert balance(dst=p) == INVALID            # in place
    assert balance(g=0) == INVALID
    assert balance(r=3) == INVALID              # rows must divide the block
    assert balance(b=64, r=2, g=64) == INVALID  # granule must divide a row range
    assert balance(e=2000) == UNSUPPORTED
    assert balance(n=0) == OK

    def copy(**kw):
        return lib.sarathi_stream_copy(kw.get("dst", q), kw.get("src", p), i64(kw.get("n", 64)),
                                       ci(kw.get("kib", 8)), null)
    assert copy(n=24) == INVALID                # not a multiple of 16 bytes
    assert copy(dst=vp(q.value + 4)) == INVALID # unaligned
    assert copy(kib=5) == UNSUPPORTED           # no such launch shape
    assert copy(n=0) == OK


def test_rider_entry_points_validate_arguments_without_gpu(lib):
    """sarathi_moe_plan_riders and sarathi_moe_grouped_gemm_riders reject what the rider kernel does
    not cover (other block sizes, packed weights, fp32) before anything is launched."""
    i64, ci, vp = ctypes.c_int64, ctypes.c_int, ctypes.c_void_p
    buf = ctypes.create_string_buffer(256)
    p = ctypes.cast(buf, vp)
    null = vp(None)
    INVALID, UNSUPPORTED, OK = -1, -2, 0

    def plan(**kw):
        return lib.sarathi_moe_plan_riders(
            kw.get("ids", p), p, p, i64(kw.get("valid", 4)), i64(kw.get("len", 512)),
            ci(kw.get("bm", 256)), kw.get("out", p), i64(kw.get("out_len", 2)), null)
    assert plan(ids=null) == INVALID
    assert plan(out=null) == INVALID
    assert plan(out_len=1) == INVALID           # one entry per slot block
    assert plan(valid=-1) == INVALID
    assert plan(bm=128) == UNSUPPORTED
    assert plan(len=0, out_len=0) == OK

    def gemm(**kw):
        return lib.sarathi_moe_grouped_gemm_riders(
            kw.get("a", p), p, p, p, p, p, p, i64(kw.get("valid", 4)), i64(256),
            i64(64), i64(64), i64(64), i64(64 * 128), i64(64), ci(kw.get("bm", 256)), ci(2),
            ci(0), ci(kw.get("layout", 0)), ci(kw.get("dt", 2)), kw.get("riders", p), null)
    assert gemm(riders=null) == INVALID
    assert gemm(a=null) == INVALID
    assert gemm(bm=128) == UNSUPPORTED
    assert gemm(layout=1) == UNSUPPORTED
    assert gemm(dt=0) == UNSUPPORTED
    assert gemm(valid=0) == OK


def test_plan_blocks_validates_arguments_without_gpu(lib):
    i64, ci, vp = ctypes.c_int64, ctypes.c_int, ctypes.c_void_p
    buf = ctypes.create_string_buffer(256)
    p = ctypes.cast(buf, vp)
    q = vp(p.value + 128)
    null = vp(None)
    INVALID, UNSUPPORTED, OK = -1, -2, 0

    def plan(**kw):
        return lib.sarathi_moe_plan_blocks(
            kw.get("src", p), kw.get("dst", q), p, p, i64(kw.get("len", 512)), ci(kw.get("e", 8)),
            ci(kw.get("bm", 256)), ci(4), kw.get("riders", p), i64(kw.get("riders_len", 2)), null)
    assert plan(src=null) == INVALID
    assert plan(dst=p) == INVALID               # in place
    assert plan(riders=null) == INVALID
    assert plan(riders_len=1) == INVALID        # one entry per slot block
    assert plan(e=0) == INVALID
    assert plan(bm=64) == UNSUPPORTED
    assert plan(e=2000) == UNSUPPORTED
    assert plan(len=0, riders_len=0) == OK
