"""The drop-in boundary itself on the GPU: libsarathi_ops_hip.so driven through ctypes with
device pointers and a stream handle, no torch binding in between (the stub a non-torch host writes;
the reference's side of this boundary is csrc/layernorm.cpp:9-14, csrc/activation.cpp:15-19,
csrc/pos_encoding.cpp:11-16, csrc/moe.cpp:19-28), checked against the CPU oracle.  A second part
installs the four one-line shim modules under the reference's package name and calls the ops as
the reference's layers do (`from sarathi import layernorm_ops`)."""
import sys

import pytest
import torch

import abi_ctypes as abi
from helpers import assert_close_dtype, cos_sin_cache, gen, hybrid_positions, randn, THETA_LLAMA3
from oracle import c_oracle

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def lib():
    return abi.load()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_rms_norm_and_fused_add_through_the_c_abi(lib, dev, dtype):
    g = gen(100)
    T, H = 300, 4096
    x, r = randn((T, H), g, dtype), randn((T, H), g, dtype)
    w = randn((H,), g, dtype, mean=1.0, std=0.1)
    want = torch.empty_like(x)
    c_oracle.rms_norm(want, x, w, 1e-5)
    xd, wd = x.to(dev), w.to(dev)
    out = torch.empty_like(xd)
    abi.check(lib, lib.sarathi_rms_norm(abi.ptr(out), abi.ptr(xd), abi.ptr(wd), 1e-5, T, H, H, H,
                                        abi.DT[dtype], abi.stream()))
    torch.cuda.synchronize()
    if dtype == torch.float32:
        torch.testing.assert_close(out.cpu(), want, atol=2e-6, rtol=2e-5)
    else:
        assert_close_dtype(out, want)

    wx, wr = x.clone(), r.clone()
    c_oracle.fused_add_rms_norm(wx, wr, w, 1e-5)
    gx, gr = x.to(dev), r.to(dev)
    abi.check(lib, lib.sarathi_fused_add_rms_norm(abi.ptr(gx), abi.ptr(gr), abi.ptr(wd), 1e-5, T, H,
                                                  H, H, abi.DT[dtype], abi.stream()))
    torch.cuda.synchronize()
    assert torch.equal(gr.cpu(), wr)  # the sum rounds once: bit-exact
    if dtype == torch.float32:
        torch.testing.assert_close(gx.cpu(), wx, atol=2e-6, rtol=2e-5)
    else:
        assert_close_dtype(gx, wx)


def test_silu_and_mul_and_moe_sum_through_the_c_abi(lib, dev):
    g = gen(101)
    T, d = 257, 14336
    x = randn((T, 2 * d), g)
    want = torch.empty((T, d), dtype=x.dtype)
    c_oracle.silu_and_mul(want, x)
    xd = x.to(dev)
    out = torch.empty((T, d), dtype=x.dtype, device=dev)
    abi.check(lib, lib.sarathi_silu_and_mul(abi.ptr(out), abi.ptr(xd), T, d, 2 * d, d,
                                            abi.DT[x.dtype], abi.stream()))
    torch.cuda.synchronize()
    assert_close_dtype(out, want)

    k, H = 2, 4096
    y = randn((T, k, H), g)
    yd = y.to(dev)
    acc = torch.empty((T, H), dtype=y.dtype, device=dev)
    abi.check(lib, lib.sarathi_moe_sum(abi.ptr(acc), abi.ptr(yd), T, k, H, k * H, H, H,
                                       abi.DT[y.dtype], abi.stream()))
    torch.cuda.synchronize()
    # fp32 accumulation in ascending j, one rounding: exact for two addends
    assert torch.equal(acc.cpu(), (y[:, 0].float() + y[:, 1].float()).to(y.dtype))


@pytest.mark.parametrize("is_neox", [True, False])
def test_rotary_embedding_through_the_c_abi_bit_exact(lib, dev, is_neox):
    """q and k are views of a packed qkv buffer (row stride 6144), as models/llama.py:176 makes."""
    g = gen(102)
    T, nq, nkv, D = 515, 32, 8, 128
    pos = hybrid_positions(T, 400, g)
    cache = cos_sin_cache(8192, D, THETA_LLAMA3, torch.bfloat16)
    qkv = randn((T, (nq + 2 * nkv) * D), g)
    want = qkv.clone()
    c_oracle.rotary_embedding(pos, want[:, : nq * D], want[:, nq * D:(nq + nkv) * D], D, cache,
                              is_neox)
    got = qkv.to(dev)
    q, k = got[:, : nq * D], got[:, nq * D:(nq + nkv) * D]
    pd, cd = pos.to(dev), cache.to(dev)
    abi.check(lib, lib.sarathi_rotary_embedding(
        abi.ptr(pd), abi.ptr(q), abi.ptr(k), abi.ptr(cd), T, nq, nkv, D, D, q.stride(0),
        k.stride(0), int(is_neox), abi.DT[qkv.dtype], abi.stream()))
    torch.cuda.synchronize()
    assert torch.equal(got.cpu().view(torch.int16), want.view(torch.int16))  # v part included


@pytest.mark.parametrize("T,E,k", [(4096, 8, 2), (333, 64, 6), (100, 60, 4)])
def test_topk_softmax_through_the_c_abi(lib, dev, T, E, k):
    g = gen(103 + E)
    gating = torch.randn((T, E), generator=g, dtype=torch.float32)
    ww = torch.empty((T, k), dtype=torch.float32)
    wi = torch.empty((T, k), dtype=torch.int32)
    ws = torch.empty((T, k), dtype=torch.int32)
    c_oracle.topk_softmax(ww, wi, ws, gating)
    gd = gating.to(dev)
    gw = torch.empty((T, k), dtype=torch.float32, device=dev)
    gi = torch.empty((T, k), dtype=torch.int32, device=dev)
    gs = torch.empty((T, k), dtype=torch.int32, device=dev)
    abi.check(lib, lib.sarathi_topk_softmax(abi.ptr(gw), abi.ptr(gi), abi.ptr(gs), abi.ptr(gd), T,
                                            E, k, 0, abi.stream()))
    torch.cuda.synchronize()
    assert torch.equal(gi.cpu(), wi) and torch.equal(gs.cpu(), ws)
    torch.testing.assert_close(gw.cpu(), ww, atol=1e-6, rtol=0)


@pytest.mark.parametrize("numel,E,B", [(8192, 8, 64), (50_000, 8, 64), (20_000, 300, 16), (20_000, 200, 16)])
@pytest.mark.parametrize("with_workspace", [False, True])
def test_moe_align_block_size_through_the_c_abi(lib, dev, numel, E, B, with_workspace):
    g = gen(104 + numel)
    ids = torch.randint(0, E, (numel,), generator=g, dtype=torch.int32)
    ws_, we, wp = abi.align_buffers(numel, E, B, "cpu")
    c_oracle.moe_align_block_size(ids, E, B, ws_, we, wp)
    idd = ids.to(dev)
    s, e, p = abi.align_buffers(numel, E, B, dev)
    need = lib.sarathi_moe_align_workspace_bytes(numel, E) if with_workspace else 0
    # scratch is of use above 32 768 ids, or above 16 384 with more than 256 experts
    assert (need > 0) == (with_workspace and (numel > 32768 or (numel > 16384 and E > 256)))
    scratch = torch.empty((need,), dtype=torch.uint8, device=dev) if need else None
    abi.check(lib, lib.sarathi_moe_align_block_size(
        abi.ptr(idd), abi.ID_DT[ids.dtype], numel, E, B, abi.ptr(s), s.numel(), abi.ptr(e),
        e.numel(), abi.ptr(p), 0, abi.ptr(scratch), need, abi.stream()))
    torch.cuda.synchronize()
    assert torch.equal(p.cpu(), wp) and torch.equal(s.cpu(), ws_)
    nblk = int(wp.item()) // B
    assert torch.equal(e.cpu()[:nblk], we[:nblk]) and bool((e.cpu()[nblk:] == -7).all())


def test_ops_under_the_reference_package_name(tmp_path, dev):
    """The four shim modules a maintainer adds to the reference's `sarathi/` package, installed in
    a scratch package of that name; the calls below are the reference layers' calls
    (layers/layernorm.py:33-39, layers/activation.py:22-23, layers/rotary_embedding.py:94-101,
    fused_moe.py:356-368, :192-203)."""
    pkg = tmp_path / "sarathi"
    pkg.mkdir()
    (pkg / "__init__.py").write_text("")
    for name in ("layernorm_ops", "activation_ops", "pos_encoding_ops", "moe_ops"):
        (pkg / (name + ".py")).write_text("from sarathi_amd.%s import *\n" % name)
    assert "sarathi" not in sys.modules
    sys.path.insert(0, str(tmp_path))
    try:
        from sarathi import activation_ops, layernorm_ops, moe_ops, pos_encoding_ops
        g = gen(105)
        x = randn((64, 4096), g)
        w = randn((4096,), g, mean=1.0, std=0.1)
        want = torch.empty_like(x)
        c_oracle.rms_norm(want, x, w, 1e-6)
        out = torch.empty_like(x, device=dev)
        layernorm_ops.rms_norm(out, x.to(dev), w.to(dev), 1e-6)
        assert_close_dtype(out, want)

        a = randn((64, 2 * 1024), g)
        want = torch.empty((64, 1024), dtype=a.dtype)
        c_oracle.silu_and_mul(want, a)
        out = torch.empty((64, 1024), dtype=a.dtype, device=dev)
        activation_ops.silu_and_mul(out, a.to(dev))
        assert_close_dtype(out, want)

        pos = torch.arange(64, dtype=torch.int64)
        cache = cos_sin_cache(128, 128, 10000.0, torch.bfloat16)
        q, k = randn((64, 4 * 128), g), randn((64, 128), g)
        wq, wk = q.clone(), k.clone()
        c_oracle.rotary_embedding(pos, wq, wk, 128, cache, True)
        gq, gk = q.to(dev), k.to(dev)
        pos_encoding_ops.rotary_embedding(pos.to(dev), gq, gk, 128, cache.to(dev), True)
        assert torch.equal(gq.cpu(), wq) and torch.equal(gk.cpu(), wk)

        gating = torch.randn((64, 8), generator=g, dtype=torch.float32)
        tw = torch.empty((64, 2), dtype=torch.float32, device=dev)
        ti = torch.empty((64, 2), dtype=torch.int32, device=dev)
        ts = torch.empty((64, 2), dtype=torch.int32, device=dev)
        moe_ops.topk_softmax(tw, ti, ts, gating.to(dev))
        ww, wi, wsrc = (torch.empty((64, 2), dtype=d) for d in (torch.float32, torch.int32, torch.int32))
        c_oracle.topk_softmax(ww, wi, wsrc, gating)
        assert torch.equal(ti.cpu(), wi) and torch.equal(ts.cpu(), wsrc)
        s, e, p = abi.align_buffers(128, 8, 16, dev)
        moe_ops.moe_align_block_size(ti, 8, 16, s, e, p)
        ws_, we, wp = abi.align_buffers(128, 8, 16, "cpu")
        c_oracle.moe_align_block_size(wi, 8, 16, ws_, we, wp)
        assert torch.equal(s.cpu(), ws_) and torch.equal(p.cpu(), wp)
    finally:
        sys.path.remove(str(tmp_path))
        for m in [m for m in sys.modules if m == "sarathi" or m.startswith("sarathi.")]:
            del sys.modules[m]


@pytest.mark.parametrize("nbytes", [16, 1024 + 48, 24 * 1024, 3 * 36 * 1024 + 16, 18874368])
def test_stream_copy_every_launch_shape_byte_exact(lib, dev, nbytes):
    """The copy that bench.py uses as the ceiling: every launch shape moves exactly `nbytes` bytes
    (sizes that end inside a wave's span, inside a vector row, and the 2304 x 4096 bf16 tensor) and
    touches nothing beyond them."""
    from sarathi_amd import stream_ops
    lib.sarathi_stream_copy.argtypes = [abi.vp, abi.vp, abi.i64, abi.ci, abi.vp]
    lib.sarathi_stream_copy.restype = abi.ci
    g = torch.Generator().manual_seed(nbytes)
    src = torch.randint(0, 256, (nbytes,), generator=g, dtype=torch.uint8).to(dev)
    for kib in stream_ops.COPY_SHAPES_KIB:
        buf = torch.full((nbytes + 4096,), 0xA5, dtype=torch.uint8, device=dev)
        abi.check(lib, lib.sarathi_stream_copy(abi.ptr(buf), abi.ptr(src), nbytes, kib, abi.stream()))
        torch.cuda.synchronize()
        assert torch.equal(buf[:nbytes], src), "copy differs at %d KiB per wave" % kib
        assert bool((buf[nbytes:] == 0xA5).all()), "bytes beyond the end were written"
    out = torch.empty_like(src)
    stream_ops.stream_copy(out, src, 24)       # through the torch front end
    assert torch.equal(out, src)
    assert lib.sarathi_stream_copy(abi.ptr(out), abi.ptr(src), nbytes, 5, abi.stream()) == -2
    assert lib.sarathi_stream_copy(abi.ptr(out), abi.ptr(src), 24, 8, abi.stream()) == -1
