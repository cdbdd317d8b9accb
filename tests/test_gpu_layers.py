"""GPU: the layer counterparts produce what the ops produce, with the reference's call shapes."""
import pytest
import torch

from helpers import assert_close_dtype, gen, hybrid_positions, randn
from oracle import c_oracle

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def L(ops):
    from sarathi_amd import layers
    return layers


def test_rmsnorm_layer_plain_and_fused(L, dev):
    g = gen(20)
    T, H = 96, 4096
    x, r = randn((T, H), g), randn((T, H), g)
    norm = L.RMSNorm(H, eps=1e-5).to(device=dev, dtype=torch.bfloat16)
    norm.weight.data.copy_(randn((H,), g, mean=1.0, std=0.1))
    w = norm.weight.data.cpu()
    want = torch.empty_like(x)
    c_oracle.rms_norm(want, x, w, 1e-5)
    xd = x.to(dev)
    out = norm(xd)
    assert torch.equal(xd.cpu(), x)                       # input untouched
    assert_close_dtype(out, want)
    wx, wr = x.clone(), r.clone()
    c_oracle.fused_add_rms_norm(wx, wr, w, 1e-5)
    gx, gr = norm(x.to(dev), r.to(dev))
    assert torch.equal(gr.cpu(), wr)
    assert_close_dtype(gx, wx)


def test_activation_layers(L, dev):
    g = gen(21)
    x = randn((40, 2 * 1536), g)
    want = torch.empty((40, 1536), dtype=torch.bfloat16)
    c_oracle.silu_and_mul(want, x)
    assert_close_dtype(L.SiluAndMul()(x.to(dev)), want)
    for name, cls in (("gelu_new", L.NewGELU), ("gelu_fast", L.FastGELU)):
        want = torch.empty_like(x)
        getattr(c_oracle, name)(want, x)
        assert_close_dtype(cls()(x.to(dev)), want, max_mismatch_frac=2e-2)


def test_rotary_layer_on_packed_qkv(L, dev):
    g = gen(22)
    T, nq, nkv, D = 200, 32, 8, 128
    rope = L.get_rope(D, D, 8192, 500000, True, None, device="cpu", dtype=torch.bfloat16)
    cache = rope.cos_sin_cache.clone()
    rope = rope.to(dev)
    pos = hybrid_positions(T, 160, g)
    qkv = randn((T, (nq + 2 * nkv) * D), g)
    want = qkv.clone()
    wq, wk, _ = want.split([nq * D, nkv * D, nkv * D], dim=-1)
    c_oracle.rotary_embedding(pos, wq, wk, D, cache, True)
    got = qkv.to(dev)
    q, k, v = got.split([nq * D, nkv * D, nkv * D], dim=-1)      # strided views, as models/llama.py:176
    rq, rk = rope(pos.to(dev), q, k)
    assert rq.data_ptr() == q.data_ptr() and rk.data_ptr() == k.data_ptr()   # in place
    assert torch.equal(got.cpu(), want)


def test_rotary_table_built_on_the_device_matches_the_host_table(L, dev):
    """The reference builds its table on the GPU; cos/sin there may differ from the host's in the
    last fp32 place, which can flip a bf16 rounding now and then, never more."""
    a = L.get_rope(128, 128, 8192, 500000, True, None, device=dev, dtype=torch.bfloat16).cos_sin_cache
    b = L.get_rope(128, 128, 8192, 500000, True, None, device="cpu", dtype=torch.bfloat16).cos_sin_cache
    assert a.device.type == "cuda"
    diff = (a.cpu().float() - b.float()).abs()
    assert diff.max().item() <= 2.0 ** -7            # one bf16 step at magnitude 1
    assert (diff > 0).float().mean().item() < 2e-2


def test_fused_topk_and_align_wrappers(L, dev):
    g = gen(3)
    M, E, k, B = 4096, 8, 2, 64
    gating = torch.randn((M, E), generator=g, dtype=torch.float32)
    hidden = torch.empty((M, 16), dtype=torch.bfloat16, device=dev)
    ww, wi, ws = torch.empty((M, k)), torch.empty((M, k), dtype=torch.int32), torch.empty((M, k), dtype=torch.int32)
    c_oracle.topk_softmax(ww, wi, ws, gating)
    w, ids = L.fused_topk(hidden, gating.to(dev), k, renormalize=False)
    assert torch.equal(ids.cpu(), wi) and torch.allclose(w.cpu(), ww, rtol=0, atol=1e-6)
    wr, ids2 = L.fused_topk(hidden, gating.to(dev).bfloat16().float().bfloat16(), k, renormalize=True)
    assert wr.dtype == torch.float32 and ids2.shape == (M, k)
    assert torch.allclose(wr.sum(-1).cpu(), torch.ones(M), atol=1e-6)
    s, e, p = L.moe_align_block_size(ids, B, E)
    n = M * k + E * (B - 1)
    sw = torch.full((n,), M * k, dtype=torch.int32)
    ew = torch.full(((n + B - 1) // B,), -1, dtype=torch.int32)
    pw = torch.zeros((1,), dtype=torch.int32)
    c_oracle.moe_align_block_size(wi, E, B, sw, ew, pw)
    nb = int(pw.item()) // B
    assert s.shape == sw.shape and e.shape == ew.shape
    assert torch.equal(s.cpu(), sw) and torch.equal(p.cpu(), pw) and torch.equal(e.cpu()[:nb], ew[:nb])
