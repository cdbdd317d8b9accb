"""GPU: more tokens than one grid dimension holds (65535).  The streaming kernels put the token
index in grid.y, spill whole multiples into grid.z and launch the ragged remainder separately with
shifted pointers; narrow rows keep the inputs small while every token still goes through those
paths.  Checked bit-exactly (or to the stated tolerance) against the oracle over all tokens."""
import numpy as np
import pytest
import torch

from helpers import assert_close_dtype, cos_sin_cache, gen, randn
from oracle import c_oracle, paged_kv

pytestmark = pytest.mark.gpu

T_BIG = 2 * 65535 + 41      # two full grid.z slices and a remainder


def test_silu_and_mul_and_gelu_beyond_one_grid_dimension(ops, dev):
    g = gen(1)
    x = randn((T_BIG, 32), g)
    want = torch.empty((T_BIG, 16), dtype=torch.bfloat16)
    c_oracle.silu_and_mul(want, x)
    got = torch.empty((T_BIG, 16), dtype=torch.bfloat16, device=dev)
    ops.activation_ops.silu_and_mul(got, x.to(dev))
    assert_close_dtype(got, want)
    want = torch.empty_like(x)
    c_oracle.gelu_new(want, x)
    got = torch.empty_like(x, device=dev)
    ops.activation_ops.gelu_new(got, x.to(dev))
    assert_close_dtype(got, want)


def test_norms_beyond_one_grid_dimension(ops, dev):
    g = gen(2)
    x, r = randn((T_BIG, 64), g), randn((T_BIG, 64), g)
    w = randn((64,), g, mean=1.0, std=0.1)
    wx, wr = x.clone(), r.clone()
    c_oracle.fused_add_rms_norm(wx, wr, w, 1e-5)
    gx, gr = x.to(dev), r.to(dev)
    ops.layernorm_ops.fused_add_rms_norm(gx, gr, w.to(dev), 1e-5)
    assert torch.equal(gr.cpu(), wr)
    assert_close_dtype(gx, wx)


@pytest.mark.parametrize("neox", [True, False])
def test_rotary_and_kv_append_beyond_one_grid_dimension(ops, dev, neox):
    """One request of T_BIG tokens appended in one call (page size 16), heads of 16 elements."""
    nq, nkv, D, page = 2, 1, 16, 16
    g = gen(3)
    table = cos_sin_cache(256, D, 10000.0, torch.bfloat16)
    pos = torch.randint(0, 256, (T_BIG,), generator=g, dtype=torch.int64)
    qkv = randn((T_BIG, (nq + 2 * nkv) * D), g)
    wq, wk, wv = (want := qkv.clone()).split([nq * D, nkv * D, nkv * D], dim=-1)
    c_oracle.rotary_embedding(pos, wq, wk, D, table, neox)
    # plain rotary
    gq, gk, _ = (got := qkv.to(dev)).split([nq * D, nkv * D, nkv * D], dim=-1)
    ops.pos_encoding_ops.rotary_embedding(pos.to(dev), gq, gk, D, table.to(dev), neox)
    assert torch.equal(got.cpu().view(torch.int16), want.view(torch.int16))
    # fused with the append, and the stand-alone append of the rotated keys
    pages = (T_BIG + page - 1) // page
    rng = np.random.default_rng(4)
    kv_indices = rng.permutation(pages).astype(np.int32)
    kv_indptr = np.array([0, pages], dtype=np.int32)
    b = np.zeros(T_BIG, dtype=np.int32)
    ap = np.arange(T_BIG, dtype=np.int32)
    bits = lambda t: t.contiguous().view(torch.int16).numpy()   # noqa: E731
    want_cache = np.zeros((pages, 2, page, nkv, D), dtype=np.int16)
    paged_kv.append_paged_kv_cache(bits(wk).reshape(T_BIG, nkv, D), bits(wv).reshape(T_BIG, nkv, D),
                                   b, ap, want_cache[:, 0], want_cache[:, 1], kv_indices, kv_indptr)
    t = lambda a: torch.from_numpy(a).to(dev)   # noqa: E731
    fq, fk, fv = (fused := qkv.to(dev)).split([nq * D, nkv * D, nkv * D], dim=-1)
    cache = torch.zeros((pages, 2, page, nkv, D), dtype=torch.bfloat16, device=dev)
    ops.kv_cache_ops.rotary_embedding_append_paged_kv(pos.to(dev), fq, fk, fv, D, table.to(dev), neox,
                                                      t(b), t(ap), cache, t(kv_indices), t(kv_indptr))
    assert np.array_equal(bits(cache.cpu()), want_cache)
    assert torch.equal(fq.cpu().view(torch.int16), wq.contiguous().view(torch.int16))
    cache2 = torch.zeros_like(cache)
    slots = ops.kv_cache_ops.get_kv_slot_mapping(t(b), t(ap), t(kv_indices), t(kv_indptr), page)
    ops.kv_cache_ops.append_paged_kv_cache(gk.reshape(T_BIG, nkv, D), fv.reshape(T_BIG, nkv, D), t(b),
                                           t(ap), cache2, t(kv_indices), t(kv_indptr),
                                           slot_mapping=slots)
    assert torch.equal(cache2, cache)
