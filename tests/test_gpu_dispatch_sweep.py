"""GPU: seeded sweeps over the shapes at which the launch shapes of the row-wise ops change.

rms_norm, fused_add_rms_norm and rotary_embedding (alone and fused with the cache append) choose
among several kernel shapes by row width, head counts and rows per compute unit.  The fixed cases
of the other test files sit on the boundaries known when they were written; these sweeps draw head
counts, widths, dtypes and token counts around every multiple of the compute-unit count that a
rule could use, so that a rule added later is exercised on both sides without a test of its own.
Each case goes through the op namespace -> C ABI and is compared with the oracle (rotary: bit for
bit; norms: the dtype tolerance of the dense-op tests) or, for the fused append, bit for bit with
the two stand-alone ops.  The activations, whose only rule is whole vectors or not, get a smaller
sweep over widths, strides and dtypes, and the grouped GEMM one over expert loads, for the per-expert
choice between riders and the even fill of its slot blocks.
"""
import os
import random

import pytest
import torch

from helpers import THETA_LLAMA3, assert_close_dtype, cos_sin_cache, gen, hybrid_positions, randn
from oracle import c_oracle

pytestmark = pytest.mark.gpu

# A longer sweep on request: SARATHI_SWEEP_SCALE multiplies the number of cases of every sweep,
# SARATHI_SWEEP_OFFSET shifts all seeds.
_SCALE = int(os.environ.get("SARATHI_SWEEP_SCALE", "1"))
_OFFSET = int(os.environ.get("SARATHI_SWEEP_OFFSET", "0"))


def _units():
    return torch.cuda.get_device_properties(0).multi_processor_count


def _token_counts(rng, n, waves_per_token=(1,), top=6000):
    """Token counts within one of a multiple of the compute-unit count divided by the number of
    waves a token may be dealt to, plus a few small and unremarkable ones."""
    units = _units()
    out = []
    while len(out) < n:
        if rng.random() < 0.2:
            t = rng.choice([1, 2, 63, 300, 777, 1500, 3333])
        else:
            k = rng.choice([3, 4, 5, 8, 9, 10, 10.25, 12, 16, 24])
            t = int(k * units / rng.choice(waves_per_token)) + rng.choice([-1, 0, 1])
        if 1 <= t <= top:
            out.append(t)
    return out


def _rope_bits_equal(got, want):
    assert torch.equal(got, want)
    if got.dtype == torch.float32:
        assert torch.equal(got.view(torch.int32), want.view(torch.int32))
        return
    nz = want != 0   # the bf16 vector path stores +0 where the reference's arithmetic yields -0
    assert torch.equal(got.view(torch.int16)[nz], want.view(torch.int16)[nz])


ROPE_CASES = 48 * _SCALE


@pytest.mark.parametrize("case", range(ROPE_CASES))
def test_rotary_embedding_sweep_bit_exact(ops, dev, case):
    rng = random.Random(1000 + case + _OFFSET)
    nq = rng.choice([1, 3, 8, 9, 16, 20, 24, 28, 32, 40, 48, 56, 64, 71])
    nkv = rng.choice([1, 2, 4, 8, nq]) if rng.random() < 0.8 else rng.randint(1, nq)
    nkv = min(nkv, nq)
    D = rng.choice([128, 128, 128, 64, 64, 256, 32])
    dtype = rng.choice([torch.bfloat16, torch.bfloat16, torch.float16, torch.float32])
    is_neox = rng.random() < 0.75
    T = _token_counts(rng, 1, waves_per_token=(1, 1, 2, 3, 4), top=5200)[0]
    packed = rng.random() < 0.6
    g = gen(case)
    table = cos_sin_cache(8192, D, THETA_LLAMA3, dtype)
    pos = hybrid_positions(T, min((T * 8) // 9, 4000), g)
    if packed:
        qkv = randn((T, (nq + 2 * nkv) * D), g, dtype)
        want = qkv.clone()
        wq, wk, _ = want.split([nq * D, nkv * D, nkv * D], dim=-1)
        c_oracle.rotary_embedding(pos, wq, wk, D, table, is_neox)
        got = qkv.to(dev)
        gq, gk, _ = got.split([nq * D, nkv * D, nkv * D], dim=-1)
        ops.pos_encoding_ops.rotary_embedding(pos.to(dev), gq, gk, D, table.to(dev), is_neox)
        _rope_bits_equal(got.cpu(), want)
    else:
        q, k = randn((T, nq * D), g, dtype), randn((T, nkv * D), g, dtype)
        wq, wk = q.clone(), k.clone()
        c_oracle.rotary_embedding(pos, wq, wk, D, table, is_neox)
        gq, gk = q.to(dev), k.to(dev)
        ops.pos_encoding_ops.rotary_embedding(pos.to(dev), gq, gk, D, table.to(dev), is_neox)
        _rope_bits_equal(gq.cpu(), wq)
        _rope_bits_equal(gk.cpu(), wk)


APPEND_CASES = 32 * _SCALE


@pytest.mark.parametrize("case", range(APPEND_CASES))
def test_fused_rope_append_sweep_equals_separate_ops(ops, dev, case):
    rng = random.Random(2000 + case + _OFFSET)
    nq = rng.choice([8, 9, 16, 24, 28, 32, 40, 48, 56, 64, 71])
    nkv = min(nq, rng.choice([1, 2, 4, 8, 8, nq]))
    D = rng.choice([128, 128, 64])
    is_neox = rng.random() < 0.75
    write_key = rng.random() < 0.5
    T = _token_counts(rng, 1, waves_per_token=(1, 1, 2, 3, 4), top=4500)[0]
    n = max(1, T - rng.choice([0, 0, 1, 50]))     # appended rows; the rest are rotated in place only
    page_size = 16
    g = gen(3000 + case)
    pages = (n + page_size - 1) // page_size
    table_pages = torch.randperm(pages + 3, generator=g)[:pages].to(torch.int32).to(dev)
    indptr = torch.tensor([0, pages], dtype=torch.int32, device=dev)
    b = torch.zeros(n, dtype=torch.int32, device=dev)
    pos = torch.arange(n, dtype=torch.int32, device=dev)
    positions = torch.randint(0, 4096, (T,), generator=g, dtype=torch.int64).to(dev)
    table = cos_sin_cache(4096, D, 10000.0, torch.bfloat16).to(dev)
    qkv = randn((T, (nq + 2 * nkv) * D), g, torch.bfloat16).to(dev)
    cache = randn((pages + 3, 2, page_size, nkv, D), g, torch.bfloat16).to(dev)

    ref, want_cache = qkv.clone(), cache.clone()
    rq, rk, rv = ref.split([nq * D, nkv * D, nkv * D], dim=-1)
    ops.pos_encoding_ops.rotary_embedding(positions, rq, rk, D, table, is_neox)
    ops.kv_cache_ops.append_paged_kv_cache(rk[:n].reshape(n, nkv, D), rv[:n].reshape(n, nkv, D), b,
                                           pos, want_cache, table_pages, indptr)
    got, got_cache = qkv.clone(), cache.clone()
    q, k, v = got.split([nq * D, nkv * D, nkv * D], dim=-1)
    ops.kv_cache_ops.rotary_embedding_append_paged_kv(
        positions, q, k, v, D, table, is_neox, b, pos, got_cache, table_pages, indptr,
        num_append_tokens=n, write_key=write_key)
    assert torch.equal(got_cache, want_cache)
    assert torch.equal(q, rq) and torch.equal(v, rv) and torch.equal(k[n:], rk[n:])
    if write_key:
        assert torch.equal(k[:n], rk[:n])
    else:
        assert torch.equal(k[:n], qkv.split([nq * D, nkv * D, nkv * D], dim=-1)[1][:n])


NORM_CASES = 48 * _SCALE


@pytest.mark.parametrize("case", range(NORM_CASES))
def test_rms_norm_and_fused_sweep_match_oracle(ops, dev, case):
    rng = random.Random(4000 + case + _OFFSET)
    dtype = rng.choice([torch.bfloat16, torch.bfloat16, torch.float16, torch.float32])
    per_vec = 4 if dtype == torch.float32 else 8
    if rng.random() < 0.7:     # whole vectors: widths around every vector count a rule may use
        nvec = rng.choice([64, 128, 129, 256, 257, 384, 512, 513, 568, 640, 641, 768, 769, 896,
                           1024, 1025, 2048]) + rng.choice([0, 0, 0, -1])
        H = max(1, nvec) * per_vec
    else:                      # widths that are not whole vectors: the element-wise path
        H = rng.choice([100, 1000, 4100, 5001])
    top = 4400 if H * (4 if dtype == torch.float32 else 2) <= 16384 else 1200
    T = _token_counts(rng, 1, top=top)[0]
    g = gen(5000 + case)
    x, r = randn((T, H), g, dtype), randn((T, H), g, dtype)
    w = randn((H,), g, dtype, mean=1.0, std=0.1)
    if dtype == torch.float32:
        tol = dict(atol=2e-6, rtol=2e-5, max_ulps=None, max_mismatch_frac=1.0)
    else:
        tol = dict(atol=1e-2, rtol=1e-2, max_ulps=2, max_mismatch_frac=5e-3)
    pad = per_vec * rng.choice([0, 1, 8])        # row stride = width + pad
    want = torch.empty_like(x)
    c_oracle.rms_norm(want, x, w, 1e-5)
    in_buf = torch.zeros((T, H + pad), dtype=dtype, device=dev)
    out_buf = torch.zeros((T, H + 2 * pad), dtype=dtype, device=dev)
    in_buf[:, :H].copy_(x)
    ops.layernorm_ops.rms_norm(out_buf[:, :H], in_buf[:, :H], w.to(dev), 1e-5)
    assert_close_dtype(out_buf[:, :H], want, **tol)
    assert bool((out_buf[:, H:] == 0).all())

    wx, wr = x.clone(), r.clone()
    c_oracle.fused_add_rms_norm(wx, wr, w, 1e-5)
    gx_buf = torch.zeros((T, H + pad), dtype=dtype, device=dev)
    gr_buf = torch.zeros((T, H + 2 * pad), dtype=dtype, device=dev)
    gx, gr = gx_buf[:, :H], gr_buf[:, :H]
    gx.copy_(x)
    gr.copy_(r)
    ops.layernorm_ops.fused_add_rms_norm(gx, gr, w.to(dev), 1e-5)
    assert torch.equal(gr.cpu(), wr), "residual = T(x + r) must be bit-exact"
    assert_close_dtype(gx, wx, **tol)
    assert bool((gx_buf[:, H:] == 0).all()) and bool((gr_buf[:, H:] == 0).all())


ACT_CASES = 30 * _SCALE


@pytest.mark.parametrize("case", range(ACT_CASES))
def test_activation_sweep_matches_oracle(ops, dev, case):
    """silu_and_mul (row views with strides of their own) and gelu_new / gelu_fast over widths that
    are and are not whole 16-byte vectors or whole 1 KiB segments."""
    rng = random.Random(6000 + case + _OFFSET)
    dtype = rng.choice([torch.bfloat16, torch.bfloat16, torch.float16, torch.float32])
    per_vec = 4 if dtype == torch.float32 else 8
    d = rng.choice([1, 3, per_vec, 5 * per_vec, 64 * per_vec, 64 * per_vec + per_vec, 1000, 3584,
                    4095, 11008, 14336])
    T = rng.choice([1, 2, 37, 300, 1025, 2304]) if d > 4096 else _token_counts(rng, 1, top=3000)[0]
    g = gen(7000 + case)
    if dtype == torch.float32:
        tol = dict(atol=2e-6, rtol=2e-5, max_ulps=None, max_mismatch_frac=1.0)
    else:
        tol = dict(atol=1e-2, rtol=1e-2, max_ulps=2, max_mismatch_frac=5e-3)
    x = randn((T, 2 * d), g, dtype, std=2.0)
    want = torch.empty((T, d), dtype=dtype)
    c_oracle.silu_and_mul(want, x)
    pad = per_vec * rng.choice([0, 0, 2])
    in_buf = torch.zeros((T, 2 * d + pad), dtype=dtype, device=dev)
    out_buf = torch.zeros((T, d + 2 * pad), dtype=dtype, device=dev)
    in_buf[:, :2 * d].copy_(x)
    ops.activation_ops.silu_and_mul(out_buf[:, :d], in_buf[:, :2 * d])
    assert_close_dtype(out_buf[:, :d], want, **tol)
    assert bool((out_buf[:, d:] == 0).all())

    name = rng.choice(["gelu_new", "gelu_fast"])
    xg = x[:, :d].contiguous()
    wantg = torch.empty_like(xg)
    getattr(c_oracle, name)(wantg, xg)
    gotg = torch.empty_like(xg, device=dev)
    getattr(ops.activation_ops, name)(gotg, xg.to(dev))
    tol["max_mismatch_frac"] = max(tol["max_mismatch_frac"], 2e-2)
    assert_close_dtype(gotg, wantg, **tol)


PLAN_CASES = 24 * _SCALE


@pytest.mark.parametrize("case", range(PLAN_CASES))
def test_planned_blocks_sweep_same_bits_as_plain_gemm(ops, dev, case):
    """The grouped GEMM at 256-slot blocks with its blocks planned per expert (riders or the even
    fill) against the same GEMM on moe_align_block_size's own layout, bit for bit: expert counts,
    top-k, skewed and uniform expert loads, ragged N, all three epilogues, both 16-bit dtypes."""
    rng = random.Random(8000 + case + _OFFSET)
    E = rng.choice([2, 4, 8, 16, 24])
    k = rng.choice([kk for kk in (1, 2, 4) if kk <= E])
    per_expert = rng.choice([90, 200, 256, 257, 290, 400, 520, 545, 800, 1030, 1300])
    T = max(1, per_expert * E // k + rng.randint(-7, 7))
    N = 8 * rng.randint(32, 140)
    K = 64 * rng.randint(1, 6)
    dtype = rng.choice([torch.bfloat16, torch.float16])
    mul, silu = rng.choice([(False, False), (True, False), (False, True)])
    g = gen(9000 + case)
    logits = torch.randn((T, E), generator=g, dtype=torch.float32)
    if rng.random() < 0.5:                       # some experts hot, some nearly idle
        logits += torch.randn((E,), generator=g) * rng.choice([0.3, 1.0])
    weights, ids = torch.topk(torch.softmax(logits, dim=-1), k, dim=-1)
    ids = ids.to(torch.int32).to(dev)
    wd = weights.contiguous().to(dev)
    bm = 256
    n_sorted = T * k + E * (bm - 1)
    sd = torch.empty((n_sorted,), dtype=torch.int32, device=dev)
    ed = torch.zeros(((n_sorted + bm - 1) // bm,), dtype=torch.int32, device=dev)
    pd = torch.empty((1,), dtype=torch.int32, device=dev)
    ops.moe_ops.moe_align_block_size_filled(ids, E, bm, sd, ed, pd)
    planned = torch.empty_like(sd)
    riders = torch.empty((ed.numel(),), dtype=torch.int32, device=dev)
    ops.moe_ops.moe_plan_blocks(sd, planned, ed, pd, E, bm, T * k, riders)
    # every slot is still there exactly once
    live = int(pd.item())
    kept = planned[:live][planned[:live] < T * k]
    assert torch.equal(torch.sort(kept).values, torch.arange(T * k, dtype=torch.int32, device=dev))
    A = randn((T, K), g, dtype, std=0.5).to(dev)
    Bw = randn((E, N, K), g, dtype, std=0.5).to(dev)
    cols = N // 2 if silu else N
    base = torch.full((T, k, cols), 7.0, dtype=dtype, device=dev)
    got = torch.full((T, k, cols), -3.0, dtype=dtype, device=dev)
    ops.moe_ops.moe_grouped_gemm(A, Bw, base, wd, sd, ed, pd, T * k, bm, k, mul, False, N, silu)
    ops.moe_ops.moe_grouped_gemm(A, Bw, got, wd, planned, ed, pd, T * k, bm, k, mul, False, N, silu, riders)
    assert torch.equal(got, base)
