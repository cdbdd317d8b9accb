"""Property-based tests (hypothesis): random shapes, strides and index patterns instead of a fixed
list of cases.  The CPU half exercises the oracle's invariants; the GPU half (marked ``gpu``)
compares the HIP ops with the oracle on the drawn inputs, bit-exact wherever the op is integer /
byte / index work or pure rounding-defined arithmetic."""
import os

import numpy as np
import pytest
import torch
from hypothesis import HealthCheck, given, settings
from hypothesis import strategies as st

from helpers import assert_close_dtype, cos_sin_cache, gen, randn
from oracle import c_oracle, paged_kv

# SARATHI_TEST_EXAMPLES scales the number of drawn cases for an occasional longer soak
_SCALE = max(1, int(os.environ.get("SARATHI_TEST_EXAMPLES", "1")))
# the default run draws the same cases every time (a fixed regression set); a soak draws fresh ones
_FIXED = "SARATHI_TEST_EXAMPLES" not in os.environ
CPU = settings(max_examples=60 * _SCALE, deadline=None, derandomize=_FIXED, database=None,
               suppress_health_check=list(HealthCheck))
GPU = settings(max_examples=40 * _SCALE, deadline=None, derandomize=_FIXED, database=None,
               suppress_health_check=list(HealthCheck))


def _align_oracle(ids, E, B):
    n = ids.numel() + E * (B - 1)
    s = torch.full((n,), ids.numel(), dtype=torch.int32)
    e = torch.full(((n + B - 1) // B,), -1, dtype=torch.int32)
    p = torch.zeros((1,), dtype=torch.int32)
    c_oracle.moe_align_block_size(ids, E, B, s, e, p)
    return s, e, p


@CPU
@given(E=st.integers(1, 64), B=st.sampled_from([1, 2, 4, 16, 64, 128]), n=st.integers(0, 400),
       seed=st.integers(0, 2 ** 31 - 1), skew=st.booleans())
def test_moe_align_oracle_invariants(E, B, n, seed, skew):
    """Every id appears exactly once, inside its expert's run, in ascending order (stable); runs are
    padded to multiples of B with the pad value; expert_ids names the run of every block."""
    g = gen(seed)
    hi = max(1, E // 4) if skew else E
    ids = torch.randint(0, hi, (n,), generator=g, dtype=torch.int32)
    s, e, p = _align_oracle(ids, E, B)
    total = int(p.item())
    counts = torch.bincount(ids.long(), minlength=E)
    padded = (counts + B - 1) // B * B
    assert total == int(padded.sum()) and total % B == 0
    at = 0
    for x in range(E):
        run = s[at:at + int(padded[x])]
        real = run[:int(counts[x])]
        assert torch.equal(real.long(), torch.nonzero(ids == x).flatten())
        assert bool((run[int(counts[x]):] == n).all())
        assert bool((e[at // B:(at + int(padded[x])) // B] == x).all())
        at += int(padded[x])


@CPU
@given(page_size=st.sampled_from([1, 2, 8, 16]), data=st.data())
def test_paged_kv_oracle_round_trip(page_size, data):
    R = data.draw(st.integers(1, 6))
    before = [data.draw(st.integers(0, 40)) for _ in range(R)]
    new = [data.draw(st.integers(0, 20)) for _ in range(R)]
    totals = [a + b for a, b in zip(before, new)]
    need = [(t + page_size - 1) // page_size for t in totals]
    rng = np.random.default_rng(data.draw(st.integers(0, 10 ** 6)))
    pages = sum(need) + 2
    kv_indices = rng.permutation(pages)[:sum(need)].astype(np.int32)
    kv_indptr = np.concatenate([[0], np.cumsum(need)]).astype(np.int32)
    last = np.array([(t % page_size) or page_size if t else 0 for t in totals], dtype=np.int32)
    indptr = np.concatenate([[0], np.cumsum(new)]).astype(np.int32)
    nnz = int(indptr[-1])
    seq_lens = paged_kv.get_seq_lens(kv_indptr, last, page_size)
    assert seq_lens.tolist() == totals
    b, pos = paged_kv.get_batch_indices_positions(indptr, seq_lens, nnz)
    k = rng.standard_normal((nnz, 1, 2)).astype(np.float32)
    cache = np.zeros((pages, 2, page_size, 1, 2), dtype=np.float32)
    paged_kv.append_paged_kv_cache(k, -k, b, pos, cache[:, 0], cache[:, 1], kv_indices, kv_indptr)
    for r in range(R):
        got = paged_kv.gather_sequence(cache[:, 0], kv_indices, kv_indptr, seq_lens, r)
        assert np.array_equal(got[before[r]:], k[indptr[r]:indptr[r + 1]])
        assert not got[:before[r]].any()
    assert int((cache[:, 0] != 0).any(axis=(-1, -2)).sum()) <= nnz


# ---- GPU ------------------------------------------------------------------------------------------

DTYPES = [torch.bfloat16, torch.float16, torch.float32]


def _tol(dt):
    """bf16 / fp16: the stated 1e-2 tolerance plus the 2-ulp bound; fp32: reduction order and the
    last place of the hardware exp / rsqrt show directly, so an absolute / relative bound."""
    if dt == torch.float32:
        return dict(atol=2e-6, rtol=2e-5, max_ulps=None, max_mismatch_frac=1.0)
    return {}


@pytest.mark.gpu
@GPU
@given(T=st.integers(1, 40), H=st.integers(1, 700), dt=st.sampled_from(DTYPES),
       pad=st.sampled_from([0, 0, 8, 3]), seed=st.integers(0, 10 ** 6))
def test_gpu_norms_any_shape(ops, dev, T, H, dt, pad, seed):
    g = gen(seed)
    full = randn((T, H + pad), g, dt)
    x = full[:, :H]                       # row stride H + pad: exercises strided and unaligned rows
    w = randn((H,), g, dt, mean=1.0, std=0.2)
    want = torch.empty((T, H), dtype=dt)
    c_oracle.rms_norm(want, x.contiguous(), w, 1e-5)
    xd = full.to(dev)[:, :H]
    got = torch.empty((T, H), dtype=dt, device=dev)
    ops.layernorm_ops.rms_norm(got, xd, w.to(dev), 1e-5)
    assert_close_dtype(got, want, **_tol(dt))
    r = randn((T, H), g, dt)
    wx, wr = x.contiguous().clone(), r.clone()
    c_oracle.fused_add_rms_norm(wx, wr, w, 1e-5)
    gx, gr = full.to(dev)[:, :H], r.to(dev)
    ops.layernorm_ops.fused_add_rms_norm(gx, gr, w.to(dev), 1e-5)
    assert torch.equal(gr.cpu(), wr)
    assert_close_dtype(gx, wx, **_tol(dt))


@pytest.mark.gpu
@GPU
@given(T=st.integers(1, 30), nq=st.integers(1, 6), nkv=st.integers(1, 3),
       half=st.sampled_from([1, 3, 4, 8, 16, 32, 64]), tail=st.sampled_from([0, 0, 2, 16]),
       neox=st.booleans(), dt=st.sampled_from(DTYPES), seed=st.integers(0, 10 ** 6))
def test_gpu_rotary_any_shape_bitwise(ops, dev, T, nq, nkv, half, tail, neox, dt, seed):
    rot, D = 2 * half, 2 * half + tail
    g = gen(seed)
    table = cos_sin_cache(64, rot, 10000.0, dt)
    pos = torch.randint(0, 64, (T,), generator=g, dtype=torch.int64)
    qkv = randn((T, (nq + 2 * nkv) * D), g, dt)
    wq, wk, _ = (want := qkv.clone()).split([nq * D, nkv * D, nkv * D], dim=-1)
    c_oracle.rotary_embedding(pos, wq, wk, D, table, neox)
    gq, gk, _ = (got := qkv.to(dev)).split([nq * D, nkv * D, nkv * D], dim=-1)
    ops.pos_encoding_ops.rotary_embedding(pos.to(dev), gq, gk, D, table.to(dev), neox)
    bits = torch.int16 if dt != torch.float32 else torch.int32
    assert torch.equal(got.cpu().view(bits), want.view(bits))


@pytest.mark.gpu
@GPU
@given(T=st.integers(1, 30), d=st.integers(1, 600), dt=st.sampled_from(DTYPES),
       seed=st.integers(0, 10 ** 6))
def test_gpu_activations_any_shape(ops, dev, T, d, dt, seed):
    g = gen(seed)
    x = randn((T, 2 * d), g, dt, std=2.0)
    want = torch.empty((T, d), dtype=dt)
    c_oracle.silu_and_mul(want, x)
    got = torch.empty((T, d), dtype=dt, device=dev)
    ops.activation_ops.silu_and_mul(got, x.to(dev))
    assert_close_dtype(got, want, **_tol(dt))
    for name in ("gelu_new", "gelu_fast"):
        want = torch.empty((T, 2 * d), dtype=dt)
        getattr(c_oracle, name)(want, x)
        got = torch.empty((T, 2 * d), dtype=dt, device=dev)
        getattr(ops.activation_ops, name)(got, x.to(dev))
        assert_close_dtype(got, want, **_tol(dt))


@pytest.mark.gpu
@GPU
@given(T=st.integers(0, 40), k=st.integers(1, 8), H=st.integers(1, 700), dt=st.sampled_from(DTYPES),
       pad_k=st.integers(0, 2), pad_h=st.sampled_from([0, 8, 24]), seed=st.integers(0, 10 ** 6))
def test_gpu_moe_sum_any_shape(ops, dev, T, k, H, dt, pad_k, pad_h, seed):
    """Any shape, dtype and input strides against the library sum: two addends bit for bit, more
    within one ulp of the dtype (the fp32 order of additions may differ)."""
    g = gen(seed)
    big = randn((T, k + pad_k, H + pad_h), g, dt, std=1.5)
    x = big[:, :k, :H]
    want = torch.sum(x, dim=1)
    got = torch.full((T, H), 5.0, dtype=dt, device=dev)
    ops.moe_ops.moe_sum(big.to(dev)[:, :k, :H], got)
    if k <= 2:
        assert torch.equal(got.cpu(), want)
    elif dt == torch.float32:
        torch.testing.assert_close(got.cpu(), want, atol=4e-6, rtol=4e-6)
    else:
        assert_close_dtype(got, want, max_ulps=1)


@pytest.mark.gpu
@GPU
@given(E=st.integers(1, 300), B=st.sampled_from([1, 4, 16, 64, 128]), n=st.integers(0, 3000),
       idt=st.sampled_from([torch.uint8, torch.int8, torch.int16, torch.int32, torch.int64]),
       seed=st.integers(0, 10 ** 6), skew=st.booleans(), fill=st.booleans())
def test_gpu_moe_align_any_input_bitwise(ops, dev, E, B, n, idt, seed, skew, fill):
    if idt == torch.uint8:
        E = min(E, 255)
    if idt == torch.int8:
        E = min(E, 127)
    g = gen(seed)
    hi = max(1, E // 5) if skew else E
    ids = torch.randint(0, hi, (n,), generator=g, dtype=torch.int64).to(idt)
    s, e, p = _align_oracle(ids, E, B)
    sg = torch.full_like(s, -3 if fill else n).to(dev)
    eg = torch.full_like(e, -1).to(dev)
    pg = torch.zeros((1,), dtype=torch.int32, device=dev)
    op = ops.moe_ops.moe_align_block_size_filled if fill else ops.moe_ops.moe_align_block_size
    op(ids.to(dev), E, B, sg, eg, pg)
    nb = int(p.item()) // B
    assert int(pg.item()) == int(p.item())
    assert torch.equal(sg.cpu(), s)
    assert torch.equal(eg.cpu()[:nb], e[:nb]) and bool((eg.cpu()[nb:] == -1).all())


@pytest.mark.gpu
@GPU
@given(E=st.integers(1, 200), k=st.integers(1, 8), T=st.integers(1, 70), renorm=st.booleans(),
       seed=st.integers(0, 10 ** 6))
def test_gpu_topk_softmax_any_expert_count(ops, dev, E, k, T, renorm, seed):
    k = min(k, E)
    gating = torch.randn((T, E), generator=gen(seed), dtype=torch.float32) * 3.0
    top = torch.sort(gating, dim=-1, descending=True).values[:, :k + 1]
    if top.shape[1] > 1 and (top[:, :-1] - top[:, 1:]).min().item() < 1e-5:
        return          # a near-tie: the winner depends on the last place of expf
    ww, wi, ws = (torch.empty((T, k)), torch.empty((T, k), dtype=torch.int32),
                  torch.empty((T, k), dtype=torch.int32))
    c_oracle.topk_softmax(ww, wi, ws, gating)
    if renorm:
        ww = ww / ww.sum(dim=-1, keepdim=True)
    gw, gi, gs = (torch.empty((T, k), device=dev), torch.empty((T, k), dtype=torch.int32, device=dev),
                  torch.empty((T, k), dtype=torch.int32, device=dev))
    (ops.moe_ops.topk_softmax_renorm if renorm else ops.moe_ops.topk_softmax)(gw, gi, gs,
                                                                             gating.to(dev))
    assert torch.equal(gi.cpu(), wi) and torch.equal(gs.cpu(), ws)
    assert torch.allclose(gw.cpu(), ww, rtol=1e-6, atol=1e-6)


@pytest.mark.gpu
@GPU
@given(page=st.sampled_from([1, 4, 16, 32]), nkv=st.integers(1, 4),
       D=st.sampled_from([8, 24, 64, 128, 6]), dt=st.sampled_from(DTYPES), neox=st.booleans(),
       write_key=st.booleans(), use_slots=st.booleans(), pad=st.integers(0, 3), data=st.data())
def test_gpu_kv_append_and_fusion_any_layout(ops, dev, page, nkv, D, dt, neox, write_key, use_slots,
                                             pad, data):
    """Stand-alone append against the numpy oracle (byte-exact); the rotary + append fusion against
    the two separate GPU ops (byte-exact on cache, query, key and value)."""
    R = data.draw(st.integers(1, 5))
    before = [data.draw(st.integers(0, 50)) for _ in range(R)]
    new = [data.draw(st.integers(0, 12)) for _ in range(R)]
    seed = data.draw(st.integers(0, 10 ** 6))
    totals = [a + b for a, b in zip(before, new)]
    need = [(t + page - 1) // page for t in totals]
    rng = np.random.default_rng(seed)
    pages = sum(need) + 1
    kv_indices = rng.permutation(pages)[:sum(need)].astype(np.int32)
    kv_indptr = np.concatenate([[0], np.cumsum(need)]).astype(np.int32)
    last = np.array([(t % page) or page if t else 0 for t in totals], dtype=np.int32)
    indptr = np.concatenate([[0], np.cumsum(new)]).astype(np.int32)
    n = int(indptr[-1])
    T = n + pad
    if T == 0:
        return
    nq = 2
    g = gen(seed)
    t = lambda a: torch.from_numpy(a).to(dev)  # noqa: E731
    seq_lens = ops.kv_cache_ops.get_seq_lens(t(kv_indptr), t(last), page)
    assert seq_lens.cpu().tolist() == totals
    b, ap = ops.kv_cache_ops.get_batch_indices_positions(t(indptr), seq_lens, n)
    wb, wap = paged_kv.get_batch_indices_positions(indptr, np.array(totals), n)
    assert b.cpu().tolist() == wb.tolist() and ap.cpu().tolist() == wap.tolist()
    slots = ops.kv_cache_ops.get_kv_slot_mapping(b, ap, t(kv_indices), t(kv_indptr), page) \
        if use_slots else None

    qkv = randn((T, (nq + 2 * nkv) * D), g, dt)
    cache0 = randn((pages, 2, page, nkv, D), g, dt)
    table = cos_sin_cache(64, D, 10000.0, dt).to(dev)
    pos = torch.randint(0, 64, (T,), generator=g, dtype=torch.int64).to(dev)
    split = [nq * D, nkv * D, nkv * D]
    bits = torch.int16 if dt != torch.float32 else torch.int32

    # separate ops: rotary in place, then append the first n rows
    sep = qkv.to(dev)
    sq, sk, sv = sep.split(split, dim=-1)
    ops.pos_encoding_ops.rotary_embedding(pos, sq, sk, D, table, neox)
    cache_sep = cache0.to(dev)
    ops.kv_cache_ops.append_paged_kv_cache(sk[:n], sv[:n], b, ap, cache_sep, t(kv_indices),
                                           t(kv_indptr), slot_mapping=slots)
    want = cache0.clone().view(bits).numpy()
    paged_kv.append_paged_kv_cache(sk[:n].cpu().contiguous().view(bits).numpy().reshape(n, nkv, D),
                                   sv[:n].cpu().contiguous().view(bits).numpy().reshape(n, nkv, D),
                                   wb, wap, want[:, 0], want[:, 1], kv_indices, kv_indptr)
    assert np.array_equal(cache_sep.cpu().view(bits).numpy(), want)

    fused = qkv.to(dev)
    fq, fk, fv = fused.split(split, dim=-1)
    cache_fused = cache0.to(dev)
    ops.kv_cache_ops.rotary_embedding_append_paged_kv(pos, fq, fk, fv, D, table, neox, b, ap,
                                                      cache_fused, t(kv_indices), t(kv_indptr),
                                                      num_append_tokens=n, write_key=write_key,
                                                      slot_mapping=slots)
    assert torch.equal(cache_fused.view(bits), cache_sep.view(bits))
    assert torch.equal(fq.contiguous().view(bits), sq.contiguous().view(bits))
    assert torch.equal(fv.contiguous().view(bits), sv.contiguous().view(bits))
    assert torch.equal(fk[n:].contiguous().view(bits), sk[n:].contiguous().view(bits))
    key_want = sk[:n] if write_key else qkv.to(dev).split(split, dim=-1)[1][:n]
    assert torch.equal(fk[:n].contiguous().view(bits), key_want.contiguous().view(bits))


@pytest.mark.gpu
@GPU
@given(T=st.integers(1, 300), E=st.sampled_from([1, 2, 4, 8, 16]), k=st.integers(1, 4),
       BM=st.sampled_from([32, 64, 128, 256]), n4=st.integers(1, 90), ksteps=st.integers(1, 5),
       epi=st.sampled_from(["plain", "weight", "silu"]), packed=st.booleans(),
       dt=st.sampled_from([torch.bfloat16, torch.float16]), seed=st.integers(0, 10 ** 6))
def test_gpu_grouped_gemm_any_shape(ops, dev, T, E, k, BM, n4, ksteps, epi, packed, dt, seed):
    from oracle import torch_formulations
    from sarathi_amd.layers import pack_expert_weights
    k = min(k, E)
    K = 64 * ksteps
    N = 4 * n4 * (2 if epi == "silu" else 1)
    if packed and epi == "silu" and (N // 2) % 32:
        N = 64 * ((N // 2 + 31) // 32)        # packed gate / up tiles must not straddle
    g = gen(seed)
    gating = torch.randn((T, E), generator=g, dtype=torch.float32)
    w = torch.empty((T, k))
    ids = torch.empty((T, k), dtype=torch.int32)
    src = torch.empty((T, k), dtype=torch.int32)
    c_oracle.topk_softmax(w, ids, src, gating)
    s, e, p = _align_oracle(ids, E, BM)
    A = randn((T, K), g, dt, std=0.5)
    B = randn((E, N, K), g, dt, std=0.5)
    full = torch.zeros((T, k, N), dtype=dt)
    torch_formulations.moe_grouped_gemm(A, B, full, w, s, e, p, T * k, BM, k, epi == "weight")
    if epi == "silu":
        want = torch.empty((T * k, N // 2), dtype=dt)
        torch_formulations.silu_and_mul(want, full.view(-1, N))
    else:
        want = full.view(T * k, N)
    got = torch.full(want.shape, 5.0, dtype=dt, device=dev)
    Bd = B.to(dev)
    ops.moe_ops.moe_grouped_gemm(A.to(dev), pack_expert_weights(Bd).data if packed else Bd, got,
                                 w.to(dev), s.to(dev), e.to(dev), p.to(dev), T * k, BM, k,
                                 epi == "weight", packed, N, epi == "silu")
    got, want = got.float().cpu(), want.float()
    tol = 2e-2 * want.abs().max().item() + 2e-2 * want.abs()
    assert bool(((got - want).abs() <= tol).all()), "max diff %.4g" % (got - want).abs().max().item()
