"""GPU parity of the dense layer ops (rms_norm, fused_add_rms_norm, silu_and_mul, gelu_*,
rotary_embedding) against the CPU oracle on identical seeded inputs.

Every call goes through the shipped op namespaces, i.e. pybind front end -> C ABI -> HIP kernel.
Tolerance for 16-bit outputs: |got - want| <= 1e-2 + 1e-2 * |want| (atol = rtol = 1e-2); the
helper additionally requires every mismatch to be a single unit in the last place.  rotary_embedding
and the residual output of fused_add_rms_norm have no transcendental and must be bit-exact.
"""
import pytest
import torch

from helpers import (THETA_LLAMA3, assert_close_dtype, cos_sin_cache, gen, hybrid_positions, randn)
from oracle import c_oracle

pytestmark = pytest.mark.gpu

DTYPES = [torch.bfloat16, torch.float16, torch.float32]


def _tol(dtype):
    if dtype == torch.float32:
        # fp32 outputs show the reduction order and the last place of exp / rsqrt / tanh directly;
        # bound them far inside the stated 1e-2 instead of counting ulps
        return dict(atol=2e-6, rtol=2e-5, max_ulps=None, max_mismatch_frac=1.0)
    return dict(atol=1e-2, rtol=1e-2, max_ulps=2, max_mismatch_frac=5e-3)


# ---------------------------------------------------------------- rms_norm

@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("T,H", [(512, 4096), (37, 8192), (5, 1024), (3, 512), (7, 320), (2, 16384),
                                 (4, 100), (1, 8)])
def test_rms_norm_matches_oracle(ops, dev, dtype, T, H):
    g = gen(100 + H)
    x = randn((T, H), g, dtype)
    w = randn((H,), g, dtype, mean=1.0, std=0.1)
    want = torch.empty_like(x)
    c_oracle.rms_norm(want, x, w, 1e-5)
    got = torch.empty_like(x, device=dev)
    ops.layernorm_ops.rms_norm(got, x.to(dev), w.to(dev), 1e-5)
    assert_close_dtype(got, want, **_tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("T,H", [(512, 4096), (37, 8192), (5, 1024), (7, 320), (2, 16384), (4, 100)])
def test_fused_add_rms_norm_matches_oracle(ops, dev, dtype, T, H):
    # (512, 4096) bf16 is the benchmark's CPU-path configuration
    g = gen(0)
    x = randn((T, H), g, dtype)
    r = randn((T, H), g, dtype)
    w = randn((H,), g, dtype, mean=1.0, std=0.1)
    wx, wr = x.clone(), r.clone()
    c_oracle.fused_add_rms_norm(wx, wr, w, 1e-5)
    gx, gr = x.to(dev), r.to(dev)
    ops.layernorm_ops.fused_add_rms_norm(gx, gr, w.to(dev), 1e-5)
    assert torch.equal(gr.cpu(), wr), "residual = T(x + r) must be bit-exact"
    assert_close_dtype(gx, wx, **_tol(dtype))


@pytest.mark.parametrize("T,H,dtype", [
    (1100, 5120, torch.bfloat16), (1024, 4544, torch.bfloat16), (1500, 6144, torch.float16),
    (1300, 7168, torch.bfloat16), (2048, 8192, torch.bfloat16), (2049, 8192, torch.bfloat16),
    (1100, 4104, torch.float16), (1200, 3000, torch.float32), (1200, 4096, torch.float32),
    (3072, 5120, torch.bfloat16), (3073, 5120, torch.bfloat16), (4096, 5120, torch.bfloat16),
    (4097, 5120, torch.bfloat16), (3073, 8192, torch.float16)])
def test_rms_norm_long_rows_one_wave_per_row(ops, dev, T, H, dtype):
    """Rows of 513..1024 sixteen-byte vectors from four rows per compute unit on: one wave per
    row with 10, 12, 14 or 16 vectors per lane (whole and ragged widths), for both ops, up to the
    row counts where each hands over to the multi-wave shapes (one row below and above).  Same
    results as the oracle through views whose row stride differs from the width."""
    g = gen(T + H)
    x, r = randn((T, H), g, dtype), randn((T, H), g, dtype)
    w = randn((H,), g, dtype, mean=1.0, std=0.1)
    pad = 64
    # plain norm
    want = torch.empty_like(x)
    c_oracle.rms_norm(want, x, w, 1e-5)
    in_buf = torch.zeros((T, H + pad), dtype=dtype, device=dev)
    out_buf = torch.zeros((T, H + 2 * pad), dtype=dtype, device=dev)
    in_buf[:, :H].copy_(x)
    ops.layernorm_ops.rms_norm(out_buf[:, :H], in_buf[:, :H], w.to(dev), 1e-5)
    assert_close_dtype(out_buf[:, :H], want, **_tol(dtype))
    assert bool((out_buf[:, H:] == 0).all())
    # fused op
    wx, wr = x.clone(), r.clone()
    c_oracle.fused_add_rms_norm(wx, wr, w, 1e-5)
    gx_buf = torch.zeros((T, H + pad), dtype=dtype, device=dev)
    gr_buf = torch.zeros((T, H + 8), dtype=dtype, device=dev)
    gx, gr = gx_buf[:, :H], gr_buf[:, :H]
    gx.copy_(x)
    gr.copy_(r)
    ops.layernorm_ops.fused_add_rms_norm(gx, gr, w.to(dev), 1e-5)
    assert torch.equal(gr.cpu(), wr), "residual = T(x + r) must be bit-exact"
    assert_close_dtype(gx, wx, **_tol(dtype))
    assert bool((gx_buf[:, H:] == 0).all()) and bool((gr_buf[:, H:] == 0).all())


@pytest.mark.parametrize("T,H,dtype", [
    (2304, 4096, torch.bfloat16), (2305, 4096, torch.bfloat16), (1030, 4096, torch.bfloat16),
    (2304, 3072, torch.bfloat16), (1537, 2560, torch.bfloat16), (2248, 2048, torch.bfloat16),
    (1500, 4096, torch.float16), (1500, 2048, torch.float32), (1100, 1032, torch.float32),
    (3072, 4096, torch.bfloat16), (3073, 4096, torch.bfloat16), (4096, 4096, torch.bfloat16),
    (4099, 3072, torch.float16), (6144, 2048, torch.bfloat16), (6145, 2048, torch.bfloat16),
    (40960, 4096, torch.bfloat16), (40963, 4096, torch.bfloat16), (43008, 3072, torch.float16)])
def test_fused_add_rms_norm_rows_per_workgroup(ops, dev, T, H, dtype):
    """The launch shapes of the fused op on rows of up to 512 vectors: one wave per row with the
    stores held back (more than 1024 rows, up to 6144 rows of at most 256 vectors or 40960 longer
    ones: whole and ragged widths, both vector counts per lane, all dtypes), one workgroup per row
    for more short rows, and two or three rows per one-wave workgroup for more long ones (40963 ->
    2, 43008 -> 3, with ragged last workgroups).  Same results as the oracle over every row,
    through views whose row stride differs from the width."""
    g = gen(T + H)
    x, r = randn((T, H), g, dtype), randn((T, H), g, dtype)
    w = randn((H,), g, dtype, mean=1.0, std=0.1)
    wx, wr = x.clone(), r.clone()
    c_oracle.fused_add_rms_norm(wx, wr, w, 1e-5)
    # views into wider buffers: the row stride differs from the width
    gx_buf = torch.zeros((T, H + 64), dtype=x.dtype, device=dev)
    gr_buf = torch.zeros((T, H + 8), dtype=x.dtype, device=dev)
    gx, gr = gx_buf[:, :H], gr_buf[:, :H]
    gx.copy_(x)
    gr.copy_(r)
    ops.layernorm_ops.fused_add_rms_norm(gx, gr, w.to(dev), 1e-5)
    assert torch.equal(gr.cpu(), wr), "residual = T(x + r) must be bit-exact"
    assert_close_dtype(gx, wx, **_tol(dtype))
    assert bool((gx_buf[:, H:] == 0).all()) and bool((gr_buf[:, H:] == 0).all())


def test_fused_add_equals_add_then_norm(ops, dev):
    """fused(x, r) == (r' = x + r in bf16; rms_norm(r')) using the library's own rms_norm: the
    fusion changes traffic, not arithmetic.  The residual is bit-exact; the normed output may
    differ in a rare last place because the two kernels split a row over lanes differently and
    therefore add the squares in a different order."""
    g = gen(3)
    T, H = 2304, 4096
    x, r = randn((T, H), g).to(dev), randn((T, H), g).to(dev)
    w = randn((H,), g, mean=1.0, std=0.1).to(dev)
    z = r + x
    want = torch.empty_like(z)
    ops.layernorm_ops.rms_norm(want, z, w, 1e-5)
    ops.layernorm_ops.fused_add_rms_norm(x, r, w, 1e-5)
    assert torch.equal(r, z)
    assert_close_dtype(x, want, max_mismatch_frac=1e-4)


def test_rms_norm_row_strides(ops, dev):
    """Rows may be views with a row stride larger than the width."""
    g = gen(4)
    big = randn((64, 3 * 1024), g).to(dev)
    x = big[:, 1024:2048]
    w = randn((1024,), g, mean=1.0, std=0.1).to(dev)
    out_big = torch.zeros((64, 2048), dtype=torch.bfloat16, device=dev)
    out = out_big[:, :1024]
    ops.layernorm_ops.rms_norm(out, x, w, 1e-6)
    want = torch.empty((64, 1024), dtype=torch.bfloat16)
    c_oracle.rms_norm(want, x.cpu().contiguous(), w.cpu(), 1e-6)
    assert_close_dtype(out.contiguous(), want)
    assert bool((out_big[:, 1024:] == 0).all())


def test_rms_norm_full_size_properties(ops, dev):
    """Llama-3-70B shape [4608, 8192]: scale invariance in the input (x -> 2x leaves the output
    unchanged up to eps), and rows are independent (a permutation of rows permutes the output)."""
    g = gen(5)
    T, H = 4608, 8192
    x = randn((T, H), g).to(dev)
    w = randn((H,), g, mean=1.0, std=0.1).to(dev)
    a, b = torch.empty_like(x), torch.empty_like(x)
    ops.layernorm_ops.rms_norm(a, x, w, 0.0)
    ops.layernorm_ops.rms_norm(b, x * 2, w, 0.0)        # exact doubling in bf16
    assert torch.equal(a, b)
    perm = torch.randperm(T, generator=g).to(dev)
    c = torch.empty_like(x)
    ops.layernorm_ops.rms_norm(c, x[perm].contiguous(), w, 0.0)
    assert torch.equal(c, a[perm])


# -------------------------------------------------------------- activation

@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("T,d", [(64, 14336), (9, 4096), (5, 1000), (3, 7), (1, 8)])
def test_silu_and_mul_matches_oracle(ops, dev, dtype, T, d):
    g = gen(2)
    x = randn((T, 2 * d), g, dtype, std=2.0)
    want = torch.empty((T, d), dtype=dtype)
    c_oracle.silu_and_mul(want, x)
    got = torch.empty((T, d), dtype=dtype, device=dev)
    ops.activation_ops.silu_and_mul(got, x.to(dev))
    assert_close_dtype(got, want, **_tol(dtype))


def test_silu_and_mul_special_values(ops, dev):
    xs = torch.tensor([0.0, -0.0, 1.0, -1.0, 30.0, -30.0, 100.0, -100.0, 1e4, -1e4,
                       float("inf"), 1e-3, -1e-3, 88.0, -88.0, -104.0], dtype=torch.float32)
    x = torch.cat((xs, torch.ones_like(xs))).bfloat16().reshape(1, -1)
    want = torch.empty((1, xs.numel()), dtype=torch.bfloat16)
    c_oracle.silu_and_mul(want, x)
    got = torch.empty_like(want, device=dev)
    ops.activation_ops.silu_and_mul(got, x.to(dev))
    assert_close_dtype(got, want, max_mismatch_frac=1.0)


def test_silu_and_mul_full_size_properties(ops, dev):
    """Llama-3-8B MLP shape [2304, 2*14336]: y = 1 reduces the op to silu (library routine), and
    the op is odd-linear in y: f(x, -y) = -f(x, y) exactly."""
    g = gen(6)
    T, d = 2304, 14336
    x = randn((T, 2 * d), g).to(dev)
    out = torch.empty((T, d), dtype=torch.bfloat16, device=dev)
    ops.activation_ops.silu_and_mul(out, x)
    neg = x.clone()
    neg[:, d:] = -neg[:, d:]
    out2 = torch.empty_like(out)
    ops.activation_ops.silu_and_mul(out2, neg)
    assert torch.equal(out2, -out)
    ones = x.clone()
    ones[:, d:] = 1.0
    ops.activation_ops.silu_and_mul(out2, ones)
    ref = torch.nn.functional.silu(x[:, :d].float()).bfloat16()
    assert_close_dtype(out2, ref, max_mismatch_frac=5e-3)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["gelu_new", "gelu_fast"])
@pytest.mark.parametrize("T,d", [(33, 4096), (5, 1001), (1, 3)])
def test_gelu_matches_oracle(ops, dev, dtype, name, T, d):
    g = gen(7)
    x = randn((T, d), g, dtype, std=2.0)
    want = torch.empty_like(x)
    getattr(c_oracle, name)(want, x)
    got = torch.empty_like(x, device=dev)
    getattr(ops.activation_ops, name)(got, x.to(dev))
    # the chains of dtype roundings amplify a last-place difference in tanh by up to 2 ulp
    tol = _tol(dtype)
    tol["max_mismatch_frac"] = max(tol["max_mismatch_frac"], 2e-2)
    assert_close_dtype(got, want, **tol)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["gelu_new", "gelu_fast"])
def test_gelu_saturation_and_non_finite_inputs(ops, dev, dtype, name):
    """The tanh inside is 1 - 2 / (1 + e^{2u}) with no clamp: it must saturate to +-1 through an
    infinite or zero exponential, and NaN / infinities must come out as the arithmetic of the
    reference's expression gives them (0.5 * -inf * (1 + -1) is NaN, for one)."""
    vals = [0.0, -0.0, 0.5, -0.5, 3.0, -3.0, 9.0, -9.0, 20.0, -20.0, 100.0, -100.0, 1e4, -1e4,
            float("inf"), float("-inf"), float("nan")]
    x = torch.tensor(vals * 8, dtype=torch.float32).to(dtype).reshape(1, -1)   # 136 = 17 vectors
    want = torch.empty_like(x)
    getattr(c_oracle, name)(want, x)
    got = torch.empty_like(x, device=dev)
    getattr(ops.activation_ops, name)(got, x.to(dev))
    got = got.cpu()
    assert torch.equal(torch.isnan(got), torch.isnan(want))
    sat = ~torch.isnan(want) & ((x.float().abs() >= 20.0) | (x.float() == 0.0))
    assert torch.equal(got[sat], want[sat])   # saturated values, infinities and signed zeros: exact
    mid = ~torch.isnan(want) & ~sat
    assert_close_dtype(got[mid].reshape(1, -1), want[mid].reshape(1, -1), **_tol(dtype))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("name", ["gelu_new", "gelu_fast"])
def test_gelu_table_path_every_bit_pattern_same_bits_as_arithmetic_path(ops, dev, dtype, name):
    """From 12 Mi elements on, 16-bit tensors go through the 65536-entry table in LDS.  A tensor that
    holds every bit pattern 256 times (shuffled) plus a ragged tail of 5 elements takes that path; the
    same values in chunks below the threshold take the arithmetic kernel.  Both must give the same
    bits for every pattern, NaNs, infinities, subnormals and signed zeros included; a sample of the
    finite values is also checked against the oracle."""
    op = getattr(ops.activation_ops, name)
    g = gen(11)
    pats = torch.arange(65536, dtype=torch.int32).repeat(256)
    pats = pats[torch.randperm(pats.numel(), generator=g)]
    pats = torch.cat([pats, torch.tensor([0x3f80, 0xbf80, 0x0001, 0x7fc0, 0x4000], dtype=torch.int32)])
    x = pats.to(torch.int16).view(dtype).reshape(1, -1).to(dev)            # [1, 2^24 + 5]
    assert x.numel() == (1 << 24) + 5
    got = torch.full_like(x, 7.0)
    op(got, x)                                                               # table path
    want = torch.full_like(x, 9.0)
    chunk = 1 << 20
    for lo in range(0, x.numel(), chunk):                                    # arithmetic path
        hi = min(lo + chunk, x.numel())
        piece = torch.empty((1, hi - lo), dtype=dtype, device=dev)
        op(piece, x[:, lo:hi].contiguous())
        want[:, lo:hi] = piece
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))
    # a second call (table complete by now, or still behind its build on this stream) and a call
    # on another stream give the same bits
    again = torch.empty_like(x)
    op(again, x)
    assert torch.equal(again.view(torch.int16), got.view(torch.int16))
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        other = torch.empty_like(x)
        op(other, x)
    side.synchronize()
    assert torch.equal(other.view(torch.int16), got.view(torch.int16))
    xs = x[:, :4096].cpu()
    ref = torch.empty_like(xs)
    getattr(c_oracle, name)(ref, xs)
    fin = torch.isfinite(ref.float()) & torch.isfinite(xs.float())
    tol = _tol(dtype)
    tol["max_mismatch_frac"] = max(tol["max_mismatch_frac"], 2e-2)
    assert_close_dtype(got[:, :4096].cpu()[fin].reshape(1, -1), ref[fin].reshape(1, -1), **tol)


@pytest.mark.parametrize("name", ["gelu_new", "gelu_fast"])
def test_gelu_table_path_full_size_matches_oracle(ops, dev, name):
    """[2304, 14336] bf16 (the table path) against the oracle on sampled rows."""
    g = gen(12)
    x = randn((2304, 14336), g, torch.bfloat16, std=1.5)
    got = torch.empty_like(x, device=dev)
    getattr(ops.activation_ops, name)(got, x.to(dev))
    rows = torch.randperm(2304, generator=g)[:48]
    xs = x[rows].contiguous()
    want = torch.empty_like(xs)
    getattr(c_oracle, name)(want, xs)
    tol = _tol(torch.bfloat16)
    tol["max_mismatch_frac"] = max(tol["max_mismatch_frac"], 2e-2)
    assert_close_dtype(got.cpu()[rows], want, **tol)


def test_gelu_table_path_replayed_in_a_hip_graph(ops, dev):
    """A large gelu captured into a HIP graph (the table is complete by then: one eager call and a
    synchronisation first) and replayed on changing inputs gives the eager result every time."""
    g = gen(13)
    n = 1 << 24
    x = randn((1, n), g, torch.bfloat16).to(dev)
    eager = torch.empty_like(x)
    ops.activation_ops.gelu_new(eager, x)
    torch.cuda.synchronize()
    out = torch.empty_like(x)
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            ops.activation_ops.gelu_new(out, x)
    for rep in range(3):
        x.copy_(randn((1, n), g, torch.bfloat16))
        out.fill_(3.0)
        ops.activation_ops.gelu_new(eager, x)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out.view(torch.int16), eager.view(torch.int16)), rep


# ------------------------------------------------------------------ rotary

def _rope_case(ops, dev, dtype, T, nq, nkv, D, R, is_neox, packed, seed=1, prefill=None):
    g = gen(seed)
    cache = cos_sin_cache(8192, R, THETA_LLAMA3, dtype)
    # prefill positions start at 4096 and the table has 8192 rows
    pos = hybrid_positions(T, prefill if prefill is not None else min((T * 8) // 9, 4096), g)
    assert int(pos.max()) < cache.shape[0]
    if packed:
        qkv = randn((T, (nq + 2 * nkv) * D), g, dtype)
        want = qkv.clone()
        wq, wk, _ = want.split([nq * D, nkv * D, nkv * D], dim=-1)
        c_oracle.rotary_embedding(pos, wq, wk, D, cache, is_neox)
        got = qkv.to(dev)
        gq, gk, _ = got.split([nq * D, nkv * D, nkv * D], dim=-1)
        ops.pos_encoding_ops.rotary_embedding(pos.to(dev), gq, gk, D, cache.to(dev), is_neox)
        return got.cpu(), want
    q, k = randn((T, nq * D), g, dtype), randn((T, nkv * D), g, dtype)
    wq, wk = q.clone(), k.clone()
    c_oracle.rotary_embedding(pos, wq, wk, D, cache, is_neox)
    gq, gk = q.to(dev), k.to(dev)
    ops.pos_encoding_ops.rotary_embedding(pos.to(dev), gq, gk, D, cache.to(dev), is_neox)
    return torch.cat((gq.cpu(), gk.cpu()), -1), torch.cat((wq, wk), -1)

def _assert_rope_bits(got, want):
    """Bit for bit wherever the expected value is non-zero (compared as integers, so NaN payloads
    and signs count), by value where it is exactly zero: the bf16 vector path stores +0 where the
    reference's arithmetic yields -0."""
    assert torch.equal(got, want)
    if got.dtype == torch.float32:
        assert torch.equal(got.view(torch.int32), want.view(torch.int32))
        return
    nz = want != 0
    assert torch.equal(got.view(torch.int16)[nz], want.view(torch.int16)[nz])



@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("is_neox", [True, False])
@pytest.mark.parametrize("packed", [False, True])
def test_rope_llama3_8b_hybrid_batch_bit_exact(ops, dev, dtype, is_neox, packed):
    """The benchmark configuration: T = 2304 = 2048 prefill + 256 decode, 32 q / 8 kv heads of 128."""
    got, want = _rope_case(ops, dev, dtype, 2304, 32, 8, 128, 128, is_neox, packed, prefill=2048)
    _assert_rope_bits(got, want)


@pytest.mark.parametrize("is_neox", [True, False])
@pytest.mark.parametrize("T,nq,nkv,D,R", [
    (4608 // 8, 64, 8, 128, 128),   # Llama-3-70B head counts
    (17, 4, 4, 64, 64),
    (9, 8, 2, 128, 64),             # partial rotary: elements >= rot_dim untouched
    (5, 3, 1, 96, 32),
    (3, 2, 2, 80, 20),              # rot_dim/2 not a multiple of the vector width -> element path
    (1, 1, 1, 256, 256),
    (11, 160, 8, 128, 128),         # more heads than one pass of the block covers
    (1700, 20, 4, 128, 128),        # one wave per token: 3 NeoX segments / 6 of interleaved pairs
    (1700, 28, 8, 128, 128),        # 5 / 9 segments
    (1600, 44, 4, 128, 128),        # 6 NeoX segments (one wave per segment) / 12
    (700, 32, 32, 128, 128),        # a token dealt to two waves: 2 x 4 NeoX segments / 2 x 8
    (600, 64, 8, 128, 128),         # 3 x 3 / 2 x 9
    (560, 28, 24, 128, 128),        # 7 as 4 + 3 (the last segment of the second wave is empty) / 2 x 7
    (520, 40, 40, 128, 128),        # 2 x 5 / 2 x 10
    (5000, 8, 1, 128, 128),         # two segments: one wave per token at every batch size
])
def test_rope_shapes_bit_exact(ops, dev, T, nq, nkv, D, R, is_neox):
    for packed in (False, True):
        got, want = _rope_case(ops, dev, torch.bfloat16, T, nq, nkv, D, R, is_neox, packed, seed=T)
        _assert_rope_bits(got, want)


@pytest.mark.parametrize("dtype,D", [(torch.bfloat16, 64), (torch.float16, 64), (torch.float32, 32)])
@pytest.mark.parametrize("T,nq,nkv", [
    (37, 71, 1),       # Falcon-7B: 71 query heads and one key head, one wave per segment
    (1700, 71, 1),     # six segments: still one wave per segment
    (1700, 40, 8),     # three segments: one wave per token
    (1500, 9, 9),      # nine heads in segments of sixteen, one wave per token
    (300, 128, 8),     # Falcon-40B
    (2304, 16, 16),    # whole segments only
])
def test_rope_neox_heads_of_128_bytes_bit_exact(ops, dev, dtype, D, T, nq, nkv):
    """NeoX heads of 128 bytes (head_size 64 in a 16-bit type, 32 in float32), fully rotated: the
    kernels read them in memory order, eight lanes per head, and lanes trade registers before and
    after the rotation.  Same bits as the oracle, contiguous and packed qkv."""
    for packed in (False, True):
        got, want = _rope_case(ops, dev, dtype, T, nq, nkv, D, D, True, packed, seed=T + nq)
        _assert_rope_bits(got, want)


@pytest.mark.parametrize("T", [1279, 1280, 2624, 2625])
def test_rope_launch_shape_boundaries_bit_exact(ops, dev, T):
    """Either side of the token counts at which the launch switches between one wave per segment and
    one wave per token (5 and 10.25 waves per compute unit on a 256-unit device), at the Llama-3-8B
    head counts, packed qkv."""
    got, want = _rope_case(ops, dev, torch.bfloat16, T, 32, 8, 128, 128, True, True, seed=T)
    _assert_rope_bits(got, want)


@pytest.mark.parametrize("is_neox", [True, False])
def test_rope_bf16_subnormal_range_and_signed_zeros(ops, dev, is_neox):
    """The bf16 vector path forms each sum of two rounded products with the packed dot-product
    instruction, which truncates its fp32 result instead of rounding it to nearest; that cannot
    change the result once it is rounded to bf16.  Checked where it would show first: inputs
    around 2^-121, so that many products and sums are subnormal.  Every non-zero output matches
    the oracle bit for bit; an exactly zero output matches in value (the instruction returns +0
    where the reference's subtraction returns -0)."""
    g = gen(77)
    T, nq, nkv, D = 64, 32, 8, 128
    cache = cos_sin_cache(8192, D, THETA_LLAMA3, torch.bfloat16)
    pos = hybrid_positions(T, 32, g)
    q = (randn((T, nq * D), g, torch.float32) * 2.0 ** -121).to(torch.bfloat16)
    k = (randn((T, nkv * D), g, torch.float32) * 2.0 ** -121).to(torch.bfloat16)
    q[:, ::7] = 0.0
    k[:, ::5] = -0.0
    k[:, 1::5] = -0.0
    wq, wk = q.clone(), k.clone()
    c_oracle.rotary_embedding(pos, wq, wk, D, cache, is_neox)
    gq, gk = q.to(dev), k.to(dev)
    ops.pos_encoding_ops.rotary_embedding(pos.to(dev), gq, gk, D, cache.to(dev), is_neox)
    subnormal = 0
    for got, want in ((gq.cpu(), wq), (gk.cpu(), wk)):
        assert torch.equal(got, want)                       # by value: -0 == +0
        nz = want != 0
        assert torch.equal(got.view(torch.int16)[nz], want.view(torch.int16)[nz])
        subnormal += int(((want.float().abs() < 2.0 ** -126) & nz).sum())
    assert subnormal > 1000, "inputs were meant to reach the subnormal range"


def test_rope_position_zero_is_identity_and_norm_preserved(ops, dev):
    g = gen(8)
    T, nq, nkv, D = 256, 32, 8, 128
    cache = cos_sin_cache(8192, D, THETA_LLAMA3, torch.float32)
    q, k = randn((T, nq * D), g, torch.float32), randn((T, nkv * D), g, torch.float32)
    gq, gk = q.to(dev), k.to(dev)
    ops.pos_encoding_ops.rotary_embedding(torch.zeros(T, dtype=torch.int64, device=dev), gq, gk, D,
                                          cache.to(dev), True)
    assert torch.equal(gq.cpu(), q) and torch.equal(gk.cpu(), k)     # cos = 1, sin = 0
    pos = hybrid_positions(T, 128, g)
    ops.pos_encoding_ops.rotary_embedding(pos.to(dev), gq, gk, D, cache.to(dev), True)
    n0 = q.view(T, nq, 2, D // 2).pow(2).sum(2)
    n1 = gq.cpu().view(T, nq, 2, D // 2).pow(2).sum(2)
    assert torch.allclose(n0, n1, rtol=1e-5, atol=1e-6)              # rotations keep |(x, y)|


def test_empty_batch_is_a_no_op_everywhere(ops, dev):
    """Zero tokens: every op returns without touching anything (empty tensors own no memory, so
    the C ABI sees null data pointers); the slot sort still reports zero padded tokens."""
    bf = torch.bfloat16
    e = lambda *shape, dt=bf: torch.empty(shape, dtype=dt, device=dev)  # noqa: E731
    w = torch.ones(64, dtype=bf, device=dev)
    ops.layernorm_ops.rms_norm(e(0, 64), e(0, 64), w, 1e-5)
    ops.layernorm_ops.fused_add_rms_norm(e(0, 64), e(0, 64), w, 1e-5)
    ops.activation_ops.silu_and_mul(e(0, 32), e(0, 64))
    ops.activation_ops.gelu_new(e(0, 64), e(0, 64))
    ops.activation_ops.gelu_fast(e(0, 64), e(0, 64))
    table = torch.zeros((16, 32), dtype=bf, device=dev)
    ops.pos_encoding_ops.rotary_embedding(e(0, dt=torch.int64), e(0, 128), e(0, 64), 32, table, True)
    i32 = torch.int32
    ops.moe_ops.topk_softmax(e(0, 2, dt=torch.float32), e(0, 2, dt=i32), e(0, 2, dt=i32),
                             e(0, 8, dt=torch.float32))
    post = torch.full((1,), -1, dtype=i32, device=dev)
    ops.moe_ops.moe_align_block_size(e(0, 2, dt=i32), 8, 1, e(0, dt=i32), e(0, dt=i32), post)
    assert int(post.item()) == 0
    post.fill_(-1)
    sorted_ids = torch.full((8 * 15,), -7, dtype=i32, device=dev)
    ops.moe_ops.fused_topk_align(e(0, 2, dt=torch.float32), e(0, 2, dt=i32), e(0, 2, dt=i32),
                                 e(0, 8, dt=torch.float32), True, 16, sorted_ids,
                                 e(8, dt=i32), post, False)
    assert int(post.item()) == 0 and bool((sorted_ids == -7).all())
    cache = torch.zeros((4, 2, 16, 2, 32), dtype=bf, device=dev)
    ops.kv_cache_ops.append_paged_kv_cache(e(0, 2, 32), e(0, 2, 32), e(0, dt=i32), e(0, dt=i32), cache,
                                           e(0, dt=i32), torch.zeros(1, dtype=i32, device=dev))
    assert not bool(cache.any())
    torch.cuda.synchronize()
