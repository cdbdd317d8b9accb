"""Seeded inputs of the benchmark configurations and comparison helpers shared by the tests.

Inputs are always drawn on the CPU in fp32 from a seeded generator and then cast, so the oracle
(CPU) and the HIP kernels (GPU copy of the same tensor) see identical bits.
"""
import torch

THETA_LLAMA3 = 500000.0


def gen(seed):
    return torch.Generator().manual_seed(seed)


def randn(shape, g, dtype=torch.bfloat16, mean=0.0, std=1.0):
    return (torch.randn(shape, generator=g, dtype=torch.float32) * std + mean).to(dtype)


def hybrid_positions(num_tokens, prefill_len, g, prefill_start=4096, max_pos=8192):
    """One prefill chunk at consecutive positions followed by decode tokens at random positions
    (prefill tokens come first in a hybrid batch: sarathi/model_executor/model_runner.py:76-104)."""
    pre = torch.arange(prefill_start, prefill_start + prefill_len, dtype=torch.int64)
    dec = torch.randint(1, max_pos, (num_tokens - prefill_len,), generator=g, dtype=torch.int64)
    return torch.cat((pre, dec))


def cos_sin_cache(max_pos, rot_dim, theta, dtype):
    """cos || sin table as sarathi/model_executor/layers/rotary_embedding.py:55-84 builds it,
    computed on the CPU in fp32 and cast to the model dtype."""
    inv_freq = 1.0 / (theta ** (torch.arange(0, rot_dim, 2, dtype=torch.float32) / rot_dim))
    t = torch.arange(max_pos, dtype=torch.float32)
    freqs = torch.outer(t, inv_freq)
    return torch.cat((freqs.cos(), freqs.sin()), dim=-1).to(dtype)


def ulp_of(t):
    """Spacing of the tensor's dtype at each element's magnitude (as float32).  Magnitudes below
    2^-100 are treated as 2^-100: differences down there are flush-to-zero effects of the hardware
    reciprocal, far below anything the stated tolerance can see."""
    mant = {torch.bfloat16: 7, torch.float16: 10, torch.float32: 23}[t.dtype]
    mag = t.float().abs().clamp_min(2.0 ** -100)
    return torch.exp2(torch.floor(torch.log2(mag)) - mant)


def assert_close_dtype(got, want, atol=1e-2, rtol=1e-2, max_ulps=2, max_mismatch_frac=5e-3):
    """The stated tolerance (|got-want| <= atol + rtol*|want|, i.e. torch.allclose semantics with
    atol = rtol = 1e-2) plus the much tighter bound the kernels actually meet: no element is off
    by more than `max_ulps` units in the last place of the dtype and only a small fraction is off
    at all.  Ops that round twice (rms_norm, silu_and_mul) can turn a one-ulp flip of the
    intermediate into two ulps of the result, hence the default of 2.  Non-finite values must
    match exactly.  max_ulps=None skips the ulp bound (fp32 outputs, where reduction order and
    the transcendental's last place show directly)."""
    got, want = got.cpu(), want.cpu()
    assert got.shape == want.shape and got.dtype == want.dtype
    g, w = got.float(), want.float()
    fin = torch.isfinite(w)
    assert torch.equal(torch.isfinite(g), fin), "non-finite positions differ"
    assert torch.equal(g[~fin].nan_to_num(nan=7.0), w[~fin].nan_to_num(nan=7.0))
    g, w = g[fin], w[fin]
    diff = (g - w).abs()
    if diff.numel() == 0:
        return 0.0
    assert bool((diff <= atol + rtol * w.abs()).all()), (
        "outside tolerance: max abs %.4g" % diff.max().item())
    bad = diff > 0
    frac = bad.float().mean().item()
    if bad.any() and max_ulps is not None:
        ulp = torch.maximum(ulp_of(got), ulp_of(want))[fin]
        ulps = (diff / ulp)[bad].max().item()
        assert ulps <= max_ulps + 1e-3, "max error %.2f ulp" % ulps
    # the fraction is a statistical bound: for n elements that each flip with probability
    # max_mismatch_frac, allow the mean count plus four standard deviations plus two
    n = diff.numel()
    allowed = max_mismatch_frac * n + 4.0 * (max_mismatch_frac * n) ** 0.5 + 2.0
    assert int(bad.sum()) <= allowed, "mismatching fraction %.3g (%d of %d)" % (frac, int(bad.sum()), n)
    return frac
