"""Pins the CPU oracle (oracle/sarathi_ops_oracle.c) without a GPU.

The reference ships no tests and only two known-answer vectors for this path (both for
moe_align_block_size; tests/golden/moe_align_block_size_vectors.json).  Everything else is pinned
by what the mathematics fixes:

  * an exact-arithmetic evaluation (python Fractions, a generic "round to p significant bits,
    ties to even" written independently of the C bit tricks) on tiny inputs, including the
    intermediate roundings to the tensor dtype that the reference's scalar_t arithmetic performs;
  * special cases with closed forms, reductions to library routines (F.silu, F.gelu, softmax +
    sort, transformers' rotate_half formulation), invariants (rotation = complex multiplication,
    GPT-J == NeoX on de-interleaved data, permutation/stability properties of the sort);
  * the independently written tensor-level formulations in oracle/torch_formulations.py.

Each "discriminates" assertion shows that the inputs used would expose the plausible mistake
named in it (a dropped rounding, a missing epsilon, a flipped sign): the mutated formula gives a
different answer on them.
"""
import json
import math
import os
from fractions import Fraction

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from helpers import THETA_LLAMA3, cos_sin_cache, gen, hybrid_positions, randn, ulp_of
from oracle import c_oracle, torch_formulations

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden",
                      "moe_align_block_size_vectors.json")

MANT_BITS = {torch.bfloat16: 8, torch.float16: 11, torch.float32: 24}   # incl. the hidden bit
MIN_EXP = {torch.bfloat16: -126, torch.float16: -14, torch.float32: -126}


def rne(q, dtype):
    """Round the rational q to the nearest value of `dtype` (ties to even), generically:
    scale so that one unit is the spacing at q's binade (or the subnormal spacing), round the
    integer, scale back.  Returns a Fraction."""
    q = Fraction(q)
    if q == 0:
        return q
    p = MANT_BITS[dtype]
    a = abs(q)
    e = a.numerator.bit_length() - a.denominator.bit_length()
    if Fraction(2) ** e > a:
        e -= 1
    e = max(e, MIN_EXP[dtype])
    unit = Fraction(2) ** (e - (p - 1))
    n = a / unit
    lo = n.numerator // n.denominator
    rem = n - lo
    if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and lo % 2 == 1):
        lo += 1
    return (lo * unit) if q > 0 else -(lo * unit)


def fr(t):
    """tensor -> list of exact Fractions"""
    return [Fraction(float(v)) for v in t.flatten().tolist()]


def to_t(vals, dtype, shape):
    return torch.tensor([float(v) for v in vals], dtype=torch.float64).to(dtype).reshape(shape)


# --------------------------------------------------------------- conversions

def test_bf16_and_f16_conversions_match_library_casts():
    g = gen(40)
    vals = torch.cat([
        torch.randn(20000, generator=g) * 3,
        torch.randn(5000, generator=g) * 1e-6,            # fp16 subnormal range
        torch.randn(2000, generator=g) * 7e4,             # fp16 overflow edge
        torch.tensor([0.0, -0.0, 1.0, 65504.0, 65519.9, 65520.0, 5.96e-8, 2.98e-8, 2.99e-8,
                      float("inf"), -float("inf"), 1.00390625, 1.01171875]),
    ]).float()
    lib = c_oracle.lib()
    b = np.array([lib.oracle_f32_to_bf16(float(v)) for v in vals], dtype=np.uint16)
    h = np.array([lib.oracle_f32_to_f16(float(v)) for v in vals], dtype=np.uint16)
    assert np.array_equal(b, vals.bfloat16().view(torch.int16).numpy().view(np.uint16))
    assert np.array_equal(h, vals.numpy().astype(np.float16).view(np.uint16))
    back = np.array([lib.oracle_f16_to_f32(int(x)) for x in h[:5000]], dtype=np.float32)
    assert np.array_equal(back, h[:5000].view(np.float16).astype(np.float32))


def test_generic_rounding_helper_agrees_with_library_casts():
    g = gen(41)
    vals = (torch.randn(3000, generator=g, dtype=torch.float64) * 2).tolist()
    for dtype in (torch.bfloat16, torch.float16):
        want = torch.tensor(vals, dtype=torch.float64).to(torch.float32).to(dtype).double().tolist()
        # the cast above rounds twice (f64 -> f32 -> dtype); feed the helper the f32 value
        f32 = torch.tensor(vals, dtype=torch.float64).float().double().tolist()
        got = [float(rne(Fraction(v), dtype)) for v in f32]
        assert got == want


# ------------------------------------------------------------------ rms_norm

def _exact_rms_row(x, w, eps, dtype, fused_res=None):
    """Exact-arithmetic rms_norm of one row with the reference's two roundings
    (csrc/layernorm_kernels.cu:27,33).  sqrt via float64 (53 bits, far below bf16/fp16 spacing)."""
    xs = fr(x)
    new_res = None
    if fused_res is not None:
        xs = [rne(a + b, dtype) for a, b in zip(xs, fr(fused_res))]
        new_res = xs
    ss = sum(v * v for v in xs)
    s = Fraction(1.0 / math.sqrt(float(ss / len(xs) + Fraction(eps))))
    out = [rne(rne(v * s, dtype) * wv, dtype) for v, wv in zip(xs, fr(w))]
    single = [rne(v * s * wv, dtype) for v, wv in zip(xs, fr(w))]
    return out, single, new_res


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_rms_norm_exact_arithmetic_tiny(dtype):
    g = gen(42)
    T, H = 24, 48
    x = randn((T, H), g, dtype)
    w = randn((H,), g, dtype, mean=1.0, std=0.1)
    eps = float(np.float32(1e-5))
    got = torch.empty_like(x)
    c_oracle.rms_norm(got, x, w, eps)
    want, single = [], []
    for r in range(T):
        o, s1, _ = _exact_rms_row(x[r], w, eps, dtype)
        want += o
        single += s1
    want_t, single_t = to_t(want, dtype, (T, H)), to_t(single, dtype, (T, H))
    # fp32 accumulation vs exact sums can flip a rounding that sits on a boundary: allow a
    # handful of one-ulp flips, nothing else
    diff = (got.float() - want_t.float()).abs()
    assert (diff > 0).float().mean().item() < 0.01
    assert bool((diff <= ulp_of(want_t) * 2).all())
    # discriminates: a single rounding (dropping the cast before the weight multiply) differs
    assert (single_t != want_t).float().mean().item() > 0.02


def test_rms_norm_closed_forms_and_library():
    # constant row, unit weight: out = T(T(c * rsqrt(c^2 + eps)))
    for c in (0.5, 3.0, -7.25):
        x = torch.full((2, 64), c, dtype=torch.bfloat16)
        out = torch.empty_like(x)
        c_oracle.rms_norm(out, x, torch.ones(64, dtype=torch.bfloat16), 1e-6)
        want = torch.tensor(c / math.sqrt(c * c + 1e-6)).bfloat16()
        assert bool((out == want).all())
    x = torch.zeros((3, 40), dtype=torch.bfloat16)
    out = torch.ones_like(x)
    c_oracle.rms_norm(out, x, torch.ones(40, dtype=torch.bfloat16), 1e-5)
    assert bool((out == 0).all())
    # fp32 path against torch's own rms_norm (library routine)
    g = gen(43)
    x = torch.randn((33, 1000), generator=g)
    w = torch.randn((1000,), generator=g) * 0.1 + 1
    out = torch.empty_like(x)
    c_oracle.rms_norm(out, x, w, 1e-5)
    assert torch.allclose(out, F.rms_norm(x, (1000,), w, 1e-5), rtol=2e-6, atol=1e-6)
    # discriminates: epsilon matters on a row of small values
    xs = (torch.randn((4, 64), generator=g) * 1e-3).bfloat16()
    a, b = torch.empty_like(xs), torch.empty_like(xs)
    c_oracle.rms_norm(a, xs, torch.ones(64, dtype=torch.bfloat16), 1e-5)
    c_oracle.rms_norm(b, xs, torch.ones(64, dtype=torch.bfloat16), 0.0)
    assert (a != b).float().mean().item() > 0.9


def test_rms_norm_block_reduce_shapes():
    """Hidden sizes around the reference's 1024-thread block and 32-lane warps (reduction_utils.cuh)
    stay within fp32 rounding of the exact sum."""
    g = gen(44)
    for H in (1, 31, 32, 33, 1023, 1024, 1025, 4096, 5000):
        x = torch.randn((3, H), generator=g)
        out = torch.empty_like(x)
        c_oracle.rms_norm(out, x, torch.ones(H), 1e-5)
        ref = x.double() / torch.sqrt(x.double().pow(2).mean(-1, keepdim=True) + 1e-5)
        assert torch.allclose(out.double(), ref, rtol=3e-6, atol=1e-7)


def test_fused_add_rms_norm_is_add_then_norm():
    """models/llama.py:248-252: residual = T(x + r); x = rms_norm(residual), bit for bit."""
    g = gen(0)
    for dtype in (torch.bfloat16, torch.float16, torch.float32):
        x, r = randn((64, 512), g, dtype), randn((64, 512), g, dtype)
        w = randn((512,), g, dtype, mean=1.0, std=0.1)
        fx, fr_ = x.clone(), r.clone()
        c_oracle.fused_add_rms_norm(fx, fr_, w, 1e-5)
        z = x + r                                  # one rounding to the dtype (library add)
        want = torch.empty_like(z)
        c_oracle.rms_norm(want, z, w, 1e-5)
        assert torch.equal(fr_, z) and torch.equal(fx, want)
        # r = 0 reduces the fused op to rms_norm
        fx2, zero = x.clone(), torch.zeros_like(x)
        c_oracle.fused_add_rms_norm(fx2, zero, w, 1e-5)
        plain = torch.empty_like(x)
        c_oracle.rms_norm(plain, x, w, 1e-5)
        assert torch.equal(fx2, plain) and torch.equal(zero, x)
    # discriminates: the variance is taken over the ROUNDED sum, not over x + r in fp32
    x, r = randn((8, 64), g), randn((8, 64), g)
    w = torch.ones(64, dtype=torch.bfloat16)
    fx, fr_ = x.clone(), r.clone()
    c_oracle.fused_add_rms_norm(fx, fr_, w, 1e-5)
    exact_rows = []
    for i in range(8):
        o, _, _ = _exact_rms_row(x[i], w, float(np.float32(1e-5)), torch.bfloat16, fused_res=r[i])
        exact_rows += o
    want = to_t(exact_rows, torch.bfloat16, (8, 64))
    assert (fx != want).float().mean().item() < 0.02


def test_c1_config_against_torch_formulation():
    """Benchmark configuration 1: fused_add_rms_norm on bf16 [512, 4096], weight ~N(1, 0.1),
    eps 1e-5: the C oracle and the tensor-level formulation agree except for rare one-ulp flips
    caused by the order of the fp32 sum."""
    g = gen(0)
    x, r = randn((512, 4096), g), randn((512, 4096), g)
    w = randn((4096,), g, mean=1.0, std=0.1)
    ax, ar, bx, br = x.clone(), r.clone(), x.clone(), r.clone()
    c_oracle.fused_add_rms_norm(ax, ar, w, 1e-5)
    torch_formulations.fused_add_rms_norm(bx, br, w, 1e-5)
    assert torch.equal(ar, br)
    d = (ax.float() - bx.float()).abs()
    assert (d > 0).float().mean().item() < 1e-3 and bool((d <= 2 * ulp_of(ax)).all())


# ---------------------------------------------------------------- activation

@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_silu_and_mul_exact_arithmetic_tiny(dtype):
    g = gen(45)
    T, d = 16, 40
    inp = randn((T, 2 * d), g, dtype, std=2.5)
    got = torch.empty((T, d), dtype=dtype)
    c_oracle.silu_and_mul(got, inp)
    want, single = [], []
    for t in range(T):
        xs, ys = fr(inp[t, :d]), fr(inp[t, d:])
        for xv, yv in zip(xs, ys):
            sig = Fraction(float(xv)) / Fraction(1.0 + math.exp(-float(xv)))
            want.append(rne(rne(sig, dtype) * yv, dtype))
            single.append(rne(sig * yv, dtype))
    want_t, single_t = to_t(want, dtype, (T, d)), to_t(single, dtype, (T, d))
    diff = (got.float() - want_t.float()).abs()
    assert (diff > 0).float().mean().item() < 0.01 and bool((diff <= 2 * ulp_of(want_t)).all())
    assert (single_t != want_t).float().mean().item() > 0.02     # discriminates: dropped rounding


def test_silu_and_mul_library_and_limits():
    g = gen(46)
    x = randn((32, 2 * 1024), g)
    out = torch.empty((32, 1024), dtype=torch.bfloat16)
    c_oracle.silu_and_mul(out, x)
    assert torch.equal(out, F.silu(x[:, :1024]) * x[:, 1024:])       # library silu, bf16 multiply
    ones = x.clone()
    ones[:, 1024:] = 1.0
    c_oracle.silu_and_mul(out, ones)
    assert torch.equal(out, F.silu(x[:, :1024]))                       # y = 1 reduces to silu
    xs = torch.tensor([[0.0, 40.0, -200.0, 1e4, -1e4, 2.0, 2.0, 2.0, 2.0, 2.0]], dtype=torch.bfloat16)
    out = torch.empty((1, 5), dtype=torch.bfloat16)
    c_oracle.silu_and_mul(out, xs)
    assert out[0].tolist() == [0.0, 80.0, -0.0, 19968.0, -0.0]         # x->+inf: x ; x->-inf: -0
    # discriminates: x and y halves are not interchangeable
    swapped = torch.cat((x[:, 1024:], x[:, :1024]), -1).contiguous()
    o1, o2 = torch.empty((32, 1024), dtype=torch.bfloat16), torch.empty((32, 1024), dtype=torch.bfloat16)
    c_oracle.silu_and_mul(o1, x)
    c_oracle.silu_and_mul(o2, swapped)
    assert (o1 != o2).float().mean().item() > 0.9


@pytest.mark.parametrize("name", ["gelu_new", "gelu_fast"])
def test_gelu_library_and_exact_arithmetic(name):
    g = gen(47)
    # fp32 path == the tanh GELU of the library (formula, constants)
    x = torch.randn((16, 333), generator=g) * 2
    out = torch.empty_like(x)
    getattr(c_oracle, name)(out, x)
    assert torch.allclose(out, F.gelu(x, approximate="tanh"), rtol=1e-5, atol=2e-6)
    # bf16: the reference's sequence of casts (csrc/activation_kernels.cu:86-98), exactly
    dtype = torch.bfloat16
    xb = randn((6, 50), g, dtype, std=2.0)
    got = torch.empty_like(xb)
    getattr(c_oracle, name)(got, xb)
    c79, c04 = Fraction(float(np.float32(0.79788456))), Fraction(float(np.float32(0.044715)))
    R = lambda q: rne(q, dtype)  # noqa: E731
    R32 = lambda q: rne(q, torch.float32)  # noqa: E731
    want = []
    for v in fr(xb):
        if name == "gelu_new":
            x3 = R(R(v * v) * v)
            inner = R(R32(c79 * R(v + R(R32(c04 * x3)))))
        else:
            inner = R(R(R32(v * c79)) * R(1 + R(R(R32(c04 * v)) * v)))
        t = R(Fraction(math.tanh(float(inner))))
        want.append(R(R(Fraction(1, 2) * v) * R(1 + t)))
    want_t = to_t(want, dtype, xb.shape)
    diff = (got.float() - want_t.float()).abs()
    assert (diff > 0).float().mean().item() < 0.02 and bool((diff <= 2 * ulp_of(want_t)).all())
    assert torch.allclose(got.float(), F.gelu(xb.float(), approximate="tanh"), rtol=3e-2, atol=3e-2)


# -------------------------------------------------------------------- rotary

def _rope_inputs(dtype, T=12, nq=3, nkv=2, D=16, R=16, seed=48):
    g = gen(seed)
    cache = cos_sin_cache(64, R, 10000.0, dtype)
    pos = torch.randint(0, 64, (T,), generator=g, dtype=torch.int64)
    q, k = randn((T, nq * D), g, dtype), randn((T, nkv * D), g, dtype)
    return pos, q, k, cache


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("is_neox", [True, False])
def test_rope_exact_arithmetic_tiny(dtype, is_neox):
    T, nq, nkv, D, Rd = 12, 3, 2, 16, 8          # partial rotary: dims >= 8 untouched
    pos, q, k, cache = _rope_inputs(dtype, T, nq, nkv, D, Rd)
    gq, gk = q.clone(), k.clone()
    c_oracle.rotary_embedding(pos, gq, gk, D, cache, is_neox)
    R = lambda v: rne(v, dtype)  # noqa: E731
    flipped = 0
    for arr, got, nh in ((q, gq, nq), (k, gk, nkv)):
        for t in range(T):
            crow = fr(cache[pos[t]])
            for h in range(nh):
                head = fr(arr[t, h * D:(h + 1) * D])
                want = list(head)
                wrong_sign = list(head)
                for i in range(Rd // 2):
                    xi, yi = (i, Rd // 2 + i) if is_neox else (2 * i, 2 * i + 1)
                    c, s = crow[i], crow[Rd // 2 + i]
                    x, y = head[xi], head[yi]
                    want[xi] = R(R(x * c) - R(y * s))
                    want[yi] = R(R(y * c) + R(x * s))
                    wrong_sign[xi] = R(R(x * c) + R(y * s))
                exp = to_t(want, dtype, (D,))
                assert torch.equal(got[t, h * D:(h + 1) * D], exp)
                flipped += int((to_t(wrong_sign, dtype, (D,)) != exp).sum())
    assert flipped > T        # discriminates: a flipped sign changes the answer on these inputs


def test_rope_is_complex_rotation_and_matches_rotate_half_formulation():
    """fp32: (x + iy) * (cos + i sin); and the HF Llama formulation q*cos + rotate_half(q)*sin."""
    T, nq, nkv, D = 40, 4, 2, 32
    g = gen(49)
    cache = cos_sin_cache(256, D, THETA_LLAMA3, torch.float32)
    pos = torch.randint(0, 256, (T,), generator=g, dtype=torch.int64)
    q, k = torch.randn((T, nq * D), generator=g), torch.randn((T, nkv * D), generator=g)
    gq, gk = q.clone(), k.clone()
    c_oracle.rotary_embedding(pos, gq, gk, D, cache, True)
    cos, sin = cache[pos][:, : D // 2], cache[pos][:, D // 2:]
    z = torch.complex(q.view(T, nq, 2, D // 2)[:, :, 0], q.view(T, nq, 2, D // 2)[:, :, 1])
    rot = z * torch.complex(cos, sin).unsqueeze(1)
    want = torch.stack((rot.real, rot.imag), dim=2).reshape(T, nq * D)
    assert torch.allclose(gq, want, rtol=1e-5, atol=1e-6)
    try:
        from transformers.models.llama.modeling_llama import rotate_half
    except Exception:                                            # pragma: no cover
        rotate_half = lambda x: torch.cat((-x[..., x.shape[-1] // 2:], x[..., : x.shape[-1] // 2]), -1)  # noqa: E731
    cos_full, sin_full = torch.cat((cos, cos), -1).unsqueeze(1), torch.cat((sin, sin), -1).unsqueeze(1)
    kv = k.view(T, nkv, D)
    want_k = (kv * cos_full + rotate_half(kv) * sin_full).reshape(T, nkv * D)
    assert torch.allclose(gk, want_k, rtol=1e-5, atol=1e-6)
    # position 0 is the identity (cos = 1, sin = 0), bit for bit
    iq, ik = q.clone(), k.clone()
    c_oracle.rotary_embedding(torch.zeros(T, dtype=torch.int64), iq, ik, D, cache, True)
    assert torch.equal(iq, q) and torch.equal(ik, k)


def test_rope_gptj_equals_neox_on_deinterleaved_data_and_strides():
    T, nq, nkv, D = 30, 4, 2, 64
    g = gen(50)
    cache = cos_sin_cache(512, D, 10000.0, torch.bfloat16)
    pos = hybrid_positions(T, 20, g, prefill_start=100, max_pos=512)
    qkv = randn((T, (nq + 2 * nkv) * D), g)
    # GPT-J on interleaved (x0,y0,x1,y1,..) == NeoX on (x0,x1,..,y0,y1,..)
    a = qkv.clone()
    aq, ak, _ = a.split([nq * D, nkv * D, nkv * D], -1)
    c_oracle.rotary_embedding(pos, aq, ak, D, cache, False)
    heads = qkv.view(T, nq + 2 * nkv, D)
    de = torch.cat((heads[..., 0::2], heads[..., 1::2]), -1).reshape(T, -1).contiguous()
    bq, bk, _ = de.split([nq * D, nkv * D, nkv * D], -1)
    c_oracle.rotary_embedding(pos, bq, bk, D, cache, True)
    back = de.view(T, nq + 2 * nkv, 2, D // 2).transpose(2, 3).reshape(T, -1)
    assert torch.equal(a, back)
    # strided views of the packed buffer == contiguous copies; the v part is untouched
    cq, ck = qkv[:, : nq * D].contiguous(), qkv[:, nq * D:(nq + nkv) * D].contiguous()
    c_oracle.rotary_embedding(pos, cq, ck, D, cache, False)
    assert torch.equal(aq, cq) and torch.equal(ak, ck)
    assert torch.equal(a[:, (nq + nkv) * D:], qkv[:, (nq + nkv) * D:])
    # tensor-level formulation agrees bit for bit
    t = qkv.clone()
    tq, tk, _ = t.split([nq * D, nkv * D, nkv * D], -1)
    torch_formulations.rotary_embedding(pos, tq, tk, D, cache, False)
    assert torch.equal(t, a)


# ------------------------------------------------------------- topk_softmax

def _topk(gating, k):
    T = gating.shape[0]
    w = torch.empty((T, k))
    i = torch.empty((T, k), dtype=torch.int32)
    s = torch.empty((T, k), dtype=torch.int32)
    c_oracle.topk_softmax(w, i, s, gating)
    return w, i, s


@pytest.mark.parametrize("E,k", [(8, 2), (1, 1), (2, 2), (4, 3), (16, 4), (64, 6), (128, 8),
                                 (256, 8), (6, 2), (60, 4), (300, 5), (1000, 3)])
def test_topk_softmax_against_library_softmax_and_sort(E, k):
    g = gen(3)
    T = 300
    gating = torch.randn((T, E), generator=g)
    w, i, s = _topk(gating, k)
    p = torch.softmax(gating.double(), -1)
    order = torch.sort(p, dim=-1, descending=True, stable=True)
    assert torch.equal(i.long(), order.indices[:, :k])
    assert torch.allclose(w.double(), order.values[:, :k], rtol=0, atol=2e-7)
    assert torch.equal(s, (torch.arange(k).unsqueeze(0) * T + torch.arange(T).unsqueeze(1)).int())
    assert bool((w[:, :-1] >= w[:, 1:]).all())
    if k == E:
        assert torch.equal(torch.sort(i, -1).values, torch.arange(E).int().expand(T, E))
        assert torch.allclose(w.sum(-1), torch.ones(T), atol=1e-6)


def test_topk_softmax_ties_take_lower_index():
    rows = torch.tensor([[1.0] * 8,
                         [0.0, 5.0, 5.0, 0.0, 5.0, 0.0, 0.0, 0.0],
                         [0.0, -300.0, -200.0, -250.0, -400.0, -210.0, -220.0, -230.0]])
    w, i, _ = _topk(rows, 3)
    assert i.tolist() == [[0, 1, 2], [1, 2, 4], [0, 1, 2]]
    assert w[0].tolist() == [0.125] * 3 and w[2].tolist() == [1.0, 0.0, 0.0]
    for E in (6, 16, 64, 100, 256):          # generic and grouped layouts alike
        _, i, _ = _topk(torch.zeros((2, E)), min(E, 5))
        assert i[0].tolist() == list(range(min(E, 5)))


# ---------------------------------------------------- moe_align_block_size

def _align(fn, ids, E, B):
    n = ids.numel() + E * (B - 1)
    s = torch.full((n,), ids.numel(), dtype=torch.int32)
    e = torch.full(((n + B - 1) // B,), -1, dtype=torch.int32)
    p = torch.full((1,), -1, dtype=torch.int32)
    fn(ids, E, B, s, e, p)
    return s, e, p


def test_moe_align_reference_vectors():
    with open(GOLDEN) as f:
        vectors = json.load(f)["vectors"]
    assert len(vectors) == 2
    for v in vectors:
        ids = torch.tensor(v["topk_ids"], dtype=torch.int32)
        for fn in (c_oracle.moe_align_block_size, torch_formulations.moe_align_block_size):
            s, e, p = _align(fn, ids, v["num_experts"], v["block_size"])
            n = v["num_tokens_post_pad"]
            assert p.item() == n
            assert s[:n].tolist() == v["sorted_token_ids_prefix"]
            assert bool((s[n:] == ids.numel()).all())
            assert e[: n // v["block_size"]].tolist() == v["expert_ids_prefix"]


def _brute_force_align(flat, E, B):
    out, eids = [], []
    for x in range(E):
        toks = [i for i, v in enumerate(flat) if v == x]      # ascending = stable
        nb = (len(toks) + B - 1) // B
        out += toks + [len(flat)] * (nb * B - len(toks))
        eids += [x] * nb
    return out, eids


@pytest.mark.parametrize("numel,E,B", [(0, 4, 4), (1, 1, 1), (9, 5, 4), (100, 8, 16), (777, 60, 8),
                                       (4096 * 2, 8, 64), (1000, 256, 32), (333, 7, 1)])
def test_moe_align_brute_force_and_invariants(numel, E, B):
    g = gen(numel + E)
    ids = torch.randint(0, E, (numel,), generator=g, dtype=torch.int32)
    want, want_e = _brute_force_align(ids.tolist(), E, B)
    for fn in (c_oracle.moe_align_block_size, torch_formulations.moe_align_block_size):
        s, e, p = _align(fn, ids, E, B)
        n = p.item()
        assert n == len(want) and n % B == 0
        assert s[:n].tolist() == want and e[: n // B].tolist() == want_e
        assert bool((s[n:] == numel).all()) and bool((e[n // B:] == -1).all())
        real = s[:n][s[:n] != numel]
        assert torch.equal(torch.sort(real).values, torch.arange(numel, dtype=torch.int32))


@pytest.mark.parametrize("dtype", [torch.uint8, torch.int8, torch.int16, torch.int32, torch.int64])
def test_moe_align_id_dtypes(dtype):
    g = gen(51)
    ids32 = torch.randint(0, 100, (500,), generator=g, dtype=torch.int32)
    a = _align(c_oracle.moe_align_block_size, ids32, 100, 8)
    b = _align(c_oracle.moe_align_block_size, ids32.to(dtype), 100, 8)
    assert all(torch.equal(x, y) for x, y in zip(a, b))


# ------------------------------------------------------- grouped expert GEMM

def _routing(T, E, k, B, seed):
    g = gen(seed)
    gating = torch.randn((T, E), generator=g)
    w, ids, _ = _topk(gating, k)
    s, e, p = _align(c_oracle.moe_align_block_size, ids, E, B)
    return gating, w, ids, s, e, p


def test_grouped_gemm_formulation_brute_force():
    """The tensor formulation of the reference's Triton kernel against a scalar float64 loop that
    does not use the sorted layout at all: C[t, j] = w[t, j] * A[t] @ B[ids[t, j]]^T."""
    T, E, k, B, N, K = 23, 4, 2, 8, 12, 16
    _, w, ids, s, e, p = _routing(T, E, k, B, 60)
    g = gen(61)
    A = randn((T, K), g)
    Bw = randn((E, N, K), g)
    for mul in (False, True):
        C = torch.full((T, k, N), 9.0, dtype=torch.bfloat16)
        torch_formulations.moe_grouped_gemm(A, Bw, C, w, s, e, p, T * k, B, k, mul)
        for t in range(T):
            for j in range(k):
                ref = A[t].double() @ Bw[int(ids[t, j])].double().t()
                if mul:
                    ref = ref * float(w[t, j])
                assert torch.allclose(C[t, j].double(), ref, rtol=2 ** -7, atol=1e-6)
    # every (token, j) row is written exactly once: no sentinel survives
    assert not bool((C == 9.0).all(dim=-1).any())
    # identity weights reproduce the token row exactly
    eye = torch.stack([torch.eye(K)] * E).bfloat16()
    C = torch.zeros((T, k, K), dtype=torch.bfloat16)
    torch_formulations.moe_grouped_gemm(A, eye, C, w, s, e, p, T * k, B, k, False)
    assert torch.equal(C, A.unsqueeze(1).expand(T, k, K))


def test_fused_moe_formulation_against_float64_dense():
    T, E, k, H, I = 40, 4, 2, 32, 48
    g = gen(62)
    x = randn((T, H), g)
    w1 = randn((E, 2 * I, H), g, std=H ** -0.5)
    w2 = randn((E, H, I), g, std=I ** -0.5)
    gating = torch.randn((T, E), generator=g)
    got = torch_formulations.fused_moe(x, w1, w2, gating, k, True)
    p = torch.softmax(gating.double(), -1)
    tw, ti = torch.topk(p, k, dim=-1)
    tw = tw / tw.sum(-1, keepdim=True)
    want = torch.zeros((T, H), dtype=torch.float64)
    for t in range(T):
        for j in range(k):
            ex = int(ti[t, j])
            gu = w1[ex].double() @ x[t].double()
            h = torch.nn.functional.silu(gu[:I]) * gu[I:]
            want[t] += tw[t, j] * (w2[ex].double() @ h)
    assert torch.allclose(got.double(), want, rtol=3e-2, atol=3e-2 * want.abs().max().item())


# ---- paged KV-cache append (oracle/paged_kv.py) ------------------------------------------------

def _paged_case(seed, page_size, lens_before, new_tokens, heads=2, head_size=4, spare_pages=3):
    """Random page tables for requests that already hold lens_before[i] tokens and get
    new_tokens[i] more."""
    import numpy as np
    rng = np.random.default_rng(seed)
    totals = [a + b for a, b in zip(lens_before, new_tokens)]
    need = [(t + page_size - 1) // page_size for t in totals]
    num_pages = sum(need) + spare_pages
    perm = rng.permutation(num_pages)
    kv_indptr = np.concatenate([[0], np.cumsum(need)]).astype(np.int32)
    kv_indices = perm[:sum(need)].astype(np.int32)
    last = np.array([(t % page_size) or page_size if t > 0 else 0 for t in totals], dtype=np.int32)
    append_indptr = np.concatenate([[0], np.cumsum(new_tokens)]).astype(np.int32)
    nnz = int(append_indptr[-1])
    k = rng.standard_normal((nnz, heads, head_size)).astype(np.float32)
    v = rng.standard_normal((nnz, heads, head_size)).astype(np.float32)
    cache = rng.standard_normal((num_pages, 2, page_size, heads, head_size)).astype(np.float32)
    return dict(kv_indptr=kv_indptr, kv_indices=kv_indices, last=last, append_indptr=append_indptr,
                nnz=nnz, k=k, v=v, cache=cache, totals=totals, page_size=page_size)


def test_paged_kv_hand_worked_example():
    """Two requests, page size 4.  Request 0 holds 5 tokens after getting 3 new ones (pages 7, 2);
    request 1 is a decode step reaching 9 tokens (pages 0, 5, 3)."""
    import numpy as np
    from oracle import paged_kv
    kv_indptr, kv_indices = [0, 2, 5], [7, 2, 0, 5, 3]
    last = [1, 1]
    seq_lens = paged_kv.get_seq_lens(kv_indptr, last, 4)
    assert seq_lens.tolist() == [5, 9]
    b, pos = paged_kv.get_batch_indices_positions([0, 3, 4], seq_lens, 4)
    assert b.tolist() == [0, 0, 0, 1] and pos.tolist() == [2, 3, 4, 8]
    cache = np.zeros((8, 2, 4, 1, 1), dtype=np.float32)
    k = np.arange(1, 5, dtype=np.float32).reshape(4, 1, 1)
    paged_kv.append_paged_kv_cache(k, -k, b, pos, cache[:, 0], cache[:, 1], kv_indices, kv_indptr)
    want = {(7, 2): 1.0, (7, 3): 2.0, (2, 0): 3.0, (3, 0): 4.0}   # (page, entry) -> key value
    for page in range(8):
        for e in range(4):
            assert cache[page, 0, e, 0, 0] == want.get((page, e), 0.0)
            assert cache[page, 1, e, 0, 0] == -want.get((page, e), 0.0)


@pytest.mark.parametrize("page_size,before,new", [
    (4, [0, 0, 0], [1, 7, 8]),                # fresh prompts, lengths around page multiples
    (16, [30, 16, 0, 5], [3, 1, 40, 1]),      # chunked prefill continuation + decodes
    (1, [2, 0], [3, 2]),                      # page size 1
    (8, [7, 8, 9], [1, 1, 1]),                # decode steps straddling a page boundary
    (8, [3, 0, 11], [0, 5, 0]),               # requests with nothing to append
])
def test_paged_kv_round_trip_and_untouched_entries(page_size, before, new):
    """Appending the new tokens after the old ones and gathering each request through its page
    table returns old || new in order; every entry nobody wrote keeps its bytes."""
    import numpy as np
    from oracle import paged_kv
    c = _paged_case(page_size + len(new), page_size, before, new)
    seq_lens = paged_kv.get_seq_lens(c["kv_indptr"], c["last"], page_size)
    assert seq_lens.tolist() == c["totals"]
    b, pos = paged_kv.get_batch_indices_positions(c["append_indptr"], seq_lens, c["nnz"])
    assert (b >= 0).all()
    for r in range(len(new)):
        lo, hi = c["append_indptr"][r], c["append_indptr"][r + 1]
        assert (b[lo:hi] == r).all()
        assert pos[lo:hi].tolist() == list(range(before[r], before[r] + new[r]))
    cache = c["cache"].copy()
    paged_kv.append_paged_kv_cache(c["k"], c["v"], b, pos, cache[:, 0], cache[:, 1],
                                   c["kv_indices"], c["kv_indptr"])
    written = np.zeros(cache.shape[:3], dtype=bool)
    for r in range(len(new)):
        lo, hi = c["append_indptr"][r], c["append_indptr"][r + 1]
        for plane, src in ((0, c["k"]), (1, c["v"])):
            got = paged_kv.gather_sequence(cache[:, plane], c["kv_indices"], c["kv_indptr"],
                                           seq_lens, r)
            old = paged_kv.gather_sequence(c["cache"][:, plane], c["kv_indices"], c["kv_indptr"],
                                           seq_lens, r)
            assert np.array_equal(got[before[r]:], src[lo:hi])
            assert np.array_equal(got[:before[r]], old[:before[r]])
        pages = c["kv_indices"][c["kv_indptr"][r]:c["kv_indptr"][r + 1]]
        for j in range(before[r], before[r] + new[r]):
            written[pages[j // page_size], :, j % page_size] = True
    assert np.array_equal(cache[~written], c["cache"][~written])
    assert not np.array_equal(cache[written], c["cache"][written]) or not written.any()


# ---- grouped_topk (oracle/torch_formulations.py) -------------------------------------------------

def test_grouped_topk_single_group_reduces_to_topk_softmax():
    """One group that is always kept: the routing is plain softmax + top-k, which is pinned above."""
    from oracle import c_oracle, torch_formulations
    g = torch.Generator().manual_seed(4)
    gating = torch.randn((64, 16), generator=g)
    w, ids = torch_formulations.grouped_topk(gating, 4, False, 1, 1)
    ww = torch.empty((64, 4)); wi = torch.empty((64, 4), dtype=torch.int32)
    ws = torch.empty((64, 4), dtype=torch.int32)
    c_oracle.topk_softmax(ww, wi, ws, gating)
    assert torch.equal(ids, wi) and torch.allclose(w, ww, rtol=0, atol=1e-6)


def test_grouped_topk_hand_worked_example():
    """6 experts in 3 groups of 2, keep 2 groups, top-3.  Logits chosen so that the probabilities
    order as e4 > e1 > e5 > e0 > e2 > e3: groups score (e1, e2, e4) -> groups 2 and 0 stay, group 1
    (e2, e3) is masked, and the three best of {e0, e1, e4, e5} are e4, e1, e5."""
    from oracle import torch_formulations
    logits = torch.tensor([[1.0, 3.0, 0.5, 0.0, 4.0, 2.0]])
    w, ids = torch_formulations.grouped_topk(logits, 3, False, 3, 2)
    assert ids.tolist() == [[4, 1, 5]]
    p = torch.softmax(logits, dim=-1)[0]
    assert torch.allclose(w[0], p[[4, 1, 5]])
    # keeping a single group: e4's group (e4, e5) only; the third pick is a masked expert with
    # weight 0, the lowest index among them
    w1, ids1 = torch_formulations.grouped_topk(logits, 3, False, 3, 1)
    assert ids1.tolist() == [[4, 5, 0]] and w1[0, 2].item() == 0.0
    # renormalised weights sum to one
    wr, _ = torch_formulations.grouped_topk(logits, 3, True, 3, 2)
    assert abs(float(wr.sum()) - 1.0) < 1e-6


def test_grouped_topk_selected_experts_stay_inside_the_kept_groups():
    from oracle import torch_formulations
    g = torch.Generator().manual_seed(9)
    gating = torch.randn((200, 160), generator=g)
    w, ids = torch_formulations.grouped_topk(gating, 6, True, 8, 3)      # DeepSeek-V2 shape
    p = torch.softmax(gating, dim=-1)
    for t in range(200):
        groups = set((ids[t] // 20).tolist())
        assert len(groups) <= 3
        gs = p[t].view(8, 20).max(dim=-1).values
        kept = set(torch.topk(gs, 3).indices.tolist())
        assert groups <= kept
        # nothing better was left behind inside the kept groups
        inside = torch.tensor([e for e in range(160) if e // 20 in kept])
        assert torch.equal(torch.sort(ids[t].long()).values,
                           torch.sort(inside[torch.topk(p[t][inside], 6).indices]).values)
