"""GPU: the grouped expert GEMM (the consumer of moe_align_block_size's layout) and the whole
fused MoE forward, against CPU formulations in fp32.

The contraction's accumulation order is not defined by the reference (Triton's tl.dot), so the
comparison is by tolerance: |got - want| <= 1e-2 * max|want| + 1e-2 * |want| for bf16/fp16
outputs.  The identity-weight case has exactly one non-zero product per output and must be exact.
"""
import pytest
import torch

from helpers import gen, randn
from oracle import c_oracle, torch_formulations

pytestmark = pytest.mark.gpu


def _route(T, E, k, B, seed):
    g = gen(seed)
    gating = torch.randn((T, E), generator=g, dtype=torch.float32)
    w = torch.empty((T, k))
    ids = torch.empty((T, k), dtype=torch.int32)
    src = torch.empty((T, k), dtype=torch.int32)
    c_oracle.topk_softmax(w, ids, src, gating)
    n = T * k + E * (B - 1)
    s = torch.full((n,), T * k, dtype=torch.int32)
    e = torch.zeros(((n + B - 1) // B,), dtype=torch.int32)
    p = torch.zeros((1,), dtype=torch.int32)
    c_oracle.moe_align_block_size(ids, E, B, s, e, p)
    return gating, w, ids, s, e, p


def _close(got, want, what):
    got, want = got.float().cpu(), want.float()
    tol = 1e-2 * want.abs().max().item() + 1e-2 * want.abs()
    bad = (got - want).abs() > tol
    assert not bool(bad.any()), "%s: %d elements outside tolerance, max diff %.4g" % (
        what, int(bad.sum()), (got - want).abs().max().item())


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("T,E,k,BM,N,K,mul", [
    (300, 8, 2, 64, 512, 256, False),
    (300, 8, 2, 64, 512, 256, True),
    (77, 4, 2, 32, 260, 128, True),      # N not a multiple of the 256-wide tile nor of 32
    (1000, 8, 2, 128, 768, 512, False),
    (1500, 4, 2, 256, 512, 256, True),   # eight-wave tile
    (40, 8, 2, 256, 300, 128, False),    # mostly padding
    (33, 16, 4, 32, 256, 64, True),      # some experts empty, single K step
    (5, 8, 1, 32, 1024, 192, False),
    (600, 8, 2, 32, 256, 128, True),     # 45 slot blocks
    (1200, 8, 2, 64, 520, 128, False),   # many blocks through both kernels' 64-slot variants, ragged N
    (2100, 4, 2, 128, 256, 64, True),    # 36 blocks of 128
    (1500, 4, 2, 256, 4100, 128, True),  # 16 slot blocks x 17 column blocks: the 256-wide tiles of
                                         # the four-wave kernel (smaller launches take 128-wide ones)
    (1200, 8, 2, 64, 6148, 64, False),   # 46 blocks of 64 x 25 column blocks: 256-wide tiles at 64 slots
])
def test_grouped_gemm_matches_formulation(ops, dev, dtype, T, E, k, BM, N, K, mul):
    _, w, ids, s, e, p = _route(T, E, k, BM, T + N)
    g = gen(K)
    A = randn((T, K), g, dtype, std=0.5)
    Bw = randn((E, N, K), g, dtype, std=0.5)
    want = torch.zeros((T, k, N), dtype=dtype)
    torch_formulations.moe_grouped_gemm(A, Bw, want, w, s, e, p, T * k, BM, k, mul)
    got = torch.full((T, k, N), 7.0, dtype=dtype, device=dev)
    ops.moe_ops.moe_grouped_gemm(A.to(dev), Bw.to(dev), got, w.to(dev), s.to(dev), e.to(dev),
                                 p.to(dev), T * k, BM, k, mul)
    _close(got, want, "grouped gemm")
    # packed weight layout: same products, same accumulation order -> same bits
    from sarathi_amd.layers import pack_expert_weights
    packed = pack_expert_weights(Bw.to(dev))
    assert packed.shape == (E, N, K)
    got2 = torch.full((T, k, N), 7.0, dtype=dtype, device=dev)
    ops.moe_ops.moe_grouped_gemm(A.to(dev), packed.data, got2, w.to(dev), s.to(dev), e.to(dev),
                                 p.to(dev), T * k, BM, k, mul, True, N)
    assert torch.equal(got2, got)


@pytest.mark.parametrize("packed", [False, True])
@pytest.mark.parametrize("BM", [64, 128, 256])
def test_grouped_gemm_padding_anywhere_in_a_block(ops, dev, BM, packed):
    """The kernels skip 32-slot tiles that hold no valid slot.  moe_align_block_size puts padding
    at the end of a block, but the operator accepts any slot order: shuffle the slots inside every
    block so that valid slots sit behind, between and in front of all-padding tiles; also covers
    blocks whose first or second half is entirely padding.  Same products per output, so the
    result must equal the unshuffled run bit for bit and the formulation within tolerance."""
    T, E, k, N, K = 90, 8, 2, 320, 192
    _, w, ids, s, e, p = _route(T, E, k, BM, 31 + BM)
    g = gen(BM)
    A = randn((T, K), g, std=0.5)
    Bw = randn((E, N, K), g, std=0.5)
    want = torch.zeros((T, k, N), dtype=torch.bfloat16)
    torch_formulations.moe_grouped_gemm(A, Bw, want, w, s, e, p, T * k, BM, k, True)
    used = int(p.item())
    shuffled = s.clone()
    for b in range(used // BM):
        perm = torch.randperm(BM, generator=g)
        shuffled[b * BM:(b + 1) * BM] = s[b * BM:(b + 1) * BM][perm]
    # one block with its valid slots moved to the very end (every earlier tile all padding)
    blk = s[:BM]
    shuffled[:BM] = torch.cat([blk[blk >= T * k], blk[blk < T * k]])
    Bd = Bw.to(dev)
    if packed:
        from sarathi_amd.layers import pack_expert_weights
        Bd = pack_expert_weights(Bd).data
    outs = []
    for order in (s, shuffled):
        got = torch.full((T, k, N), 7.0, dtype=torch.bfloat16, device=dev)
        ops.moe_ops.moe_grouped_gemm(A.to(dev), Bd, got, w.to(dev), order.to(dev), e.to(dev),
                                     p.to(dev), T * k, BM, k, True, packed, N)
        outs.append(got)
    _close(outs[0], want, "aligned order")
    assert torch.equal(outs[0], outs[1])


@pytest.mark.parametrize("packed", [False, True])
def test_grouped_gemm_half_empty_256_blocks_repeatable(ops, dev, packed):
    """256-slot blocks in which the second wave row holds only padding: those waves compute
    nothing but still move their share of the operands and must not let the others pass a
    barrier before it has landed (a wait sized for loads that the compiler had dropped once let
    them).  Many K-steps, many repetitions, every result identical and equal to the formulation."""
    T, E, k, BM, N, K = 60, 8, 2, 256, 512, 1536
    _, w, ids, s, e, p = _route(T, E, k, BM, 77)
    assert int(torch.bincount(ids.flatten().long(), minlength=E).max()) <= 128
    g = gen(78)
    A = randn((T, K), g, std=0.5)
    Bw = randn((E, N, K), g, std=0.5)
    want = torch.zeros((T, k, N), dtype=torch.bfloat16)
    torch_formulations.moe_grouped_gemm(A, Bw, want, w, s, e, p, T * k, BM, k, False)
    Bd = Bw.to(dev)
    if packed:
        from sarathi_amd.layers import pack_expert_weights
        Bd = pack_expert_weights(Bd).data
    args = (A.to(dev), Bd)
    tail = (w.to(dev), s.to(dev), e.to(dev), p.to(dev), T * k, BM, k, False, packed, N)
    first = None
    for rep in range(40):
        got = torch.full((T, k, N), 7.0, dtype=torch.bfloat16, device=dev)
        ops.moe_ops.moe_grouped_gemm(*args, got, *tail)
        if first is None:
            first = got
            _close(first, want, "half-empty blocks")
        else:
            assert torch.equal(got, first), "repetition %d differs" % rep


def test_grouped_gemm_second_stage_addressing(ops, dev):
    """top_k = 1 addressing of the down projection: A rows are slots (tokens * topk of them)."""
    T, E, k, BM, N, K = 200, 8, 2, 64, 256, 128
    _, w, ids, s, e, p = _route(T, E, k, BM, 5)
    g = gen(6)
    A = randn((T * k, K), g, std=0.5)
    Bw = randn((E, N, K), g, std=0.5)
    want = torch.zeros((T, k, N), dtype=torch.bfloat16)
    torch_formulations.moe_grouped_gemm(A, Bw, want, w, s, e, p, T * k, BM, 1, True)
    got = torch.zeros((T, k, N), dtype=torch.bfloat16, device=dev)
    ops.moe_ops.moe_grouped_gemm(A.to(dev), Bw.to(dev), got, w.to(dev), s.to(dev), e.to(dev),
                                 p.to(dev), T * k, BM, 1, True)
    _close(got, want, "second stage")


def test_grouped_gemm_identity_weights_exact(ops, dev):
    """B[e] = 2^e * I: every output has a single non-zero product, so C[slot] = 2^e * A[token]
    exactly; this pins operand layout, expert selection and slot addressing bit for bit."""
    T, E, k, BM, K = 500, 8, 2, 64, 256
    _, w, ids, s, e, p = _route(T, E, k, BM, 9)
    g = gen(10)
    A = randn((T, K), g)
    Bw = torch.stack([torch.eye(K) * (2.0 ** x) for x in range(E)]).bfloat16()
    got = torch.zeros((T, k, K), dtype=torch.bfloat16, device=dev)
    ops.moe_ops.moe_grouped_gemm(A.to(dev), Bw.to(dev), got, w.to(dev), s.to(dev), e.to(dev),
                                 p.to(dev), T * k, BM, k, False)
    want = A.float().unsqueeze(1) * torch.pow(2.0, ids.float()).unsqueeze(-1)
    assert torch.equal(got.float().cpu(), want)


@pytest.mark.parametrize("T,E,k,H,I,renorm", [(64, 8, 2, 256, 512, True), (700, 8, 2, 512, 1024, True),
                                            (129, 4, 1, 256, 256, False)])
def test_fused_moe_forward(ops, dev, T, E, k, H, I, renorm):
    from sarathi_amd import layers
    g = gen(T)
    x = randn((T, H), g, std=1.0)
    w1 = randn((E, 2 * I, H), g, std=H ** -0.5)
    w2 = randn((E, H, I), g, std=I ** -0.5)
    gating = torch.randn((T, E), generator=g, dtype=torch.float32)
    want = torch_formulations.fused_moe(x, w1, w2, gating, k, renorm)
    got = layers.fused_moe(x.to(dev), w1.to(dev), w2.to(dev), gating.to(dev), k, renorm)
    assert got.shape == (T, H) and got.dtype == torch.bfloat16
    _close(got, want, "fused_moe")
    # packed expert weights give the same bits
    p1, p2 = layers.pack_expert_weights(w1.to(dev)), layers.pack_expert_weights(w2.to(dev))
    got_p = layers.fused_moe(x.to(dev), p1, p2, gating.to(dev), k, renorm)
    assert torch.equal(got_p, got)
    # in place
    xd = x.to(dev)
    out = layers.fused_moe(xd, w1.to(dev), w2.to(dev), gating.to(dev), k, renorm, inplace=True)
    assert out.data_ptr() == xd.data_ptr()
    _close(xd, want, "fused_moe inplace")


@pytest.mark.parametrize("packed", [False, True])
@pytest.mark.parametrize("block_m", [64, 128, 256])
def test_fused_moe_same_bits_with_and_without_balanced_blocks(ops, dev, monkeypatch, packed, block_m):
    """With BALANCE_BLOCKS set, fused_experts spreads every expert's slots evenly over its blocks
    before the GEMMs; where a slot sits inside a block does not enter its dot products, so the
    layer's output is bit for bit the one computed on moe_align_block_size's own layout.  Experts
    with one, several and no blocks, every block size that is balanced, both weight layouts."""
    import importlib
    fm = importlib.import_module("sarathi_amd.layers.fused_moe")   # the module, not the function
    from sarathi_amd import layers
    T, E, k, H, I = 1500, 8, 2, 256, 512
    g = gen(77 + block_m)
    x = randn((T, H), g, std=1.0).to(dev)
    w1 = randn((E, 2 * I, H), g, std=H ** -0.5).to(dev)
    w2 = randn((E, H, I), g, std=I ** -0.5).to(dev)
    if packed:
        w1, w2 = layers.pack_expert_weights(w1), layers.pack_expert_weights(w2)
    gating = torch.randn((T, E), generator=g, dtype=torch.float32)
    gating[:, 5] = -50.0                        # an expert nobody picks
    gating[:, 2] += 1.5                         # and a popular one
    gating = gating.to(dev)
    cfg = {"BLOCK_SIZE_M": block_m, "BLOCK_SIZE_N": 256, "BLOCK_SIZE_K": 64, "GROUP_SIZE_M": 1}
    monkeypatch.setattr(fm, "BALANCE_BLOCKS", True)
    got = layers.fused_moe(x, w1, w2, gating, k, True, override_config=cfg)
    monkeypatch.setattr(fm, "BALANCE_BLOCKS", False)
    want = layers.fused_moe(x, w1, w2, gating, k, True, override_config=cfg)
    assert torch.equal(got, want)


def test_fused_moe_with_one_launch_routing(ops, dev, monkeypatch):
    """fused_moe with the routing + slot sort done by the single fused launch (the default for small
    batches) and by the two separate kernels: same bits."""
    import importlib
    fm = importlib.import_module("sarathi_amd.layers.fused_moe")   # the module, not the function
    from sarathi_amd import layers
    T, E, k, H, I = 300, 8, 2, 256, 512
    g = gen(21)
    x = randn((T, H), g, std=1.0).to(dev)
    w1 = randn((E, 2 * I, H), g, std=H ** -0.5).to(dev)
    w2 = randn((E, H, I), g, std=I ** -0.5).to(dev)
    gating = torch.randn((T, E), generator=g, dtype=torch.float32).to(dev)
    assert T * k <= fm.FUSED_ROUTING_MAX_SLOTS and E <= fm.FUSED_ROUTING_MAX_EXPERTS
    got = layers.fused_moe(x, w1, w2, gating, k, True)                 # one-launch routing
    monkeypatch.setattr(fm, "FUSED_ROUTING_MAX_SLOTS", 0)
    want = layers.fused_moe(x, w1, w2, gating, k, True)                # two kernels
    assert torch.equal(got, want)


def test_tuned_config_lookup_and_override(ops, dev):
    """The Mixtral-8x7B table shipped with the package is found on this device and the entry
    nearest to the batch size is used; override_config wins; unknown shapes use the default rule."""
    from sarathi_amd import layers
    table = layers.get_moe_configs(8, 14336, None)
    assert table is not None and 4096 in table and table[4096]["BLOCK_SIZE_M"] in (32, 64, 128, 256)
    w1_shape, w2_shape = (8, 28672, 4096), (8, 4096, 14336)
    assert layers.try_get_optimal_moe_config(w1_shape, w2_shape, 2, 3000) == table[3072]
    assert layers.try_get_optimal_moe_config(w1_shape, w2_shape, 2, 5) == table[4]
    forced = {"BLOCK_SIZE_M": 32}
    assert layers.try_get_optimal_moe_config(w1_shape, w2_shape, 2, 3000,
                                             override_config=forced) is forced
    rm = layers.get_moe_configs(8, 14336, None, packed=False)      # table for row-major weights
    assert rm is not None and rm[4096]["BLOCK_SIZE_M"] == 256
    assert layers.try_get_optimal_moe_config(w1_shape, w2_shape, 2, 4000, packed=False) == rm[4096]
    # every (E, N) the reference ships a 16-bit table for (its configs/ folder) has one here, for
    # both weight layouts
    shapes = [(8, n) for n in (14336, 8192, 7168, 4096, 3584, 2048, 1792)] + \
             [(16, 2688), (16, 1344), (64, 1280), (64, 640)]
    for e, n in shapes:
        for packed in (True, False):
            t = layers.get_moe_configs(e, n, None, packed=packed)
            assert t is not None and {1, 64, 4096} <= set(t), (e, n, packed)
            assert all(c["BLOCK_SIZE_M"] in (32, 64, 128, 256) for c in t.values())
    assert layers.get_moe_configs(7, 1234, None) is None
    assert layers.try_get_optimal_moe_config((7, 2468, 64), (7, 64, 1234), 2, 512) == \
        layers.get_default_config(512, 7, 1234, 64, 2)


def test_fused_experts_rejects_mixed_dtypes_and_packed_float32(ops, dev):
    """Activations and both weight tensors must share one of float32 / float16 / bfloat16; the packed
    layout is a 16-bit one."""
    from sarathi_amd import layers
    x = torch.zeros((4, 64), device=dev)
    w1, w2 = torch.zeros((2, 32, 64), device=dev), torch.zeros((2, 64, 16), device=dev)
    tw, ti = torch.ones((4, 1), device=dev), torch.zeros((4, 1), dtype=torch.int32, device=dev)
    with pytest.raises(TypeError, match="same dtype"):
        layers.fused_experts(x.half(), w1.half(), w2, tw, ti)
    with pytest.raises(TypeError, match="same dtype"):
        layers.fused_experts(x.double(), w1.double(), w2.double(), tw, ti)
    packed = layers.pack_expert_weights(w1.half())
    packed.dtype = torch.float32          # a 16-bit packing handed over as if it were float32
    with pytest.raises(TypeError, match="16-bit layout"):
        layers.fused_experts(x, packed, w2, tw, ti)


@pytest.mark.parametrize("T,E,k,BM,N,K,mul", [
    (300, 8, 2, 64, 512, 256, False),
    (300, 8, 2, 64, 512, 256, True),
    (77, 4, 2, 32, 260, 100, True),      # ragged N, K not a multiple of the 32-deep step
    (1000, 8, 2, 128, 768, 512, False),
    (40, 8, 2, 256, 300, 128, False),    # mostly padding
    (33, 16, 4, 32, 256, 64, True),      # some experts empty
    (5, 8, 1, 96, 1024, 192, False),     # a block size the 16-bit kernels do not have
])
def test_grouped_gemm_float32_matches_formulation(ops, dev, T, E, k, BM, N, K, mul):
    """float32 tensors: exact float32 products, float32 accumulation, output rounded through
    float16 as the reference's kernel does for every dtype but bfloat16 (fused_moe.py:142, 466).
    The accumulation order differs from the CPU matmul's (float32 sums of K products of size ~0.25
    differ by ~1e-6), so a result may land on the neighbouring float16 value: one float16 ulp of
    relative tolerance plus 1e-5 absolute, and every stored value must be a float16 value."""
    _, w, ids, s, e, p = _route(T, E, k, BM, T + N)
    g = gen(K)
    A = randn((T, K), g, torch.float32, std=0.5)
    Bw = randn((E, N, K), g, torch.float32, std=0.5)
    want = torch.zeros((T, k, N), dtype=torch.float32)
    torch_formulations.moe_grouped_gemm(A, Bw, want, w, s, e, p, T * k, BM, k, mul)
    got = torch.full((T, k, N), 7.0, dtype=torch.float32, device=dev)
    ops.moe_ops.moe_grouped_gemm(A.to(dev), Bw.to(dev), got, w.to(dev), s.to(dev), e.to(dev),
                                 p.to(dev), T * k, BM, k, mul)
    got = got.cpu()
    assert torch.equal(got, got.half().float())
    assert torch.allclose(got, want, rtol=2 ** -10, atol=1e-5)
    with pytest.raises(RuntimeError, match="float32"):
        ops.moe_ops.moe_grouped_gemm(A.to(dev), Bw.to(dev), got.to(dev), w.to(dev), s.to(dev), e.to(dev),
                                     p.to(dev), T * k, BM, k, False, False, 0, True)


def test_grouped_gemm_float32_identity_weights_exact(ops, dev):
    """One non-zero product per output: the gathered row itself, rounded through float16."""
    T, E, k, BM, K = 100, 4, 2, 64, 128
    _, w, ids, s, e, p = _route(T, E, k, BM, 5)
    A = randn((T, K), gen(6), torch.float32)
    Bw = torch.eye(K).repeat(E, 1, 1) * torch.arange(1, E + 1, dtype=torch.float32).view(E, 1, 1)
    got = torch.zeros((T, k, K), dtype=torch.float32, device=dev)
    ops.moe_ops.moe_grouped_gemm(A.to(dev), Bw.to(dev), got, w.to(dev), s.to(dev), e.to(dev),
                                 p.to(dev), T * k, BM, k, False)
    want = (A.unsqueeze(1) * (ids.float() + 1).unsqueeze(-1)).half().float()
    assert torch.equal(got.cpu(), want)


def test_fused_moe_float32_matches_dense_formulation(ops, dev):
    """The whole layer on float32 tensors (the reference admits them, fused_moe.py:430) against the
    dense formulation with the same float16 roundings of the two GEMM outputs."""
    from sarathi_amd import layers
    T, E, k, H, I = 300, 8, 2, 256, 384
    g = gen(91)
    x = randn((T, H), g, torch.float32, std=1.0)
    w1 = randn((E, 2 * I, H), g, torch.float32, std=H ** -0.5)
    w2 = randn((E, H, I), g, torch.float32, std=I ** -0.5)
    gating = torch.randn((T, E), generator=g, dtype=torch.float32)
    want = torch_formulations.fused_moe(x, w1, w2, gating, k, True)
    got = layers.fused_moe(x.to(dev), w1.to(dev), w2.to(dev), gating.to(dev), k, True)
    assert got.dtype == torch.float32
    assert torch.allclose(got.cpu(), want, rtol=4e-3, atol=4e-3 * want.abs().max().item())


@pytest.mark.parametrize("grouped", [False, True])
def test_fused_moe_module(ops, dev, grouped):
    """The FusedMoE module (weights as parameters, in-place forward) against the dense CPU
    formulation, with row-major and with packed weights."""
    from sarathi_amd import layers
    T, E, k, H, I = 200, 8, 2, 256, 512
    g = gen(31)
    layer = layers.FusedMoE(E, k, H, I, params_dtype=torch.bfloat16, renormalize=True,
                            use_grouped_topk=grouped, num_expert_group=4 if grouped else None,
                            topk_group=2 if grouped else None)
    assert layer.w13_weight.shape == (E, 2 * I, H) and layer.w2_weight.shape == (E, H, I)
    w1 = randn((E, 2 * I, H), g, std=H ** -0.5)
    w2 = randn((E, H, I), g, std=I ** -0.5)
    layer.w13_weight.data.copy_(w1)
    layer.w2_weight.data.copy_(w2)
    x = randn((T, H), g, std=1.0)
    logits = torch.randn((T, E), generator=g, dtype=torch.float32)
    if grouped:
        tw, ti = torch_formulations.grouped_topk(logits, k, True, 4, 2)
        want = torch_formulations.fused_moe(x, w1, w2, logits, k, True, topk_weights=tw, topk_ids=ti)
    else:
        want = torch_formulations.fused_moe(x, w1, w2, logits, k, True)
    xd = x.to(dev)
    out = layer(xd, logits.to(dev))
    assert out.data_ptr() == xd.data_ptr()
    _close(out, want, "FusedMoE")
    layer.pack_weights()
    out2 = layer(x.to(dev), logits.to(dev))
    assert torch.equal(out2, out)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("T,E,k,BM,I,K", [
    (300, 8, 2, 64, 256, 256),
    (1000, 8, 2, 128, 640, 128),     # I not a multiple of the 128 output columns of a workgroup
    (40, 4, 2, 256, 96, 64),
    (77, 4, 1, 32, 20, 64),          # I = 20: row-major only (packed tiles would straddle)
    (1500, 4, 2, 256, 2080, 64),     # enough workgroups for the four-wave kernel's 256-wide tiles
])
def test_gated_silu_epilogue_is_bit_identical_to_separate_kernels(ops, dev, dtype, T, E, k, BM, I, K):
    _, w, ids, s, e, p = _route(T, E, k, BM, T + I)
    g = gen(I)
    A = randn((T, K), g, dtype, std=0.5).to(dev)
    Bw = randn((E, 2 * I, K), g, dtype, std=0.5).to(dev)
    w, s, e, p = w.to(dev), s.to(dev), e.to(dev), p.to(dev)
    full = torch.zeros((T, k, 2 * I), dtype=dtype, device=dev)
    ops.moe_ops.moe_grouped_gemm(A, Bw, full, w, s, e, p, T * k, BM, k, False)
    want = torch.empty((T * k, I), dtype=dtype, device=dev)
    ops.activation_ops.silu_and_mul(want, full.view(-1, 2 * I))
    got = torch.full((T * k, I), 3.0, dtype=dtype, device=dev)
    ops.moe_ops.moe_grouped_gemm(A, Bw, got, w, s, e, p, T * k, BM, k, False, silu_and_mul=True)
    assert torch.equal(got, want)
    if I % 32 == 0:
        from sarathi_amd.layers import pack_expert_weights
        packed = pack_expert_weights(Bw)
        got2 = torch.full((T * k, I), 3.0, dtype=dtype, device=dev)
        ops.moe_ops.moe_grouped_gemm(A, packed.data, got2, w, s, e, p, T * k, BM, k, False, True,
                                     2 * I, True)
        assert torch.equal(got2, want)


# ---------------------------------------------------------------- riders

def _expected_riders(s, e, p, num_valid, bm):
    """What sarathi_moe_plan_riders documents, from moe_align_block_size's outputs (numpy-free,
    block by block)."""
    s, e = s.tolist(), e.tolist()
    live = min(int(p[0]), len(s)) // bm
    out = [-1] * ((len(s) + bm - 1) // bm)
    b = 0
    while b < live:
        last = b
        while last + 1 < live and e[last + 1] == e[b]:
            last += 1
        valid = sum(1 for x in s[last * bm:(last + 1) * bm] if x < num_valid)
        tiles = (valid + 31) // 32
        if last > b and tiles <= last - b:
            out[last] = -2
            for j in range(tiles):
                out[b + j] = last * bm + 32 * j
        b = last + 1
    return out


@pytest.mark.parametrize("T,E,k", [(1100, 4, 2), (1024, 8, 2), (2048, 8, 2), (4096, 8, 2), (300, 8, 2),
                                   (700, 2, 1), (5000, 16, 4)])
def test_moe_plan_riders_matches_its_definition(ops, dev, T, E, k):
    bm = 256
    _, _, _, s, e, p = _route(T, E, k, bm, 31 * T + E)
    want = _expected_riders(s, e, p, T * k, bm)
    got = torch.full((e.numel(),), 99, dtype=torch.int32, device=dev)
    ops.moe_ops.moe_plan_riders(s.to(dev), e.to(dev), p.to(dev), T * k, bm, got)
    assert got.cpu().tolist() == want
    if (T, E, k) in ((1100, 4, 2), (4096, 8, 2)):
        assert any(x >= 0 for x in want) and any(x == -2 for x in want)   # the case exercises riders


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("T,E,k,N,K", [
    (1100, 4, 2, 512, 256),     # 550 slots per expert: two full blocks and two tiles that ride
    (1040, 8, 2, 520, 128),     # one full block and a few slots per expert; ragged N
    (2100, 8, 2, 4104, 64),     # two K-stages only; 17 column blocks
    (300, 8, 2, 512, 256),      # nothing to ride (single blocks)
])
def test_grouped_gemm_with_riders_same_bits(ops, dev, dtype, T, E, k, N, K):
    """Row-major weights at 256-slot blocks: with the riders table the partly filled last blocks
    are multiplied by the workgroups of the full blocks; every output is formed from the same
    products in the same order, so all three epilogues give the same bits as without riders."""
    bm = 256
    _, w, ids, s, e, p = _route(T, E, k, bm, T + N)
    g = gen(K + T)
    A = randn((T, K), g, dtype, std=0.5).to(dev)
    Bw = randn((E, N, K), g, dtype, std=0.5).to(dev)
    sd, ed, pd, wd = s.to(dev), e.to(dev), p.to(dev), w.to(dev)
    riders = torch.empty((e.numel(),), dtype=torch.int32, device=dev)
    ops.moe_ops.moe_plan_riders(sd, ed, pd, T * k, bm, riders)
    for mul, silu in ((False, False), (True, False), (False, True)):
        cols = N // 2 if silu else N
        base = torch.full((T, k, cols), 7.0, dtype=dtype, device=dev)
        with_r = torch.full((T, k, cols), -3.0, dtype=dtype, device=dev)
        ops.moe_ops.moe_grouped_gemm(A, Bw, base, wd, sd, ed, pd, T * k, bm, k, mul, False, N, silu)
        ops.moe_ops.moe_grouped_gemm(A, Bw, with_r, wd, sd, ed, pd, T * k, bm, k, mul, False, N, silu,
                                     riders)
        assert torch.equal(with_r, base), (mul, silu)
    # the table is refused where the kernel that reads it does not run
    with pytest.raises(RuntimeError):
        ops.moe_ops.moe_grouped_gemm(A, Bw, base, wd, sd, ed, pd, T * k, 128, k, False, False, N, False,
                                     riders)


@pytest.mark.parametrize("loads", [
    (1024 + 33, 257, 0, 255, 512, 31),          # 2 tiles on 4 full blocks; 1 slot on one; exact blocks
    (8 * 256 + 255, 0, 0, 1),                   # a last block of eight tiles, all riding
    (8 * 256 + 256, 3 * 256 + 97, 2 * 256 + 65),  # no partial block; four tiles > three blocks; 3 > 2
    (256 + 32, 256 + 33, 512 + 64, 512 + 65),   # either side of the tile and block-count limits
])
def test_riders_with_chosen_expert_loads(ops, dev, loads):
    """Expert loads picked to sit on the limits of the plan (a tile more than there are full blocks,
    a last block that is full, empty experts, one slot): the table is the documented one and the
    GEMM has the same bits with it."""
    bm, E, N, K = 256, len(loads), 520, 192
    g = gen(sum(loads))
    order = torch.cat([torch.full((n,), x, dtype=torch.int32) for x, n in enumerate(loads)])
    ids = order[torch.randperm(order.numel(), generator=g)].view(-1, 1)
    T = ids.numel()
    n = T + E * (bm - 1)
    s = torch.full((n,), T, dtype=torch.int32)
    e = torch.zeros(((n + bm - 1) // bm,), dtype=torch.int32)
    p = torch.zeros((1,), dtype=torch.int32)
    c_oracle.moe_align_block_size(ids, E, bm, s, e, p)
    sd, ed, pd = s.to(dev), e.to(dev), p.to(dev)
    riders = torch.full((e.numel(),), 99, dtype=torch.int32, device=dev)
    ops.moe_ops.moe_plan_riders(sd, ed, pd, T, bm, riders)
    assert riders.cpu().tolist() == _expected_riders(s, e, p, T, bm)
    A = randn((T, K), g, torch.bfloat16, std=0.5).to(dev)
    Bw = randn((E, N, K), g, torch.bfloat16, std=0.5).to(dev)
    wd = torch.rand((T, 1), generator=g).to(dev)
    for mul, silu in ((True, False), (False, True)):
        cols = N // 2 if silu else N
        base = torch.full((T, 1, cols), 7.0, dtype=torch.bfloat16, device=dev)
        with_r = torch.full((T, 1, cols), -3.0, dtype=torch.bfloat16, device=dev)
        ops.moe_ops.moe_grouped_gemm(A, Bw, base, wd, sd, ed, pd, T, bm, 1, mul, False, N, silu)
        ops.moe_ops.moe_grouped_gemm(A, Bw, with_r, wd, sd, ed, pd, T, bm, 1, mul, False, N, silu, riders)
        assert torch.equal(with_r, base), (mul, silu)


def _expected_plan(s, e, p, num_valid, bm=256):
    """What sarathi_moe_plan_blocks documents: per expert, riders on the greedy layout, or the
    even fill over the two halves of each block and no riders."""
    s, e = s.tolist(), e.tolist()
    live = min(int(p[0]), len(s)) // bm
    out = list(s[:live * bm]) + [num_valid] * (len(s) - live * bm)
    ride = [-1] * ((len(s) + bm - 1) // bm)
    b = 0
    while b < live:
        last = b
        while last + 1 < live and e[last + 1] == e[b]:
            last += 1
        nb = last - b + 1
        slots = [x for x in s[b * bm:(last + 1) * bm] if x < num_valid]
        valid_last = len(slots) - (nb - 1) * bm
        tiles_last = (valid_last + 31) // 32
        if nb > 1 and tiles_last <= nb - 1:
            ride[last] = -2
            for j in range(tiles_last):
                ride[b + j] = last * bm + 32 * j
        else:
            tiles = (len(slots) + 31) // 32
            ranges = 2 * nb
            at = 0
            for j in range(ranges):
                mine = (tiles // ranges + (1 if j < tiles % ranges else 0)) * 32
                take = slots[at:at + mine]
                at += mine
                out[b * bm + j * 128:b * bm + (j + 1) * 128] = take + [num_valid] * (128 - len(take))
        b = last + 1
    return out, ride


@pytest.mark.parametrize("loads", [
    (1024 + 33, 257, 0, 255, 512, 31),
    (8 * 256 + 255, 0, 0, 1),
    (8 * 256 + 256, 3 * 256 + 97, 2 * 256 + 65),
    (256 + 32, 256 + 33, 512 + 64, 512 + 65),
    (640, 650, 630, 600, 700, 640, 1, 300),
])
def test_moe_plan_blocks_matches_its_definition_and_keeps_the_bits(ops, dev, loads):
    """moe_plan_blocks: riders for the experts whose last block fits onto their full blocks, the
    even fill for the others, in one launch; the GEMM on its outputs has the bits of the GEMM on
    moe_align_block_size's."""
    bm, E, N, K = 256, len(loads), 520, 192
    g = gen(sum(loads) + 1)
    order = torch.cat([torch.full((n,), x, dtype=torch.int32) for x, n in enumerate(loads)])
    ids = order[torch.randperm(order.numel(), generator=g)].view(-1, 1)
    T = ids.numel()
    n = T + E * (bm - 1)
    s = torch.full((n,), T, dtype=torch.int32)
    e = torch.zeros(((n + bm - 1) // bm,), dtype=torch.int32)
    p = torch.zeros((1,), dtype=torch.int32)
    c_oracle.moe_align_block_size(ids, E, bm, s, e, p)
    sd, ed, pd = s.to(dev), e.to(dev), p.to(dev)
    planned = torch.full_like(sd, -7)
    riders = torch.full((e.numel(),), 99, dtype=torch.int32, device=dev)
    ops.moe_ops.moe_plan_blocks(sd, planned, ed, pd, E, bm, T, riders)
    want_sorted, want_ride = _expected_plan(s, e, p, T)
    assert riders.cpu().tolist() == want_ride
    assert planned.cpu().tolist() == want_sorted
    A = randn((T, K), g, torch.bfloat16, std=0.5).to(dev)
    Bw = randn((E, N, K), g, torch.bfloat16, std=0.5).to(dev)
    wd = torch.rand((T, 1), generator=g).to(dev)
    for mul, silu in ((True, False), (False, True)):
        cols = N // 2 if silu else N
        base = torch.full((T, 1, cols), 7.0, dtype=torch.bfloat16, device=dev)
        got = torch.full((T, 1, cols), -3.0, dtype=torch.bfloat16, device=dev)
        ops.moe_ops.moe_grouped_gemm(A, Bw, base, wd, sd, ed, pd, T, bm, 1, mul, False, N, silu)
        ops.moe_ops.moe_grouped_gemm(A, Bw, got, wd, planned, ed, pd, T, bm, 1, mul, False, N, silu, riders)
        assert torch.equal(got, base), (mul, silu)


def test_fused_moe_same_bits_with_and_without_riders(ops, dev, monkeypatch):
    import importlib
    from sarathi_amd import layers
    fm = importlib.import_module("sarathi_amd.layers.fused_moe")   # the module, not the function
    T, E, k, H, I = 1100, 4, 2, 512, 1024
    g = gen(5)
    x = randn((T, H), g, torch.bfloat16, std=0.5).to(dev)
    w1 = randn((E, 2 * I, H), g, torch.bfloat16, std=0.05).to(dev)
    w2 = randn((E, H, I), g, torch.bfloat16, std=0.05).to(dev)
    logits = torch.randn((T, E), generator=g, dtype=torch.float32).to(dev)
    cfg = {"BLOCK_SIZE_M": 256}
    monkeypatch.setattr(fm, "RIDERS", False)
    base = layers.fused_moe(x, w1, w2, logits, k, True, override_config=cfg)
    monkeypatch.setattr(fm, "RIDERS", True)
    for even_rest in (False, True):
        monkeypatch.setattr(fm, "RIDERS_EVEN_REST", even_rest)
        got = layers.fused_moe(x, w1, w2, logits, k, True, override_config=cfg)
        assert torch.equal(got, base), even_rest


def test_fused_moe_commutes_with_a_permutation_of_the_tokens(ops, dev):
    """A token's output does not depend on where its slots land in the sorted layout (which block,
    which tile, riding or not): permuting the batch permutes the output, bit for bit, through
    routing, slot sort, block planning, both GEMMs and the top-k sum."""
    from sarathi_amd import layers
    T, E, k, H, I = 1500, 8, 2, 512, 768
    g = gen(77)
    x = randn((T, H), g, torch.bfloat16, std=0.5).to(dev)
    w1 = randn((E, 2 * I, H), g, torch.bfloat16, std=0.05).to(dev)
    w2 = randn((E, H, I), g, torch.bfloat16, std=0.05).to(dev)
    logits = torch.randn((T, E), generator=g, dtype=torch.float32).to(dev)
    perm = torch.randperm(T, generator=g).to(dev)
    for cfg in ({"BLOCK_SIZE_M": 256}, {"BLOCK_SIZE_M": 64}):
        out = layers.fused_moe(x, w1, w2, logits, k, True, override_config=cfg)
        out_p = layers.fused_moe(x[perm].contiguous(), w1, w2, logits[perm].contiguous(), k, True,
                                 override_config=cfg)
        assert torch.equal(out_p, out[perm]), cfg
