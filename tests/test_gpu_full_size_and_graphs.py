"""GPU: the benchmark configurations at their full sizes, checked against the oracle on a random
sample of token rows (every op here is per-token, so a row of the full-size output must equal the
oracle run on that row alone), and HIP-graph capture of the layer chain."""
import pytest
import torch

from helpers import (THETA_LLAMA3, assert_close_dtype, cos_sin_cache, gen, hybrid_positions, randn)
from oracle import c_oracle

pytestmark = pytest.mark.gpu


def _chain_gpu(ops, s):
    ops.layernorm_ops.fused_add_rms_norm(s["x"], s["res"], s["w1"], 1e-5)
    ops.pos_encoding_ops.rotary_embedding(s["pos"], s["q"], s["k"], s["D"], s["cache"], True)
    ops.activation_ops.silu_and_mul(s["act"], s["gate_up"])
    ops.layernorm_ops.fused_add_rms_norm(s["x"], s["res"], s["w2"], 1e-5)


def _make(T, prefill, H, nq, nkv, D, dff, seed, dev):
    """Device-side random inputs (the sampled rows are copied back for the oracle)."""
    torch.manual_seed(seed)
    g = gen(seed)
    bf = torch.bfloat16
    mk = lambda *shape: torch.randn(shape, device=dev, dtype=torch.float32).to(bf)  # noqa: E731
    s = {"D": D}
    s["x"], s["res"] = mk(T, H), mk(T, H)
    s["w1"] = randn((H,), g, mean=1.0, std=0.1).to(dev)
    s["w2"] = randn((H,), g, mean=1.0, std=0.1).to(dev)
    s["qkv"] = mk(T, (nq + 2 * nkv) * D)
    s["q"], s["k"], s["v"] = s["qkv"].split([nq * D, nkv * D, nkv * D], dim=-1)
    s["pos"] = hybrid_positions(T, prefill, g).to(dev)
    s["cache"] = cos_sin_cache(8192, D, THETA_LLAMA3, bf).to(dev)
    s["gate_up"] = mk(T, 2 * dff)
    s["act"] = torch.empty((T, dff), dtype=bf, device=dev)
    return s


@pytest.mark.parametrize("name,T,prefill,H,nq,nkv,D,dff", [
    ("llama3-8b hybrid batch", 2304, 2048, 4096, 32, 8, 128, 14336),
    ("llama3-70b chain", 4608, 4096, 8192, 64, 8, 128, 28672),
])
def test_full_size_chain_rows_match_oracle(ops, dev, name, T, prefill, H, nq, nkv, D, dff):
    s = _make(T, prefill, H, nq, nkv, D, dff, 4, dev)
    g = gen(5)
    rows = torch.cat((torch.tensor([0, prefill - 1, prefill, T - 1]),
                      torch.randint(0, T, (60,), generator=g))).unique()
    rd = rows.to(dev)
    # oracle on the sampled rows only (taken before the in-place ops run)
    ox, ores = s["x"][rd].cpu(), s["res"][rd].cpu()
    oqkv = s["qkv"][rd].cpu()
    ogu = s["gate_up"][rd].cpu()
    w1, w2, cache, pos = s["w1"].cpu(), s["w2"].cpu(), s["cache"].cpu(), s["pos"][rd].cpu()
    v_before = s["v"].clone()
    _chain_gpu(ops, s)
    torch.cuda.synchronize()

    c_oracle.fused_add_rms_norm(ox, ores, w1, 1e-5)
    oq, ok, _ = oqkv.split([nq * D, nkv * D, nkv * D], dim=-1)
    c_oracle.rotary_embedding(pos, oq, ok, D, cache, True)
    oact = torch.empty((rows.numel(), dff), dtype=torch.bfloat16)
    c_oracle.silu_and_mul(oact, ogu)
    x1 = ox.clone()                       # after the first norm
    c_oracle.fused_add_rms_norm(ox, ores, w2, 1e-5)

    assert torch.equal(s["qkv"][rd].cpu(), oqkv), name            # rope: bit-exact
    assert torch.equal(s["v"], v_before)                          # v part of the packed buffer untouched
    assert_close_dtype(s["act"][rd], oact)
    # the second fused norm consumed the first one's (tolerance-level) output, so compare it with
    # the oracle fed the oracle's own first-norm output: same tolerance, few extra flips
    assert_close_dtype(s["res"][rd], ores, max_mismatch_frac=2e-2)
    assert_close_dtype(s["x"][rd], ox, max_mismatch_frac=2e-2)
    del x1


def test_mixtral_routing_full_size(ops, dev):
    """Benchmark configuration 4: logits fp32 [4096, 8], top-2 (renormalised), align block 64."""
    g = gen(3)
    M, E, k, B = 4096, 8, 2, 64
    gating = torch.randn((M, E), generator=g, dtype=torch.float32)
    ww, wi, ws = torch.empty((M, k)), torch.empty((M, k), dtype=torch.int32), torch.empty((M, k), dtype=torch.int32)
    c_oracle.topk_softmax(ww, wi, ws, gating)
    gw = torch.empty((M, k), dtype=torch.float32, device=dev)
    gi = torch.empty((M, k), dtype=torch.int32, device=dev)
    gs = torch.empty((M, k), dtype=torch.int32, device=dev)
    ops.moe_ops.topk_softmax_renorm(gw, gi, gs, gating.to(dev))
    assert torch.equal(gi.cpu(), wi) and torch.equal(gs.cpu(), ws)
    assert torch.allclose(gw.cpu(), ww / ww.sum(-1, keepdim=True), rtol=0, atol=1e-6)
    n = M * k + E * (B - 1)
    sg = torch.empty((n,), dtype=torch.int32, device=dev)
    eg = torch.full(((n + B - 1) // B,), -1, dtype=torch.int32, device=dev)
    pg = torch.empty((1,), dtype=torch.int32, device=dev)
    ops.moe_ops.moe_align_block_size_filled(gi, E, B, sg, eg, pg)
    sw = torch.full((n,), M * k, dtype=torch.int32)
    ew = torch.full(((n + B - 1) // B,), -1, dtype=torch.int32)
    pw = torch.zeros((1,), dtype=torch.int32)
    c_oracle.moe_align_block_size(wi, E, B, sw, ew, pw)
    nb = int(pw.item()) // B
    assert n == 8696 and eg.numel() == 136
    assert torch.equal(sg.cpu(), sw) and torch.equal(pg.cpu(), pw) and torch.equal(eg.cpu()[:nb], ew[:nb])
    assert bool((eg.cpu()[nb:] == -1).all())


def test_chain_and_routing_under_hip_graph_capture(ops, dev):
    """The ops allocate nothing and launch fixed shapes, so a captured graph replays them.  Each
    replay is checked against an eager run on the same inputs, with eager work and synchronisation
    between the replays."""
    T, H, nq, nkv, D, dff = 512, 4096, 32, 8, 128, 14336
    s = _make(T, 448, H, nq, nkv, D, dff, 6, dev)
    M, E, k, B = 1024, 8, 2, 64
    g = gen(7)
    gating = torch.randn((M, E), generator=g, dtype=torch.float32).to(dev)
    tw = torch.empty((M, k), dtype=torch.float32, device=dev)
    ti = torch.empty((M, k), dtype=torch.int32, device=dev)
    ts = torch.empty((M, k), dtype=torch.int32, device=dev)
    n = M * k + E * (B - 1)
    sg = torch.empty((n,), dtype=torch.int32, device=dev)
    eg = torch.zeros(((n + B - 1) // B,), dtype=torch.int32, device=dev)
    pg = torch.empty((1,), dtype=torch.int32, device=dev)
    keys = ("x", "res", "qkv", "gate_up")
    init = {kk: s[kk].clone() for kk in keys}

    def run_all():
        _chain_gpu(ops, s)
        ops.moe_ops.topk_softmax(tw, ti, ts, gating)
        ops.moe_ops.moe_align_block_size_filled(ti, E, B, sg, eg, pg)

    def reset():
        for kk in keys:
            s[kk].copy_(init[kk])

    def snapshot():
        return [t.clone() for t in (s["x"], s["res"], s["qkv"], s["act"], tw, ti, ts, sg, eg, pg)]

    reset()
    run_all()
    torch.cuda.synchronize()
    want = snapshot()

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):          # warm-up on the capture stream, as torch requires
        reset()
        run_all()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    reset()
    torch.cuda.synchronize()
    with torch.cuda.graph(graph):
        run_all()
    for it in range(4):
        reset()
        for t in (s["act"], tw, sg):
            t.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got = snapshot()
        for a, b in zip(got, want):
            assert torch.equal(a, b), "replay %d differs from the eager run" % it
        # unrelated eager work between replays
        _ = (s["gate_up"].float().sum() + gating.sum()).item()


def test_kv_append_routing_and_expert_gemm_under_hip_graph_capture(ops, dev):
    """The rotary + KV-append fusion, the one-launch routing kernel (whose completion counter must be
    back at zero after every replay) and the grouped GEMM with both epilogues, captured once and
    replayed with eager work in between; every replay equals the eager run."""
    import numpy as np
    from sarathi_amd import layers
    T, nq, nkv, D, page = 300, 8, 2, 128, 16
    rng = np.random.default_rng(1)
    lens = [(True, 200, 260)] + [(False, 1, int(c)) for c in rng.integers(1, 90, size=100)]
    need = [(t + page - 1) // page for _, _, t in lens]
    perm = rng.permutation(sum(need))
    seqs, at = [], 0
    for (is_p, new, tot), n_pages in zip(lens, need):
        seqs.append(layers.SequenceSlice(is_p, new, tot, perm[at:at + n_pages].tolist()))
        at += n_pages
    meta = layers.build_append_metadata(seqs, page, dev)
    assert meta.num_total_tokens == T
    g = gen(11)
    qkv0 = randn((T, (nq + 2 * nkv) * D), g).to(dev)
    qkv = qkv0.clone()
    q, k, v = qkv.split([nq * D, nkv * D, nkv * D], dim=-1)
    table = cos_sin_cache(4096, D, THETA_LLAMA3, torch.bfloat16).to(dev)
    positions = meta.append_positions.long()
    kv_cache = torch.zeros((sum(need), 2, page, nkv, D), dtype=torch.bfloat16, device=dev)

    M, E, topk, B, H, I = 256, 8, 2, 64, 256, 512
    x = randn((M, H), g).to(dev)
    w1 = randn((E, 2 * I, H), g, std=H ** -0.5).to(dev)
    w2 = layers.pack_expert_weights(randn((E, H, I), g, std=I ** -0.5).to(dev))
    gating = torch.randn((M, E), generator=g, dtype=torch.float32).to(dev)
    tw = torch.empty((M, topk), dtype=torch.float32, device=dev)
    ti = torch.empty((M, topk), dtype=torch.int32, device=dev)
    ts = torch.empty((M, topk), dtype=torch.int32, device=dev)
    n = M * topk + E * (B - 1)
    sg = torch.empty((n,), dtype=torch.int32, device=dev)
    eg = torch.zeros(((n + B - 1) // B,), dtype=torch.int32, device=dev)
    pg = torch.empty((1,), dtype=torch.int32, device=dev)
    act = torch.empty((M * topk, I), dtype=torch.bfloat16, device=dev)
    down = torch.empty((M, topk, H), dtype=torch.bfloat16, device=dev)

    def run_all():
        ops.kv_cache_ops.rotary_embedding_append_paged_kv(
            positions, q, k, v, D, table, True, meta.append_batch_indices, meta.append_positions,
            kv_cache, meta.append_kv_page_indices, meta.append_kv_page_indptr,
            slot_mapping=meta.slot_mapping)
        ops.moe_ops.fused_topk_align(tw, ti, ts, gating, True, B, sg, eg, pg, True)
        ops.moe_ops.moe_grouped_gemm(x, w1, act, tw, sg, eg, pg, M * topk, B, topk, False,
                                     silu_and_mul=True)
        ops.moe_ops.moe_grouped_gemm(act, w2.data, down, tw, sg, eg, pg, M * topk, B, 1, True, True, H)

    outs = (qkv, kv_cache, tw, ti, ts, sg, eg, pg, act, down)

    def reset():
        qkv.copy_(qkv0)
        for t in (kv_cache, tw, sg, act, down):
            t.zero_()

    reset()
    run_all()
    torch.cuda.synchronize()
    want = [t.clone() for t in outs]

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        reset()
        run_all()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    reset()
    torch.cuda.synchronize()
    with torch.cuda.graph(graph):
        run_all()
    for it in range(4):
        reset()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for a, b in zip(outs, want):
            assert torch.equal(a, b), "replay %d differs from the eager run" % it
        _ = (x.float().sum() + gating.sum()).item()


def test_mixtral_expert_gemms_full_size(ops, dev):
    """The grouped expert GEMMs at the Mixtral-8x7B layer's real shape (4096 tokens, 8 experts,
    top-2, hidden 4096, intermediate 14336), where a CPU formulation of the whole product would take
    minutes.  Size-independent checks: (1) the two weight layouts run two different kernels (four
    waves with both operands through LDS; eight waves with the weights straight into registers)
    that form every output from the same products in the same order, so their results must agree
    bit for bit; (2) doubling the activations doubles every output exactly (power-of-two scaling
    commutes with every rounding as long as nothing overflows); (3) a random sample of outputs
    against float64 dot products of the gathered rows; (4) the gated epilogue against the separate
    activation kernel; (5) the kernel with riders on slot blocks planned per expert against (1)
    and (4), bit for bit."""
    from sarathi_amd import layers
    T, E, k, H, I = 4096, 8, 2, 4096, 14336
    bf = torch.bfloat16
    torch.manual_seed(11)
    x = torch.randn((T, H), device=dev, dtype=torch.float32).to(bf)
    w1 = (torch.randn((E, 2 * I, H), device=dev, dtype=torch.float32) * H ** -0.5).to(bf)
    gating = torch.randn((T, E), device=dev, dtype=torch.float32)
    tw, ti = layers.fused_topk(x, gating, k, True)
    config = dict(layers.try_get_optimal_moe_config((E, 2 * I, H), (E, H, I), k, T, packed=False))
    bm = config["BLOCK_SIZE_M"]
    s, e, p = layers.moe_align_block_size(ti, bm, E)

    def run(a, b, packed, gated):
        c = torch.full((T * k, I if gated else 2 * I), 3.0, device=dev, dtype=bf)
        ops.moe_ops.moe_grouped_gemm(a, b, c, tw, s, e, p, T * k, bm, k, False, packed, 2 * I, gated)
        return c

    plain = run(x, w1, False, False)
    packed_w1 = layers.pack_expert_weights(w1).data
    assert torch.equal(run(x, packed_w1, True, False), plain)            # (1)
    assert torch.equal(run(x * 2, w1, False, False), plain * 2)          # (2)
    # (3) 256 sampled outputs
    g = gen(12)
    slots = torch.randint(0, T * k, (256,), generator=g)
    cols = torch.randint(0, 2 * I, (256,), generator=g)
    xs = x[(slots // k).to(dev)].double().cpu()
    experts = ti.flatten()[slots.to(dev)].long()
    ws = w1[experts, cols.to(dev)].double().cpu()
    want = (xs * ws).sum(-1)
    got = plain[slots.to(dev), cols.to(dev)].double().cpu()
    assert bool(((got - want).abs() <= 1e-2 * want.abs() + 1e-2).all()), (got - want).abs().max()
    # (4)
    act = torch.empty((T * k, I), device=dev, dtype=bf)
    ops.activation_ops.silu_and_mul(act, plain)
    assert torch.equal(run(x, w1, False, True), act)
    assert torch.equal(run(x, packed_w1, True, True), act)
    # (5) slot blocks planned per expert (riders, even fill): same bits, both epilogues
    if bm == 256:
        planned = torch.empty_like(s)
        riders = torch.empty((e.numel(),), dtype=torch.int32, device=dev)
        ops.moe_ops.moe_plan_blocks(s, planned, e, p, E, bm, T * k, riders)
        assert bool((riders >= 0).any()), "this routing has tiles that ride"
        for gated, want_c in ((False, plain), (True, act)):
            c = torch.full_like(want_c, 3.0)
            ops.moe_ops.moe_grouped_gemm(x, w1, c, tw, planned, e, p, T * k, bm, k, False, False, 2 * I,
                                         gated, riders)
            assert torch.equal(c, want_c), gated


def test_fused_moe_with_riders_under_hip_graph_capture(ops, dev, monkeypatch):
    """The riders table is planned on the device from the batch's own routing: a captured
    fused_moe replayed on new activations and router logits (other expert loads, other riders)
    equals the eager layer without riders, bit for bit, on every replay."""
    import importlib
    from sarathi_amd import layers
    fm = importlib.import_module("sarathi_amd.layers.fused_moe")   # the module, not the function
    T, E, k, H, I = 1100, 4, 2, 256, 512
    cfg = {"BLOCK_SIZE_M": 256}
    g = gen(23)
    w1 = randn((E, 2 * I, H), g, std=H ** -0.5).to(dev)
    w2 = randn((E, H, I), g, std=I ** -0.5).to(dev)
    batches = []
    for i in range(4):
        x = randn((T, H), g, std=0.5).to(dev)
        logits = torch.randn((T, E), generator=g, dtype=torch.float32)
        logits[:, i % E] += 0.4 * i          # shift the loads: other blocks end up short
        batches.append((x, logits.to(dev)))
    monkeypatch.setattr(fm, "RIDERS", False)
    want = [layers.fused_moe(x, w1, w2, lg, k, True, override_config=cfg) for x, lg in batches]
    monkeypatch.setattr(fm, "RIDERS", True)
    xs, ls = batches[0][0].clone(), batches[0][1].clone()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        layers.fused_moe(xs, w1, w2, ls, k, True, override_config=cfg)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = layers.fused_moe(xs, w1, w2, ls, k, True, override_config=cfg)
    for (x, lg), expect in zip(batches + batches[:1], want + want[:1]):
        xs.copy_(x)
        ls.copy_(lg)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, expect)
        _ = (x.float().sum() + lg.sum()).item()
