"""GPU parity of MoE routing (topk_softmax, moe_align_block_size) against the CPU oracle.

Indices, sorted_token_ids, expert_ids (valid prefix) and num_tokens_post_pad must be bit-exact;
softmax weights are compared to 1e-6 (the device and host expf differ in the last place).
"""
import json
import os

import pytest
import torch

from helpers import gen
from oracle import c_oracle

pytestmark = pytest.mark.gpu

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden",
                      "moe_align_block_size_vectors.json")


def _topk_gpu(ops, dev, gating, k, renorm=False):
    T = gating.shape[0]
    w = torch.empty((T, k), dtype=torch.float32, device=dev)
    idx = torch.empty((T, k), dtype=torch.int32, device=dev)
    src = torch.empty((T, k), dtype=torch.int32, device=dev)
    fn = ops.moe_ops.topk_softmax_renorm if renorm else ops.moe_ops.topk_softmax
    fn(w, idx, src, gating.to(dev))
    return w.cpu(), idx.cpu(), src.cpu()


def _topk_oracle(gating, k):
    T = gating.shape[0]
    w = torch.empty((T, k), dtype=torch.float32)
    idx = torch.empty((T, k), dtype=torch.int32)
    src = torch.empty((T, k), dtype=torch.int32)
    c_oracle.topk_softmax(w, idx, src, gating)
    return w, idx, src


def _assert_separated(gating, k):
    """Indices are only well defined across expf implementations when the k+1 largest logits of
    every row are distinct by more than rounding noise; assert it for the seeded input."""
    top = torch.sort(gating, dim=-1, descending=True).values[:, : k + 1]
    if top.shape[1] > 1:
        assert (top[:, :-1] - top[:, 1:]).min().item() > 1e-6


@pytest.mark.parametrize("E,k", [(8, 2), (1, 1), (2, 1), (2, 2), (4, 2), (16, 4), (32, 5), (64, 6),
                                 (128, 8), (256, 8), (8, 8), (60, 4), (6, 2), (100, 3), (384, 8),
                                 (1000, 2)])
def test_topk_softmax_matches_oracle(ops, dev, E, k):
    g = gen(3)
    T = 4096 if E == 8 else 515
    gating = torch.randn((T, E), generator=g, dtype=torch.float32)
    _assert_separated(gating, min(k, E - 1))
    ww, wi, ws = _topk_oracle(gating, k)
    gw, gi, gs = _topk_gpu(ops, dev, gating, k)
    assert torch.equal(gi, wi)
    assert torch.equal(gs, ws)
    assert torch.allclose(gw, ww, rtol=0, atol=1e-6)


def test_topk_softmax_ties_and_collapsed_probabilities(ops, dev):
    """Equal logits: lower expert index first.  Logits so far below the maximum that their
    probabilities are exactly 0 tie at 0 and are also taken in index order (the reference compares
    probabilities, not logits)."""
    rows = torch.tensor([
        [1.0] * 8,
        [0.0, 5.0, 5.0, 0.0, 5.0, 0.0, 0.0, 0.0],
        [0.0, -300.0, -200.0, -250.0, -400.0, -210.0, -220.0, -230.0],
        [-1e4, -1e4, 3.0, -1e4, -1e4, -1e4, -1e4, -2e4],
    ], dtype=torch.float32)
    ww, wi, ws = _topk_oracle(rows, 3)
    gw, gi, gs = _topk_gpu(ops, dev, rows, 3)
    assert wi.tolist() == [[0, 1, 2], [1, 2, 4], [0, 1, 2], [2, 0, 1]]
    assert torch.equal(gi, wi) and torch.equal(gs, ws)
    assert torch.allclose(gw, ww, rtol=0, atol=1e-6)


def test_topk_softmax_renorm_equals_caller_side_division(ops, dev):
    g = gen(3)
    gating = torch.randn((4096, 8), generator=g, dtype=torch.float32)
    w, i, _ = _topk_gpu(ops, dev, gating, 2)
    wr, ir, _ = _topk_gpu(ops, dev, gating, 2, renorm=True)
    assert torch.equal(i, ir)
    assert torch.equal(wr, w / w.sum(dim=-1, keepdim=True))   # same fp32 add and divide


def _align_bufs(numel, E, B, device, fill=True):
    n = numel + E * (B - 1)
    s = torch.empty((n,), dtype=torch.int32, device=device)
    s.fill_(numel if fill else -7)
    e = torch.full(((n + B - 1) // B,), -1, dtype=torch.int32, device=device)
    p = torch.full((1,), -1, dtype=torch.int32, device=device)
    return s, e, p


def _align_both(ops, dev, ids, E, B, filled=False):
    ws, we, wp = _align_bufs(ids.numel(), E, B, "cpu")
    c_oracle.moe_align_block_size(ids, E, B, ws, we, wp)
    gs, ge, gp = _align_bufs(ids.numel(), E, B, dev, fill=not filled)
    fn = ops.moe_ops.moe_align_block_size_filled if filled else ops.moe_ops.moe_align_block_size
    fn(ids.to(dev), E, B, gs, ge, gp)
    return (gs.cpu(), ge.cpu(), gp.cpu()), (ws, we, wp)


def _check_align(got, want, B):
    (gs, ge, gp), (ws, we, wp) = got, want
    assert torch.equal(gp, wp)
    assert torch.equal(gs, ws)                       # full length, padding slots included
    nblk = int(wp.item()) // B
    assert torch.equal(ge[:nblk], we[:nblk])
    assert bool((ge[nblk:] == -1).all())             # entries past the valid prefix untouched


def test_moe_align_reference_vectors(ops, dev):
    with open(GOLDEN) as f:
        vectors = json.load(f)["vectors"]
    for v in vectors:
        ids = torch.tensor(v["topk_ids"], dtype=torch.int32)
        E, B = v["num_experts"], v["block_size"]
        for filled in (False, True):
            gs, ge, gp = _align_bufs(ids.numel(), E, B, dev, fill=not filled)
            fn = (ops.moe_ops.moe_align_block_size_filled if filled
                  else ops.moe_ops.moe_align_block_size)
            fn(ids.to(dev), E, B, gs, ge, gp)
            n = v["num_tokens_post_pad"]
            assert gp.item() == n
            assert gs.cpu()[:n].tolist() == v["sorted_token_ids_prefix"]
            assert bool((gs.cpu()[n:] == ids.numel()).all())
            assert ge.cpu()[: n // B].tolist() == v["expert_ids_prefix"]


@pytest.mark.parametrize("filled", [False, True])
@pytest.mark.parametrize("T,k,E,B", [(4096, 2, 8, 64), (4096, 2, 8, 16), (4096, 2, 8, 128),
                                     (1, 1, 8, 64), (7, 2, 8, 32), (63, 1, 4, 4), (64, 1, 4, 4),
                                     (65, 3, 16, 1), (1000, 6, 64, 16), (3000, 8, 256, 32),
                                     (500, 4, 1000, 8), (70000, 2, 8, 64), (16384, 4, 60, 128),
                                     (8193, 2, 8, 64), (30000, 4, 1000, 8), (65536, 8, 256, 16),
                                     (16000, 2, 8, 64), (16384, 2, 32, 16), (5461, 6, 64, 32),
                                     (257, 1, 17, 4), (300, 1, 2, 1)])
def test_moe_align_matches_oracle(ops, dev, T, k, E, B, filled):
    g = gen(T + E)
    ids = torch.randint(0, E, (T, k), generator=g, dtype=torch.int32)
    _check_align(*_align_both(ops, dev, ids, E, B, filled), B)


def test_moe_align_from_config4_topk(ops, dev):
    """Mixtral-shaped routing end to end: logits [4096, 8] -> top-2 -> align with block 64."""
    g = gen(3)
    gating = torch.randn((4096, 8), generator=g, dtype=torch.float32)
    _, ids, _ = _topk_gpu(ops, dev, gating, 2)
    _, want_ids, _ = _topk_oracle(gating, 2)
    assert torch.equal(ids, want_ids)
    got, want = _align_both(ops, dev, ids, 8, 64)
    _check_align(got, want, 64)
    assert got[0].numel() == 8696 and got[1].numel() == 136


@pytest.mark.parametrize("dtype", [torch.uint8, torch.int8, torch.int16, torch.int32, torch.int64])
def test_moe_align_id_dtypes(ops, dev, dtype):
    g = gen(11)
    ids = torch.randint(0, 100, (777, 2), generator=g, dtype=torch.int32).to(dtype)
    _check_align(*_align_both(ops, dev, ids, 100, 16), 16)


def test_moe_align_skewed_and_empty(ops, dev):
    # everything on one expert; some experts empty; empty input
    ids = torch.full((5000,), 3, dtype=torch.int32)
    _check_align(*_align_both(ops, dev, ids, 8, 64), 64)
    ids = torch.tensor([7, 7, 0, 7, 0], dtype=torch.int32)
    _check_align(*_align_both(ops, dev, ids, 8, 4, filled=True), 4)
    ids = torch.empty((0,), dtype=torch.int32)
    _check_align(*_align_both(ops, dev, ids, 8, 4, filled=True), 4)


@pytest.mark.parametrize("E", [8, 32])
@pytest.mark.parametrize("dtype", [torch.int32, torch.int64, torch.int8])
def test_moe_align_largest_one_launch_input_on_one_expert(ops, dev, E, dtype):
    """32768 ids, the largest input of the one-launch kernels, all on ONE expert: every per-lane
    byte counter and every 16-bit wave total of the few-experts kernel reaches its maximum."""
    for expert in (0, E - 1):
        ids = torch.full((32768,), expert, dtype=dtype)
        _check_align(*_align_both(ops, dev, ids, E, 64, filled=True), 64)
    ids = torch.full((32768,), 5, dtype=dtype)
    ids[::977] = 2                          # a few strays so that two runs exist
    _check_align(*_align_both(ops, dev, ids, E, 16), 16)


@pytest.mark.parametrize("dtype", [torch.int32, torch.int16, torch.int8])
@pytest.mark.parametrize("E", [2, 8, 32])
def test_moe_align_id_pointer_not_16_byte_aligned(ops, dev, E, dtype):
    """The id array may start anywhere: a view that begins one element into its buffer (4, 2 or 1
    bytes off a 16-byte boundary) takes the kernels without 16-byte id loads and gives the same
    result, at sizes on both sides of every launch-shape boundary."""
    g = gen(31 + E)
    for numel in (300, 5000, 32767):
        buf = torch.randint(0, E, (numel + 1,), generator=g, dtype=torch.int32).to(dtype)
        ids_cpu = buf[1:].clone()
        ids_dev = buf.to(dev)[1:]
        assert ids_dev.data_ptr() % 16 != 0
        ws, we, wp = _align_bufs(numel, E, 32, "cpu")
        c_oracle.moe_align_block_size(ids_cpu, E, 32, ws, we, wp)
        gs, ge, gp = _align_bufs(numel, E, 32, dev, fill=False)
        ops.moe_ops.moe_align_block_size_filled(ids_dev, E, 32, gs, ge, gp)
        _check_align((gs.cpu(), ge.cpu(), gp.cpu()), (ws, we, wp), 32)


def test_moe_align_invariants_large(ops, dev):
    """64K tokens x top-2 (the largest chunk the reference's caller passes, fused_moe.py:437):
    non-padding entries are a permutation of 0..numel-1, each block holds one expert's tokens in
    ascending order, post_pad = sum ceil(cnt/B)*B."""
    g = gen(12)
    T, k, E, B = 65536, 2, 8, 64
    ids = torch.randint(0, E, (T, k), generator=g, dtype=torch.int32)
    gs, ge, gp = _align_bufs(T * k, E, B, dev, fill=False)
    ops.moe_ops.moe_align_block_size_filled(ids.to(dev), E, B, gs, ge, gp)
    gs, ge, n = gs.cpu(), ge.cpu(), int(gp.item())
    flat = ids.reshape(-1)
    cnt = torch.bincount(flat.long(), minlength=E)
    assert n == int(((cnt + B - 1) // B * B).sum()) and n % B == 0
    real = gs[:n][gs[:n] != T * k]
    assert torch.equal(torch.sort(real).values, torch.arange(T * k, dtype=torch.int32))
    blocks = gs[:n].view(-1, B)
    for b in range(blocks.shape[0]):
        row = blocks[b][blocks[b] != T * k].long()
        assert bool((flat[row] == ge[b]).all())
        assert bool((row[1:] > row[:-1]).all())
    assert bool((gs[n:] == T * k).all())


def test_moe_align_workspace_is_optional(ops, dev):
    """Straight through the C ABI: with no workspace a large input takes the single-workgroup
    kernel, with one it takes the three-launch path; both give the oracle's result."""
    import ctypes
    import os
    lib = ctypes.CDLL(os.path.join(os.path.dirname(ops.__file__), "lib", "libsarathi_ops_hip.so"))
    lib.sarathi_moe_align_workspace_bytes.restype = ctypes.c_int64
    g = gen(13)
    T, k, E, B = 40000, 2, 64, 32
    ids = torch.randint(0, E, (T, k), generator=g, dtype=torch.int32)
    ws, we, wp = _align_bufs(ids.numel(), E, B, "cpu")
    c_oracle.moe_align_block_size(ids, E, B, ws, we, wp)
    need = lib.sarathi_moe_align_workspace_bytes(ctypes.c_int64(ids.numel()), ctypes.c_int(E))
    assert need > 0
    ids_d = ids.to(dev)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    for ws_bytes in (0, need // 2, need):
        scratch = torch.empty((max(ws_bytes, 4) // 4,), dtype=torch.int32, device=dev)
        gs, ge, gp = _align_bufs(ids.numel(), E, B, dev, fill=False)
        rc = lib.sarathi_moe_align_block_size(
            ctypes.c_void_p(ids_d.data_ptr()), ctypes.c_int(3), ctypes.c_int64(ids.numel()),
            ctypes.c_int(E), ctypes.c_int(B), ctypes.c_void_p(gs.data_ptr()),
            ctypes.c_int64(gs.numel()), ctypes.c_void_p(ge.data_ptr()), ctypes.c_int64(ge.numel()),
            ctypes.c_void_p(gp.data_ptr()), ctypes.c_int(1),
            ctypes.c_void_p(scratch.data_ptr() if ws_bytes else None), ctypes.c_int64(ws_bytes),
            stream)
        assert rc == 0
        torch.cuda.synchronize()
        _check_align((gs.cpu(), ge.cpu(), gp.cpu()), (ws, we, wp), B)


# ---- topk_softmax + moe_align_block_size in one launch -------------------------------------------

def _separate(ops, dev, gating, k, renorm, E, B):
    T = gating.shape[0]
    w = torch.empty((T, k), dtype=torch.float32, device=dev)
    idx = torch.empty((T, k), dtype=torch.int32, device=dev)
    src = torch.empty((T, k), dtype=torch.int32, device=dev)
    (ops.moe_ops.topk_softmax_renorm if renorm else ops.moe_ops.topk_softmax)(w, idx, src, gating)
    n = T * k + E * (B - 1)
    s = torch.full((n,), -5, dtype=torch.int32, device=dev)
    e = torch.full(((n + B - 1) // B,), -5, dtype=torch.int32, device=dev)
    p = torch.full((1,), -5, dtype=torch.int32, device=dev)
    ops.moe_ops.moe_align_block_size_filled(idx, E, B, s, e, p)
    return w, idx, src, s, e, p


@pytest.mark.parametrize("T,E,k,B,renorm", [
    (4096, 8, 2, 64, True),        # Mixtral routing of the benchmark batch: two launches
    (512, 8, 2, 64, True),         # 1024 slots: the largest case that runs as ONE launch
    (513, 8, 2, 128, False),       # one token too many: two launches, same results
    (1, 8, 2, 16, True),           # a single token: one workgroup, which is also the last one
    (17, 2, 1, 4, False),
    (170, 16, 6, 32, True),        # several workgroups, ragged last row block
    (256, 16, 4, 64, True),
    (100, 32, 4, 16, False),       # more than 16 experts: two launches
    (700, 60, 4, 32, False),       # expert count not a power of two: two launches
])
def test_fused_topk_align_equals_separate_ops(ops, dev, T, E, k, B, renorm):
    """Several calls on the same output buffers with different logits: the completion counter must
    be back at zero after every call, and the sorting workgroup must see the ids of THIS call,
    not lines cached from the previous one."""
    n = T * k + E * (B - 1)
    w = torch.empty((T, k), dtype=torch.float32, device=dev)
    idx = torch.empty((T, k), dtype=torch.int32, device=dev)
    src = torch.empty((T, k), dtype=torch.int32, device=dev)
    s = torch.empty((n,), dtype=torch.int32, device=dev)
    e = torch.empty(((n + B - 1) // B,), dtype=torch.int32, device=dev)
    p = torch.empty((1,), dtype=torch.int32, device=dev)
    for rep in range(4):
        gating = torch.randn((T, E), generator=gen(T + E + 1000 * rep), dtype=torch.float32).to(dev)
        want = _separate(ops, dev, gating, k, renorm, E, B)
        s.fill_(-5)
        e.fill_(-5)
        ops.moe_ops.fused_topk_align(w, idx, src, gating, renorm, B, s, e, p, True)
        for got, exp, name in zip((w, idx, src, s, e, p), want,
                                  ("weights", "ids", "source", "sorted", "expert_ids", "post_pad")):
            assert torch.equal(got, exp), "%s differ on call %d" % (name, rep)


def test_fused_topk_align_against_oracle(ops, dev):
    """The one-launch path against the CPU oracle directly (not only against the other kernels)."""
    T, E, k, B = 500, 8, 2, 64
    gating = torch.randn((T, E), generator=gen(77), dtype=torch.float32)
    _assert_separated(gating, k)
    ww, wi, ws = _topk_oracle(gating, k)
    n = T * k + E * (B - 1)
    os_ = torch.full((n,), T * k, dtype=torch.int32)
    oe = torch.zeros(((n + B - 1) // B,), dtype=torch.int32)
    op = torch.zeros((1,), dtype=torch.int32)
    c_oracle.moe_align_block_size(wi, E, B, os_, oe, op)
    from sarathi_amd import layers
    w, idx, s, e, p = layers.fused_topk_and_align(torch.empty((T, 4), device=dev), gating.to(dev), k,
                                                  False, B)
    assert torch.equal(idx.cpu(), wi) and torch.allclose(w.cpu(), ww, rtol=0, atol=1e-6)
    assert int(p.item()) == int(op.item())
    assert torch.equal(s.cpu(), os_)
    nb = int(op.item()) // B
    assert torch.equal(e.cpu()[:nb], oe[:nb])


# ---- grouped_topk -----------------------------------------------------------------------------------

@pytest.mark.parametrize("T,E,k,G,keep,renorm", [
    (257, 160, 6, 8, 3, True),       # DeepSeek-V2
    (64, 16, 4, 1, 1, False),        # one group: plain top-k
    (100, 64, 8, 64, 8, False),      # groups of one expert
    (33, 256, 8, 8, 4, True),
    (50, 1024, 4, 32, 2, False),
    (7, 6, 3, 3, 2, True),
])
def test_grouped_topk_matches_formulation(ops, dev, T, E, k, G, keep, renorm):
    from oracle import torch_formulations
    from sarathi_amd import layers
    gating = torch.randn((T, E), generator=gen(E + k), dtype=torch.float32)
    ww, wi = torch_formulations.grouped_topk(gating, k, renorm, G, keep)
    gw, gi = layers.grouped_topk(torch.empty((T, 4), device=dev), gating.to(dev), k, renorm, G, keep)
    assert gi.dtype == torch.int32 and gw.dtype == torch.float32
    assert torch.equal(gi.cpu(), wi)
    assert torch.allclose(gw.cpu(), ww, rtol=0, atol=1e-6)


@pytest.mark.parametrize("rows", [1, 2])
@pytest.mark.parametrize("numel,E,B", [(8192, 8, 256), (8192, 8, 64), (2000, 8, 128), (40000, 64, 256),
                                       (300, 4, 64), (5, 8, 64), (9000, 3, 256), (1024, 1, 256)])
def test_moe_balance_blocks_spreads_every_expert_evenly(ops, dev, numel, E, B, rows):
    """moe_balance_blocks on moe_align_block_size's output against the direct construction from
    the ids (oracle.torch_formulations.moe_balance_blocks): same blocks per expert, an expert's
    slots in unchanged order spread over them (or over the two halves of each) in multiples of the
    GEMM's 32-slot tile, padding elsewhere and beyond num_tokens_post_pad; skewed and empty experts
    included."""
    from oracle import torch_formulations as tf
    g = gen(numel + E)
    ids = torch.randint(0, E, (numel,), generator=g, dtype=torch.int32)
    if E > 2:
        ids[ids == 1] = 0                      # an empty expert and an overfull one
    gs, ge, gp = _align_bufs(numel, E, B, dev, fill=False)
    ops.moe_ops.moe_align_block_size_filled(ids.to(dev), E, B, gs, ge, gp)
    out = torch.full_like(gs, -5)
    ops.moe_ops.moe_balance_blocks(gs, out, ge, gp, E, B, numel, 32, rows)
    want_sorted, want_experts, want_pad = tf.moe_balance_blocks(ids, E, B, 32, rows)
    assert int(gp.item()) == want_pad
    assert out.cpu().tolist() == want_sorted
    assert ge.cpu()[:want_pad // B].tolist() == want_experts
    # the layers' wrapper returns the same tensor for the weight layout whose kernel splits so
    from sarathi_amd import layers
    for packed in (False, True):
        if ops.moe_ops.moe_gemm_slot_rows(B, packed) == rows:
            assert torch.equal(layers.balance_blocks(gs, ge, gp, B, E, numel, packed=packed), out)


def test_moe_gemm_slot_rows_table(ops):
    """Row-major weights: two wave rows from 64-slot blocks on; packed weights: only the eight-wave
    kernel at 256-slot blocks; anything but 32 / 64 / 128 / 256 is refused."""
    rows = ops.moe_ops.moe_gemm_slot_rows
    assert [rows(b, False) for b in (32, 64, 128, 256)] == [1, 2, 2, 2]
    assert [rows(b, True) for b in (32, 64, 128, 256)] == [1, 1, 1, 2]
    with pytest.raises(RuntimeError):
        rows(48, False)
