"""GPU: paged KV-cache append, its index helpers and the rotary-embedding + append fusion, through
the op namespace -> C ABI, bit-exact against the numpy restatement (oracle/paged_kv.py) and
against the two separate ops."""
import numpy as np
import pytest
import torch

from helpers import cos_sin_cache, gen, randn
from oracle import c_oracle, paged_kv

pytestmark = pytest.mark.gpu


def _bits(t: torch.Tensor) -> np.ndarray:
    """Byte-exact numpy view of a CPU tensor of any supported dtype."""
    t = t.contiguous()
    return t.view(torch.int16 if t.element_size() == 2 else torch.int32).numpy()


def _hybrid(seed, page_size, before, new, spare=5):
    rng = np.random.default_rng(seed)
    totals = [a + b for a, b in zip(before, new)]
    need = [(t + page_size - 1) // page_size for t in totals]
    num_pages = sum(need) + spare
    kv_indices = rng.permutation(num_pages)[:sum(need)].astype(np.int32)
    kv_indptr = np.concatenate([[0], np.cumsum(need)]).astype(np.int32)
    last = np.array([(t % page_size) or page_size if t else 0 for t in totals], dtype=np.int32)
    append_indptr = np.concatenate([[0], np.cumsum(new)]).astype(np.int32)
    return num_pages, kv_indices, kv_indptr, last, append_indptr, totals


CASES = [
    (16, [0, 30, 16, 5, 100], [40, 3, 1, 1, 1]),
    (4, [0, 0, 0], [1, 7, 8]),
    (1, [2, 0], [3, 2]),
    (8, [3, 0, 11], [0, 5, 0]),
]


@pytest.mark.parametrize("page_size,before,new", CASES)
def test_index_helpers_match_oracle(ops, dev, page_size, before, new):
    _, kv_indices, kv_indptr, last, append_indptr, totals = _hybrid(1, page_size, before, new)
    t = lambda a: torch.from_numpy(a).to(dev)  # noqa: E731
    seq_lens = ops.kv_cache_ops.get_seq_lens(t(kv_indptr), t(last), page_size)
    assert seq_lens.dtype == torch.int32
    assert seq_lens.cpu().tolist() == paged_kv.get_seq_lens(kv_indptr, last, page_size).tolist()
    assert seq_lens.cpu().tolist() == totals
    nnz = int(append_indptr[-1])
    b, pos = ops.kv_cache_ops.get_batch_indices_positions(t(append_indptr), seq_lens, nnz)
    wb, wp = paged_kv.get_batch_indices_positions(append_indptr, seq_lens.cpu().numpy(), nnz)
    assert b.cpu().tolist() == wb.tolist() and pos.cpu().tolist() == wp.tolist()


def test_index_helpers_leave_uncovered_tokens_untouched(ops, dev):
    """nnz larger than the last indptr entry: the tail keeps the caller's contents."""
    indptr = torch.tensor([0, 2, 5], dtype=torch.int32, device=dev)
    seq_lens = torch.tensor([4, 9], dtype=torch.int32, device=dev)
    from sarathi_amd._ext import C
    b = torch.full((8,), -7, dtype=torch.int32, device=dev)
    p = torch.full((8,), -7, dtype=torch.int32, device=dev)
    C.get_batch_indices_positions(indptr, seq_lens, b, p)
    assert b.cpu().tolist() == [0, 0, 1, 1, 1, -7, -7, -7]
    assert p.cpu().tolist() == [2, 3, 6, 7, 8, -7, -7, -7]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("page_size,before,new", CASES)
@pytest.mark.parametrize("heads,head_size", [(8, 128), (2, 20), (1, 3)])
def test_append_matches_oracle_bitwise(ops, dev, dtype, page_size, before, new, heads, head_size):
    num_pages, kv_indices, kv_indptr, last, append_indptr, totals = _hybrid(
        heads + page_size, page_size, before, new)
    nnz = int(append_indptr[-1])
    g = gen(nnz + head_size)
    k = randn((nnz, heads, head_size), g, dtype)
    v = randn((nnz, heads, head_size), g, dtype)
    cache = randn((num_pages, 2, page_size, heads, head_size), g, dtype)
    seq_lens = paged_kv.get_seq_lens(kv_indptr, last, page_size)
    b, pos = paged_kv.get_batch_indices_positions(append_indptr, seq_lens, nnz)
    want = _bits(cache).copy()
    paged_kv.append_paged_kv_cache(_bits(k), _bits(v), b, pos, want[:, 0], want[:, 1], kv_indices,
                                   kv_indptr)
    t = lambda a: torch.from_numpy(a).to(dev)  # noqa: E731
    got = cache.to(dev)
    ops.kv_cache_ops.append_paged_kv_cache(k.to(dev), v.to(dev), t(b), t(pos), got, t(kv_indices),
                                           t(kv_indptr), t(last), kv_layout="NHD")
    assert np.array_equal(_bits(got.cpu()), want)
    # separate K / V tensors and 2-D rows taken out of a packed qkv buffer
    kc, vc = cache[:, 0].contiguous().to(dev), cache[:, 1].contiguous().to(dev)
    w = heads * head_size
    qkv = torch.zeros((nnz, 4 * w), dtype=dtype)
    qkv[:, 2 * w:3 * w] = k.reshape(nnz, w)
    qkv[:, 3 * w:] = v.reshape(nnz, w)
    qkv = qkv.to(dev)
    ops.kv_cache_ops.append_paged_kv_cache(qkv[:, 2 * w:3 * w], qkv[:, 3 * w:], t(b), t(pos),
                                           (kc, vc), t(kv_indices), t(kv_indptr))
    assert np.array_equal(_bits(kc.cpu()), want[:, 0]) and np.array_equal(_bits(vc.cpu()), want[:, 1])
    # precomputed slot mapping: same bytes
    slots = ops.kv_cache_ops.get_kv_slot_mapping(t(b), t(pos), t(kv_indices), t(kv_indptr), page_size)
    want_slots = [int(kv_indices[kv_indptr[bi] + p // page_size]) * page_size + p % page_size
                  for bi, p in zip(b.tolist(), pos.tolist())]
    assert slots.cpu().tolist() == want_slots
    got2 = cache.to(dev)
    ops.kv_cache_ops.append_paged_kv_cache(k.to(dev), v.to(dev), t(b), t(pos), got2, t(kv_indices),
                                           t(kv_indptr), slot_mapping=slots)
    assert np.array_equal(_bits(got2.cpu()), want)


@pytest.mark.parametrize("nnz,heads,head_size,dtype", [
    (3001, 4, 64, torch.bfloat16),    # 512-byte rows: several tokens per wave, ragged last wave
    (2050, 1, 8, torch.bfloat16),     # one 16-byte piece per row
    (3003, 8, 96, torch.float16),     # 1.5 KiB rows: two pieces per lane, the second half empty
    (1031, 8, 96, torch.float32),     # 3 KiB rows
    (600, 8, 128, torch.float32),     # exactly 4 KiB
    (517, 16, 160, torch.bfloat16),   # 5 KiB rows: one wave per KiB piece
])
@pytest.mark.parametrize("use_slots", [False, True])
def test_append_every_row_length_class(ops, dev, nnz, heads, head_size, dtype, use_slots):
    """One request whose tokens land on shuffled pages; checked by indexing the cache with the
    slots, which is the definition of the layout (entry e of page p holds slot p * page_size + e)."""
    page_size = 16
    pages = (nnz + page_size - 1) // page_size
    g = gen(nnz)
    table = torch.randperm(pages + 5, generator=g)[:pages].to(torch.int32)
    k = randn((nnz, heads, head_size), g, dtype).to(dev)
    v = randn((nnz, heads, head_size), g, dtype).to(dev)
    cache = randn((pages + 5, 2, page_size, heads, head_size), g, dtype).to(dev)
    before = cache.clone()
    b = torch.zeros(nnz, dtype=torch.int32, device=dev)
    pos = torch.arange(nnz, dtype=torch.int32, device=dev)
    indptr = torch.tensor([0, pages], dtype=torch.int32, device=dev)
    slots = (table.long()[torch.arange(nnz) // page_size] * page_size
             + torch.arange(nnz) % page_size).to(dev)
    ops.kv_cache_ops.append_paged_kv_cache(
        k, v, b, pos, cache, table.to(dev), indptr,
        slot_mapping=slots.to(torch.int32) if use_slots else None)
    flat = cache.permute(0, 2, 1, 3, 4).reshape(-1, 2, heads, head_size)   # [slot, k/v, heads, D]
    assert torch.equal(flat[slots, 0], k) and torch.equal(flat[slots, 1], v)
    untouched = torch.ones(flat.shape[0], dtype=torch.bool, device=dev)
    untouched[slots] = False
    assert torch.equal(flat[untouched],
                       before.permute(0, 2, 1, 3, 4).reshape(flat.shape)[untouched])


def _rope_then_append(positions, q, k, v, head_size, table, is_neox, b, pos, cache, kv_indices,
                      kv_indptr, n):
    """The reference sequence on the CPU: rotary_embedding in place, then append the first n rows."""
    c_oracle.rotary_embedding(positions, q, k, head_size, table, is_neox)
    heads = k.shape[1] // head_size
    bits = _bits(cache)
    paged_kv.append_paged_kv_cache(_bits(k[:n]).reshape(n, heads, head_size),
                                   _bits(v[:n]).reshape(n, heads, head_size), b[:n], pos[:n],
                                   bits[:, 0], bits[:, 1], kv_indices, kv_indptr)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("is_neox", [True, False])
@pytest.mark.parametrize("nq,nkv,head_size,rot,pad", [
    (32, 8, 128, 128, 0),     # Llama-3-8B heads, vector path
    (8, 2, 64, 64, 3),        # three pad rows after the appended ones
    (4, 4, 128, 64, 2),       # partial rotary: element-wise path copies the un-rotated tail
    (3, 1, 24, 24, 0),        # nothing 16-byte aligned
])
@pytest.mark.parametrize("write_key", [False, True])
def test_fused_rope_append_equals_separate_ops(ops, dev, dtype, is_neox, nq, nkv, head_size, rot,
                                               pad, write_key):
    page_size, before, new = 16, [0, 30, 16, 5, 100], [40, 3, 1, 1, 1]
    num_pages, kv_indices, kv_indptr, last, append_indptr, _ = _hybrid(nq, page_size, before, new)
    n = int(append_indptr[-1])
    T = n + pad
    g = gen(T + rot)
    positions = torch.randint(0, 512, (T,), generator=g, dtype=torch.int64)
    table = cos_sin_cache(512, rot, 10000.0, dtype)
    width = (nq + 2 * nkv) * head_size
    qkv = randn((T, width), g, dtype)
    cache = randn((num_pages, 2, page_size, nkv, head_size), g, dtype)
    seq_lens = paged_kv.get_seq_lens(kv_indptr, last, page_size)
    b, pos = paged_kv.get_batch_indices_positions(append_indptr, seq_lens, n)

    ref = qkv.clone()
    want_cache = cache.clone()
    rq, rk, rv = ref.split([nq * head_size, nkv * head_size, nkv * head_size], dim=-1)
    _rope_then_append(positions, rq, rk, rv, head_size, table, is_neox, b, pos, want_cache,
                      kv_indices, kv_indptr, n)

    t = lambda a: torch.from_numpy(a).to(dev)  # noqa: E731
    dq = qkv.to(dev)
    q, k, v = dq.split([nq * head_size, nkv * head_size, nkv * head_size], dim=-1)
    got_cache = cache.to(dev)
    ops.kv_cache_ops.rotary_embedding_append_paged_kv(
        positions.to(dev), q, k, v, head_size, table.to(dev), is_neox, t(b), t(pos), got_cache,
        t(kv_indices), t(kv_indptr), num_append_tokens=n, write_key=write_key)
    assert np.array_equal(_bits(got_cache.cpu()), _bits(want_cache))
    # the same call with the destinations resolved beforehand
    slots = ops.kv_cache_ops.get_kv_slot_mapping(t(b), t(pos), t(kv_indices), t(kv_indptr), page_size)
    dq2 = qkv.to(dev)
    q2, k2, v2 = dq2.split([nq * head_size, nkv * head_size, nkv * head_size], dim=-1)
    got_cache2 = cache.to(dev)
    ops.kv_cache_ops.rotary_embedding_append_paged_kv(
        positions.to(dev), q2, k2, v2, head_size, table.to(dev), is_neox, t(b), t(pos), got_cache2,
        t(kv_indices), t(kv_indptr), num_append_tokens=n, write_key=write_key, slot_mapping=slots)
    assert torch.equal(got_cache2, got_cache) and torch.equal(dq2, dq)
    out = dq.cpu()
    oq, ok, ov = out.split([nq * head_size, nkv * head_size, nkv * head_size], dim=-1)
    assert np.array_equal(_bits(oq), _bits(rq))
    assert np.array_equal(_bits(ov), _bits(rv))                       # values never change
    assert np.array_equal(_bits(ok[n:]), _bits(rk[n:]))               # pad rows: rotated in place
    if write_key:
        assert np.array_equal(_bits(ok[:n]), _bits(rk[:n]))
    else:
        untouched = qkv.split([nq * head_size, nkv * head_size, nkv * head_size], dim=-1)[1]
        assert np.array_equal(_bits(ok[:n]), _bits(untouched[:n]))


@pytest.mark.parametrize("nq,nkv,is_neox,D", [
    (32, 8, False, 128),   # ten segments of interleaved pairs in one wave
    (28, 8, False, 128),   # nine
    (20, 4, False, 128),   # six
    (12, 4, True, 128),    # two NeoX segments
    (24, 8, True, 128),    # four
    (71, 1, True, 64),     # heads of 128 bytes (memory-order loads): Falcon-7B, five q segments + one
    (40, 8, True, 64),     # three segments, the key heads in the first half of theirs
    (9, 9, True, 64),      # ragged: nine heads in a segment of sixteen, for q and for k
    (56, 8, True, 128),    # eight segments: per segment, chunks exchanged over all eight XCDs
])
@pytest.mark.parametrize("write_key", [False, True])
@pytest.mark.parametrize("T", [1700, 1024, 4096, 4097])
def test_fused_rope_append_one_wave_per_token(ops, dev, nq, nkv, is_neox, D, write_key, T):
    """Batches of 1024..4096 tokens take the kernel shape in which one wave covers a whole token
    (4097: one wave per segment again).  Checked bit for bit against the two stand-alone ops (each
    checked against its oracle elsewhere), with fewer appended rows than tokens."""
    _fused_equals_rope_then_append(ops, dev, nq, nkv, is_neox, D, write_key, T)


@pytest.mark.parametrize("T,nq,nkv,is_neox", [
    (400, 32, 32, True),     # eight segments as two waves of four
    (384, 64, 8, True),      # nine as three of three, the key heads in the last
    (1000, 56, 8, True),     # eight as two of four; few key heads: dealt up to eight waves per unit
    (420, 28, 24, True),     # seven as four and three: the second wave's last segment is empty
    (400, 32, 32, False),    # interleaved pairs: sixteen segments as two waves of eight
    (300, 40, 40, False),    # twenty as two of ten
])
@pytest.mark.parametrize("write_key", [False, True])
def test_fused_rope_append_token_dealt_to_several_waves(ops, dev, T, nq, nkv, is_neox, write_key):
    """Tokens of more segments than one wave takes, at batch sizes where they are dealt to two or
    three waves of several segments each instead of one wave per segment."""
    _fused_equals_rope_then_append(ops, dev, nq, nkv, is_neox, 128, write_key, T)


def _fused_equals_rope_then_append(ops, dev, nq, nkv, is_neox, D, write_key, T):
    page_size, n = 16, T - 50
    g = gen(nq * 100 + nkv)
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


def test_hybrid_batch_full_size_round_trip(ops, dev):
    """Llama-3-8B hybrid batch (one 2048-token prompt chunk of a request that already holds 4096
    tokens, 256 decode requests), page size 16, through the host-side metadata builder: reading
    every request back through its page table returns its rotated keys and its values in order."""
    from sarathi_amd import layers
    rng = np.random.default_rng(0)
    page_size, nq, nkv, D = 16, 32, 8, 128
    ctx = rng.integers(1, 3000, size=256)
    lens = [(True, 2048, 4096 + 2048)] + [(False, 1, int(c)) for c in ctx]
    pages_needed = [(t + page_size - 1) // page_size for _, _, t in lens]
    perm = rng.permutation(sum(pages_needed) + 64)
    tables, at = [], 0
    for p in pages_needed:
        tables.append(perm[at:at + p].tolist())
        at += p
    seqs = [layers.SequenceSlice(a, nnew, tot, tab) for (a, nnew, tot), tab in zip(lens, tables)]
    meta = layers.build_append_metadata(seqs, page_size, dev)
    T = meta.num_total_tokens
    assert T == 2304 and meta.num_prefill_tokens == 2048
    g = gen(3)
    qkv = randn((T, (nq + 2 * nkv) * D), g).to(dev)
    table = cos_sin_cache(8192, D, 500000.0, torch.bfloat16).to(dev)
    positions = (meta.append_positions.long())          # rope position == kv position here
    cache = torch.zeros((len(perm), 2, page_size, nkv, D), dtype=torch.bfloat16, device=dev)
    q, k, v = qkv.split([nq * D, nkv * D, nkv * D], dim=-1)
    ref = qkv.clone()
    qkv_before = qkv.clone()
    rq, rk, rv = ref.split([nq * D, nkv * D, nkv * D], dim=-1)
    ops.pos_encoding_ops.rotary_embedding(positions, rq, rk, D, table, True)
    ops.kv_cache_ops.rotary_embedding_append_paged_kv(
        positions, q, k, v, D, table, True, meta.append_batch_indices, meta.append_positions, cache,
        meta.append_kv_page_indices, meta.append_kv_page_indptr)
    assert torch.equal(q, rq)
    # separate op on a second cache gives the same bytes
    cache2 = torch.zeros_like(cache)
    ops.kv_cache_ops.append_paged_kv_cache(rk.reshape(T, nkv, D), rv.reshape(T, nkv, D),
                                           meta.append_batch_indices, meta.append_positions, cache2,
                                           meta.append_kv_page_indices, meta.append_kv_page_indptr,
                                           meta.append_kv_last_page_len)
    assert torch.equal(cache, cache2)
    # the batch's own methods (slot mapping computed once per batch) give the same bytes again
    cache3, cache4 = torch.zeros_like(cache), torch.zeros_like(cache)
    meta.append(rk.reshape(T, nkv, D), rv.reshape(T, nkv, D), cache3)
    qkv2 = ref.clone()
    qkv2.copy_(qkv_before)
    q2, k2, v2 = qkv2.split([nq * D, nkv * D, nkv * D], dim=-1)
    meta.rotary_embedding_append(positions, q2, k2, v2, D, table, True, cache4)
    assert torch.equal(cache, cache3) and torch.equal(cache, cache4) and torch.equal(q2, rq)
    # read back through the page table
    qo = meta.append_qo_indptr.cpu().tolist()
    indptr = meta.append_kv_page_indptr.cpu().tolist()
    pages = meta.append_kv_page_indices.long()
    for r in (0, 1, 100, 256):
        is_prompt, nnew, total = lens[r]
        flat = cache[pages[indptr[r]:indptr[r + 1]]]           # [pages, 2, page_size, nkv, D]
        keys = flat[:, 0].reshape(-1, nkv * D)[total - nnew:total]
        vals = flat[:, 1].reshape(-1, nkv * D)[total - nnew:total]
        assert torch.equal(keys, rk[qo[r]:qo[r + 1]]) and torch.equal(vals, rv[qo[r]:qo[r + 1]])
    assert int((cache != 0).any(dim=-1).any(dim=-1).sum()) <= 2 * T   # nothing else was written
