"""sarathi_moe_align_block_size_static, the entry point that allocates nothing (its scratch is a
fixed array inside the library's device image), called through the C ABI and compared bit for bit
with sarathi_moe_align_block_size given a caller-provided workspace, and with the CPU oracle.
Two calls in a row share the array, the second with a smaller input.  Collected last on purpose.
"""
import pytest
import torch

import abi_ctypes as abi
from oracle import c_oracle

pytestmark = pytest.mark.gpu

SCRATCH_LIMIT = -4


def _run(lib, fn_static, ids_dev, E, B, fill_pad):
    numel = ids_dev.numel()
    s, e, p = abi.align_buffers(numel, E, B, ids_dev.device, fill=numel if not fill_pad else -3)
    args = [abi.ptr(ids_dev), abi.ID_DT[ids_dev.dtype], numel, E, B, abi.ptr(s), s.numel(),
            abi.ptr(e), e.numel(), abi.ptr(p), int(fill_pad)]
    if fn_static:
        rc = lib.sarathi_moe_align_block_size_static(*args, abi.stream())
        ws = None
    else:
        need = lib.sarathi_moe_align_workspace_bytes(numel, E)
        ws = torch.empty((max(need, 4),), dtype=torch.uint8, device=ids_dev.device)
        rc = lib.sarathi_moe_align_block_size(*args, abi.ptr(ws), need, abi.stream())
    abi.check(lib, rc)
    torch.cuda.synchronize()
    return s.cpu(), e.cpu(), p.cpu()


def _oracle(ids, E, B):
    numel = ids.numel()
    s, e, p = (t.cpu() for t in abi.align_buffers(numel, E, B, "cpu"))
    c_oracle.moe_align_block_size(ids, E, B, s, e, p)
    return s, e, p


def _same(got, want, B):
    assert torch.equal(got[2], want[2])
    assert torch.equal(got[0], want[0])
    nblk = int(want[2].item()) // B
    assert torch.equal(got[1][:nblk], want[1][:nblk])
    assert bool((got[1][nblk:] == -7).all())


def test_static_scratch_entry_matches_workspace_entry_twice(dev):
    lib = abi.load()
    g = torch.Generator().manual_seed(41)
    # all sizes take the three-launch path (above 32 768 ids), i.e. all use the scratch; every
    # call is smaller than the one before, so stale words of the first call's table lie beyond what it writes
    cases = [(200_000, 64, 32, torch.int32), (40_000, 8, 64, torch.int64), (36_000, 5, 16, torch.int16)]
    for numel, E, B, dt in cases:
        ids = torch.randint(0, E, (numel,), generator=g, dtype=torch.int32).to(dt)
        assert lib.sarathi_moe_align_workspace_bytes(numel, E) > 0
        ids_dev = ids.to(dev)
        for fill_pad in (0, 1):
            got = _run(lib, True, ids_dev, E, B, fill_pad)
            want = _run(lib, False, ids_dev, E, B, fill_pad)
            _same(got, want, B)
            _same(got, _oracle(ids, E, B), B)


def test_static_scratch_entry_small_inputs_and_limit(dev):
    lib = abi.load()
    g = torch.Generator().manual_seed(42)
    # small inputs take the one-launch or single-workgroup kernels: no scratch at all
    for numel, E, B in [(8192, 8, 64), (20_000, 64, 16), (1, 8, 4), (0, 8, 4)]:
        ids = torch.randint(0, E, (numel,), generator=g, dtype=torch.int32)
        got = _run(lib, True, ids.to(dev), E, B, 1)
        _same(got, _oracle(ids, E, B), B)
    # 1024 experts and 252 * 512 ids is the largest table that fits; one chunk group more does not
    E, B = 1024, 4
    for numel, ok in [(129_024, True), (129_025, False)]:
        ids = torch.randint(0, E, (numel,), generator=g, dtype=torch.int32)
        ids_dev = ids.to(dev)
        s, e, p = abi.align_buffers(numel, E, B, dev, fill=-3)
        rc = lib.sarathi_moe_align_block_size_static(
            abi.ptr(ids_dev), abi.ID_DT[ids.dtype], numel, E, B, abi.ptr(s), s.numel(), abi.ptr(e),
            e.numel(), abi.ptr(p), 1, abi.stream())
        torch.cuda.synchronize()
        if ok:
            abi.check(lib, rc)
            _same((s.cpu(), e.cpu(), p.cpu()), _oracle(ids, E, B), B)
        else:
            assert rc == SCRATCH_LIMIT
            assert b"scratch" in lib.sarathi_ops_strerror(rc)
            assert p.item() == -7 and bool((s == -3).all())  # nothing was launched


def test_static_scratch_entry_replays_in_a_hip_graph(dev):
    """The caller this entry point exists for: after ONE eager call on the device (the first call
    looks up the array's address, which is host work that must not fall into a capture), a call
    above 32 768 ids is captured into a graph and replayed on new ids, with eager work and
    synchronisation between the replays; every replay matches the oracle."""
    lib = abi.load()
    numel, E, B = 50_000, 16, 64
    g = torch.Generator().manual_seed(43)
    ids_dev = torch.zeros((numel,), dtype=torch.int32, device=dev)
    s, e, p = abi.align_buffers(numel, E, B, dev, fill=-3)

    def call(stream_ptr):
        return lib.sarathi_moe_align_block_size_static(
            abi.ptr(ids_dev), abi.ID_DT[torch.int32], numel, E, B, abi.ptr(s), s.numel(),
            abi.ptr(e), e.numel(), abi.ptr(p), 1, stream_ptr)

    abi.check(lib, call(abi.stream()))          # eager: resolves the scratch address on this device
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            abi.check(lib, call(abi.vp(side.cuda_stream)))
    for _ in range(3):
        ids = torch.randint(0, E, (numel,), generator=g, dtype=torch.int32)
        ids_dev.copy_(ids)
        s.fill_(-3)
        e.fill_(-7)
        p.fill_(-7)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        _same((s.cpu(), e.cpu(), p.cpu()), _oracle(ids, E, B), B)
