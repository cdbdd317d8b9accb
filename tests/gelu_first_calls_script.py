"""Run in a fresh process by test_gpu_gelu_table.py: the first large 16-bit gelu calls of a process,
which decide whether a call may read the 65536-entry table or must take the arithmetic kernel.

  capture   the very first call is made under stream capture (table not built: the captured launch
            must be the arithmetic kernel, and nothing may be launched outside the capture)
  streams   the first call on one stream, the second at once on another stream (the table's build
            may still be running: that call must not read the table)
Both print OK when every result equals the arithmetic path's bits (chunks below the table size).
"""
import os
import sys

import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "sarathi-serve_amd"))
from sarathi_amd import activation_ops  # noqa: E402


def arithmetic(op, x):
    out = torch.empty_like(x)
    chunk = 1 << 20
    for lo in range(0, x.numel(), chunk):
        piece = torch.empty((1, min(chunk, x.numel() - lo)), dtype=x.dtype, device=x.device)
        op(piece, x[:, lo:lo + piece.numel()].contiguous())
        out[:, lo:lo + piece.numel()] = piece
    return out


def main():
    mode = sys.argv[1]
    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(5)
    n = 1 << 24
    x = (torch.randn((1, n), generator=g) * 2).to(torch.bfloat16).to(dev)
    if mode == "capture":
        out = torch.empty_like(x)
        side = torch.cuda.Stream()
        graph = torch.cuda.CUDAGraph()
        torch.cuda.synchronize()
        with torch.cuda.stream(side):
            with torch.cuda.graph(graph, stream=side):
                activation_ops.gelu_fast(out, x)
        want = arithmetic(activation_ops.gelu_fast, x)
        for _ in range(2):
            out.fill_(5.0)
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(out.view(torch.int16), want.view(torch.int16))
        eager = torch.empty_like(x)
        activation_ops.gelu_fast(eager, x)      # builds the table now
        torch.cuda.synchronize()
        activation_ops.gelu_fast(out, x)        # and this one reads it
        torch.cuda.synchronize()
        assert torch.equal(eager.view(torch.int16), want.view(torch.int16))
        assert torch.equal(out.view(torch.int16), want.view(torch.int16))
    elif mode == "streams":
        a, b = torch.empty_like(x), torch.empty_like(x)
        s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
        torch.cuda.synchronize()
        with torch.cuda.stream(s1):
            activation_ops.gelu_new(a, x)
        with torch.cuda.stream(s2):
            activation_ops.gelu_new(b, x)
        torch.cuda.synchronize()
        want = arithmetic(activation_ops.gelu_new, x)
        assert torch.equal(a.view(torch.int16), want.view(torch.int16))
        assert torch.equal(b.view(torch.int16), want.view(torch.int16))
    else:
        raise SystemExit("unknown mode " + mode)
    print("OK")


if __name__ == "__main__":
    main()
