"""GPU: moe_sum, the sum over a token's top-k expert outputs that ends fused_experts
(reference: torch.sum(intermediate_cache3, dim=1, out=...), fused_moe.py:539-543), against
torch.sum on the CPU: fp32 accumulation and one rounding, so two addends must match bit for bit;
with more addends the fp32 order of additions may differ from the library's, one ulp of the
tensor dtype at most."""
import pytest
import torch

from helpers import assert_close_dtype, gen, randn

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("T,k,H", [(37, 2, 4096), (5, 1, 256), (64, 6, 2048), (3, 2, 77), (9, 8, 24),
                                   (1, 2, 14336)])
def test_moe_sum_matches_library_sum(ops, dev, dtype, T, k, H):
    g = gen(T * 131 + k * 7 + H)
    x = randn((T, k, H), g, dtype, std=1.5)
    want = torch.sum(x, dim=1)
    out = torch.full((T, H), 9.0, dtype=dtype, device=dev)
    ops.moe_ops.moe_sum(x.to(dev), out)
    if k <= 2:
        assert torch.equal(out.cpu(), want)
    elif dtype == torch.float32:
        torch.testing.assert_close(out.cpu(), want, atol=2e-6, rtol=2e-6)
    else:
        assert_close_dtype(out, want, max_ulps=1)


@pytest.mark.parametrize("T,k,H", [(4096, 2, 4096), (4097, 2, 4096), (2304, 1, 4096), (2305, 1, 4096),
                                   (1030, 1, 1000), (3000, 2, 1536), (2304, 2, 8192)])
def test_moe_sum_several_tokens_per_wave(ops, dev, T, k, H):
    """Token counts at which a wave takes two or three tokens (with a ragged last wave), widths
    short of the wave's span, and a width above it (general kernel): exact for one or two addends."""
    g = gen(T + k + H)
    x = randn((T, k, H), g, std=1.5)
    out_big = torch.full((T + 2, H), 9.0, dtype=x.dtype, device=dev)
    ops.moe_ops.moe_sum(x.to(dev), out_big[1:1 + T])
    assert torch.equal(out_big[1:1 + T].cpu(), torch.sum(x, dim=1))
    assert bool((out_big[0] == 9.0).all()) and bool((out_big[T + 1] == 9.0).all())


def test_moe_sum_strided_views_and_untouched_neighbours(ops, dev):
    """Input as a view with padded token and expert strides, output as a row slice of a larger
    tensor (how fused_experts passes out[begin:end]); everything outside the slice keeps its bytes."""
    T, k, H = 50, 2, 512
    g = gen(3)
    big = randn((T, k + 1, H + 64), g).to(dev)
    x = big[:, :k, :H]
    out_big = torch.full((T + 8, H), 3.0, dtype=torch.bfloat16, device=dev)
    ops.moe_ops.moe_sum(x, out_big[4:4 + T])
    assert torch.equal(out_big[4:4 + T].cpu(), torch.sum(x.cpu(), dim=1))
    assert bool((out_big[:4] == 3.0).all()) and bool((out_big[4 + T:] == 3.0).all())


def test_moe_sum_empty_and_argument_checks(ops, dev):
    out = torch.empty((0, 128), dtype=torch.bfloat16, device=dev)
    ops.moe_ops.moe_sum(torch.empty((0, 2, 128), dtype=torch.bfloat16, device=dev), out)
    x = torch.zeros((4, 2, 128), dtype=torch.bfloat16, device=dev)
    with pytest.raises(RuntimeError):
        ops.moe_ops.moe_sum(x, torch.zeros((4, 64), dtype=torch.bfloat16, device=dev))
    with pytest.raises(RuntimeError):
        ops.moe_ops.moe_sum(x, torch.zeros((4, 128), dtype=torch.float16, device=dev))
    with pytest.raises(RuntimeError):
        ops.moe_ops.moe_sum(x.cpu(), torch.zeros((4, 128), dtype=torch.bfloat16))
