"""Host-side logic of the layer counterparts, without a GPU: the cos || sin table builders of the
rotary variants (closed forms and reductions between variants), the factory, the activation
registry."""
import math

import pytest
import torch

from helpers import cos_sin_cache


@pytest.fixture(scope="module")
def L(ops):
    from sarathi_amd import layers
    return layers


def _rope(L, scaling=None, D=64, max_pos=256, base=10000, dtype=torch.float32):
    return L.get_rope(D, D, max_pos, base, True, scaling, device="cpu", dtype=dtype)


def test_default_table_closed_form(L):
    r = _rope(L)
    c = r.cos_sin_cache
    assert c.shape == (256, 64) and c.dtype == torch.float32
    for p, i in [(0, 0), (1, 0), (17, 5), (255, 31), (100, 16)]:
        ang = p / (10000 ** (2 * i / 64))
        assert abs(c[p, i].item() - math.cos(ang)) < 2e-5 and abs(c[p, 32 + i].item() - math.sin(ang)) < 2e-5
    assert torch.equal(c[0, :32], torch.ones(32)) and torch.equal(c[0, 32:], torch.zeros(32))
    # the bf16 table of the benchmark configuration is what the tests' helper builds
    big = L.get_rope(128, 128, 8192, 500000, True, None, device="cpu", dtype=torch.bfloat16)
    assert torch.equal(big.cos_sin_cache, cos_sin_cache(8192, 128, 500000.0, torch.bfloat16))


def test_linear_scaling_reduces_to_default_at_multiples(L):
    base = _rope(L).cos_sin_cache
    lin = _rope(L, {"type": "linear", "factor": 4.0})
    assert isinstance(lin, L.LinearScalingRotaryEmbedding)
    assert lin.cos_sin_cache.shape == (1024, 64)
    assert torch.allclose(lin.cos_sin_cache[0::4], base, atol=1e-6)     # position 4p uses angle p
    assert not torch.allclose(lin.cos_sin_cache[:256], base, atol=1e-3)


def test_dynamic_ntk_closed_form(L):
    f = 2.0
    dyn = _rope(L, {"type": "dynamic", "factor": f})
    assert isinstance(dyn, L.DynamicNTKScalingRotaryEmbedding)
    assert dyn.cos_sin_cache.shape == (512, 64)
    new_base = 10000 * ((f * 512 / 256) - (f - 1)) ** (64 / 62)
    for p, i in [(3, 1), (500, 20), (77, 31)]:
        ang = p / (new_base ** (2 * i / 64))
        assert abs(dyn.cos_sin_cache[p, i].item() - math.cos(ang)) < 5e-5
    one = _rope(L, {"type": "dynamic", "factor": 1.0})
    assert torch.equal(one.cos_sin_cache, _rope(L).cos_sin_cache)       # factor 1: base unchanged


def test_yarn_properties(L):
    f, D, orig = 4.0, 64, 256
    sc = {"type": "yarn", "factor": f, "original_max_position_embeddings": orig}
    y = L.get_rope(D, D, int(orig * f), 10000, True, sc, device="cpu", dtype=torch.float32)
    assert isinstance(y, L.YaRNScalingRotaryEmbedding)
    assert y.cos_sin_cache.shape == (1024, 64)
    assert abs(y.mscale - (0.1 * math.log(f) + 1.0)) < 1e-12
    inv = y._compute_inv_freq(f)
    plain = 1.0 / (10000 ** (torch.arange(0, D, 2, dtype=torch.float) / D))
    from sarathi_amd.layers.rotary import yarn_correction_range
    low, high = yarn_correction_range(32, 1, D, 10000, orig)
    assert 0 <= low < high <= D - 1
    assert torch.allclose(inv[: low + 1], plain[: low + 1])             # fast dims keep their frequency
    assert torch.allclose(inv[high:], plain[high:] / f)                 # slow dims are interpolated
    mid = inv[low + 1: high]
    assert bool((mid < plain[low + 1: high]).all()) and bool((mid > plain[low + 1: high] / f).all())
    # row 0: cos = mscale, sin = 0
    assert torch.allclose(y.cos_sin_cache[0, :32], torch.full((32,), y.mscale))
    assert torch.equal(y.cos_sin_cache[0, 32:], torch.zeros(32))
    # factor 1 is the plain table
    one = L.get_rope(D, D, orig, 10000, True, {"type": "yarn", "factor": 1.0,
                                               "original_max_position_embeddings": orig},
                     device="cpu", dtype=torch.float32)
    assert torch.allclose(one.cos_sin_cache, _rope(L, None, D, orig).cos_sin_cache, atol=1e-6)
    # extra keyword arguments are routed through the factory
    y2 = L.get_rope(D, D, int(orig * f), 10000, True, dict(sc, attn_factor=2.0, beta_fast=16),
                    device="cpu", dtype=torch.float32)
    assert abs(y2.mscale - 2.0 * y.mscale) < 1e-12 and y2.beta_fast == 16


def test_factory_errors_and_dtype(L):
    with pytest.raises(ValueError):
        _rope(L, {"type": "ntk-by-parts", "factor": 2.0})
    with pytest.raises(AssertionError):
        L.get_rope(64, 64, 1000, 10000, True, {"type": "yarn", "factor": 4.0,
                                               "original_max_position_embeddings": 256}, device="cpu")
    assert _rope(L, dtype=torch.float16).cos_sin_cache.dtype == torch.float16
    prev = torch.get_default_dtype()
    try:
        torch.set_default_dtype(torch.bfloat16)      # the reference casts to the default dtype
        assert L.get_rope(64, 64, 32, 10000, True, None, device="cpu").cos_sin_cache.dtype == torch.bfloat16
    finally:
        torch.set_default_dtype(prev)


def test_activation_registry(L):
    assert isinstance(L.get_act_fn("gelu_new"), L.NewGELU)
    assert isinstance(L.get_act_fn("GELU_FAST"), L.FastGELU)
    assert isinstance(L.get_act_fn("relu"), torch.nn.ReLU)
    assert L.get_act_fn("gelu_pytorch_tanh").approximate == "tanh"
    with pytest.raises(ValueError):
        L.get_act_fn("swish")


def test_rmsnorm_module_state(L):
    n = L.RMSNorm(128, eps=1e-5, norm_name="input_layernorm", layer_id=10)
    assert n.weight.shape == (128,) and bool((n.weight == 1).all())
    assert n.variance_epsilon == 1e-5 and n.norm_name == "input_layernorm" and n.layer_id == 10


def test_pack_expert_weights_layout_and_inplace():
    """Element (e, n, k) lands in tile n // 32, block k // 16, half (k % 16) // 8, lane row n % 32,
    element k % 8; the in-place variant produces the same bytes inside the original storage."""
    import importlib
    fm = importlib.import_module("sarathi_amd.layers.fused_moe")
    E, N, K = 3, 64, 48
    w = torch.arange(E * N * K, dtype=torch.float32).reshape(E, N, K)
    packed = fm.pack_expert_weights(w)
    assert packed.shape == (E, N, K) and packed.data.shape == (E, N // 32, K // 16, 2, 32, 8)
    for e, n, k in [(0, 0, 0), (1, 33, 17), (2, 63, 47), (1, 5, 9), (0, 32, 8)]:
        assert packed.data[e, n // 32, k // 16, (k % 16) // 8, n % 32, k % 8] == w[e, n, k]
    w2 = w.clone()
    ptr = w2.data_ptr()
    packed2 = fm.pack_expert_weights(w2, inplace=True)
    assert packed2.data.data_ptr() == ptr and torch.equal(packed2.data, packed.data)
    # rows beyond N are zero padding
    odd = fm.pack_expert_weights(torch.ones((1, 40, 16)))
    assert odd.data.shape == (1, 2, 1, 2, 32, 8) and odd.data[0, 1, 0, :, 8:, :].abs().sum() == 0


def test_override_config_block_size_is_raised_to_one_that_exists():
    """A config tuned for the reference's Triton kernel (fused_moe.py:297-318 defaults to
    BLOCK_SIZE_M = 16 for tiny batches) must not be rejected: the block size is raised to the next
    one the kernels have, everything else passes through; supported sizes are returned as given."""
    import importlib
    fm = importlib.import_module("sarathi_amd.layers.fused_moe")
    ref = {"BLOCK_SIZE_M": 16, "BLOCK_SIZE_N": 32, "BLOCK_SIZE_K": 64, "GROUP_SIZE_M": 1}
    got = fm.try_get_optimal_moe_config((8, 28672, 4096), (8, 4096, 14336), 2, 4, override_config=ref)
    assert got["BLOCK_SIZE_M"] == 32 and got["BLOCK_SIZE_N"] == 32 and ref["BLOCK_SIZE_M"] == 16
    for bm in (32, 64, 128, 256):
        cfg = {"BLOCK_SIZE_M": bm}
        assert fm.try_get_optimal_moe_config((8, 8, 64), (8, 64, 4), 2, 4, override_config=cfg) is cfg
    big = fm.try_get_optimal_moe_config((8, 8, 64), (8, 64, 4), 2, 4, override_config={"BLOCK_SIZE_M": 512})
    assert big["BLOCK_SIZE_M"] == 256


def test_tuner_script_names_its_table_as_the_loader_looks_it_up(monkeypatch):
    """``tune_fused_moe.py`` is the recipe for the tables under layers/configs: its argument parser
    builds, and the file it would write is the one ``get_moe_configs`` opens for the same (E, N),
    device name and weight layout; every committed table carries a name the script can produce."""
    import importlib
    import importlib.util
    import os
    import re
    fm = importlib.import_module("sarathi_amd.layers.fused_moe")   # the module, not the function
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    spec = importlib.util.spec_from_file_location(
        "tune_fused_moe", os.path.join(root, "sarathi-serve_amd", "tune_fused_moe.py"))
    tuner = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(tuner)
    args = tuner.build_parser().parse_args(["--experts", "16", "--intermediate", "2688",
                                            "--layout", "row_major", "--device-name", "gfx950"])
    assert (args.experts, args.topk, args.hidden, args.iters) == (16, 2, 4096, 10)
    assert [int(v) for v in args.batch_sizes.split(",")][:3] == [1, 2, 4]
    monkeypatch.setattr(torch.cuda, "get_device_name", lambda *a: "gfx950")
    for layout, packed in (("packed", True), ("row_major", False)):
        assert tuner.output_file_name(16, 2688, "gfx950", layout) == \
            fm.get_config_file_name(16, 2688, None, packed)
    pat = re.compile(r"E=(\d+),N=(\d+),device_name=([^,]+)(,layout=row_major)?\.json$")
    tables = sorted(n for n in os.listdir(fm.CONFIG_DIR) if n.endswith(".json"))
    assert tables, "no tuned tables committed"
    for name in tables:
        m = pat.match(name)
        assert m, name
        assert name == tuner.output_file_name(int(m.group(1)), int(m.group(2)), m.group(3),
                                              "row_major" if m.group(4) else "packed")


def test_norm_layer_enters_the_installed_op_timer():
    """The reference's per-op timer labels survive the layer boundary: RMSNorm enters the context
    manager that the installed factory returns for (norm_name, layer_id), where the reference enters
    its CudaTimer (sarathi/model_executor/layers/layernorm.py:29-32); without a factory, or without
    a name, it is a no-op."""
    import contextlib
    from sarathi_amd import layers
    seen = []

    @contextlib.contextmanager
    def timer(name, layer_id):
        seen.append(("enter", name, layer_id))
        yield
        seen.append(("exit", name, layer_id))

    layers.set_op_timer_factory(timer)
    try:
        norm = layers.RMSNorm(64, norm_name="input_layernorm", layer_id=3)
        unnamed = layers.RMSNorm(64)
    finally:
        layers.set_op_timer_factory(None)
    for layer in (norm, unnamed):
        with pytest.raises(Exception):          # CPU tensors are refused by the op, inside the timer
            layer(torch.zeros((2, 64), dtype=torch.bfloat16))
    assert seen == [("enter", "input_layernorm", 3)] or \
        seen == [("enter", "input_layernorm", 3), ("exit", "input_layernorm", 3)]
    assert layers.op_timer("input_layernorm", 0).__class__ is contextlib.nullcontext
