"""Throughput of the grouped expert GEMM and of the whole fused MoE forward at the Mixtral-8x7B
shape (4096 tokens, 8 experts, top-2, hidden 4096, intermediate 14336, bf16), one MI355X.

Reports time and achieved TFLOP/s against the 2.5 PFLOP/s dense bf16 MFMA peak.  Prints one JSON
line.  Not the repository's headline benchmark (that is bench.py at the root, on the element-wise
path); this covers the step after moe_align_block_size.
"""
import argparse
import json
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, HERE)

MFMA_PEAK_TFLOPS = 2500.0


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--tokens", type=int, default=4096)
    ap.add_argument("--experts", type=int, default=8)
    ap.add_argument("--topk", type=int, default=2)
    ap.add_argument("--hidden", type=int, default=4096)
    ap.add_argument("--intermediate", type=int, default=14336)
    ap.add_argument("--block-m", type=int, default=0, help="0 = the wrapper's own choice")
    ap.add_argument("--iters", type=int, default=20)
    ap.add_argument("--data", choices=["random", "constant"], default="random",
                    help="constant: every activation and weight holds the same value, which toggles "
                         "far fewer bits per operation; shows how much of the gap to the nominal "
                         "peak is the clock the chip sustains under switching power")
    args = ap.parse_args()

    import torch
    import sarathi_amd as ops
    from sarathi_amd import layers

    dev = torch.device("cuda:0")
    torch.manual_seed(0)
    T, E, k, H, I = args.tokens, args.experts, args.topk, args.hidden, args.intermediate
    bf = torch.bfloat16
    x = torch.randn((T, H), device=dev, dtype=torch.float32).to(bf)
    w1 = (torch.randn((E, 2 * I, H), device=dev, dtype=torch.float32) * H ** -0.5).to(bf)
    w2 = (torch.randn((E, H, I), device=dev, dtype=torch.float32) * I ** -0.5).to(bf)
    gating = torch.randn((T, E), device=dev, dtype=torch.float32)
    if args.data == "constant":
        x.fill_(0.0078125)
        w1.fill_(0.0078125)
        w2.fill_(0.0078125)
    tw, ti = layers.fused_topk(x, gating, k, True)
    c1 = torch.empty((T, k, 2 * I), device=dev, dtype=bf)
    c2 = torch.empty((T * k, I), device=dev, dtype=bf)
    c3 = torch.empty((T, k, H), device=dev, dtype=bf)

    def timeit(fn):
        for _ in range(3):
            fn()
        torch.cuda.synchronize()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(args.iters):
            fn()
        b.record()
        torch.cuda.synchronize()
        return a.elapsed_time(b) / args.iters

    f1 = 2.0 * T * k * H * 2 * I
    f2 = 2.0 * T * k * I * H
    res = {}
    for label in ("row_major", "packed"):
        # the block size the library picks for this layout and batch (tuned table or default rule)
        config = dict(layers.try_get_optimal_moe_config((E, 2 * I, H), (E, H, I), k, T,
                                                        packed=label == "packed"))
        if args.block_m:
            config["BLOCK_SIZE_M"] = args.block_m
        bm = config["BLOCK_SIZE_M"]
        s, e, p = layers.moe_align_block_size(ti, bm, E)
        if label == "packed":      # re-tile once, then drop the row-major copies
            p1, p2 = layers.pack_expert_weights(w1), layers.pack_expert_weights(w2)
            b1, b2, pk = p1.data, p2.data, True
            del w1, w2
            torch.cuda.empty_cache()
            wa, wb = p1, p2
        else:
            b1, b2, pk, wa, wb = w1, w2, False, w1, w2
        g1 = lambda: ops.moe_ops.moe_grouped_gemm(x, b1, c1, tw, s, e, p, T * k, bm, k, False, pk, 2 * I)  # noqa: E731
        g2 = lambda: ops.moe_ops.moe_grouped_gemm(c2, b2, c3, tw, s, e, p, T * k, bm, 1, True, pk, H)  # noqa: E731
        g1s = lambda: ops.moe_ops.moe_grouped_gemm(x, b1, c2, tw, s, e, p, T * k, bm, k, False, pk, 2 * I, True)  # noqa: E731
        ms1 = timeit(g1)
        ms_act = timeit(lambda: ops.activation_ops.silu_and_mul(c2, c1.view(-1, 2 * I)))
        ms1s = timeit(g1s)
        ops.activation_ops.silu_and_mul(c2, c1.view(-1, 2 * I))
        ms2 = timeit(g2)
        ms_all = timeit(lambda: layers.fused_moe(x, wa, wb, gating, k, True, override_config=config))
        res[label] = {
            "block_m": bm,
            "gemm_w1": {"ms": round(ms1, 4), "TFLOPs": round(f1 / ms1 * 1e-9, 1),
                        "frac_of_mfma_peak": round(f1 / ms1 * 1e-9 / MFMA_PEAK_TFLOPS, 4)},
            "silu_and_mul": {"ms": round(ms_act, 4)},
            "gemm_w1_with_silu_and_mul_epilogue": {
                "ms": round(ms1s, 4), "TFLOPs": round(f1 / ms1s * 1e-9, 1),
                "frac_of_mfma_peak": round(f1 / ms1s * 1e-9 / MFMA_PEAK_TFLOPS, 4)},
            "gemm_w2": {"ms": round(ms2, 4), "TFLOPs": round(f2 / ms2 * 1e-9, 1),
                        "frac_of_mfma_peak": round(f2 / ms2 * 1e-9 / MFMA_PEAK_TFLOPS, 4)},
            "fused_moe_forward": {"ms": round(ms_all, 4),
                                  "TFLOPs": round((f1 + f2) / ms_all * 1e-9, 1)},
        }
    out = {
        "metric": "grouped expert GEMM TFLOP/s (Mixtral-8x7B MoE layer shape)",
        "config": {"tokens": T, "experts": E, "topk": k, "hidden": H, "intermediate": I,
                   "dtype": "bf16", "data": args.data, "device": torch.cuda.get_device_name(0)},
        "weights": res,
        "weight_bytes": (E * 2 * I * H + E * H * I) * 2,
    }
    print(json.dumps(out))


if __name__ == "__main__":
    main()
