"""Pick the slot-block size of the grouped expert GEMM per batch size by measurement and write the
result in the reference's tuned-config format (a JSON map batch size -> config, looked up by
``sarathi_amd.layers.get_moe_configs``; reference: the files under
sarathi/model_executor/layers/fused_moe/configs/ and fused_moe.py:262-294).

    python sarathi-serve_amd/tune_fused_moe.py --experts 8 --hidden 4096 --intermediate 14336

times ``fused_experts`` (both GEMMs, activation, sort and top-k sum) for every block size on a grid
of batch sizes and keeps the fastest.  ``--layout row_major`` tunes for the reference's [E, N, K]
weight tensors (file name suffix ``,layout=row_major``), the default for weights re-tiled with
``pack_expert_weights``.  One MI355X, synthetic data.
"""
import argparse
import json
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, HERE)


def build_parser():
    ap = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    ap.add_argument("--experts", type=int, default=8)
    ap.add_argument("--topk", type=int, default=2)
    ap.add_argument("--hidden", type=int, default=4096)
    ap.add_argument("--intermediate", type=int, default=14336)
    ap.add_argument("--batch-sizes", type=str,
                    default="1,2,4,8,16,24,32,48,64,96,128,256,512,1024,1536,2048,3072,4096,8192")
    ap.add_argument("--iters", type=int, default=10)
    ap.add_argument("--out-dir", type=str, default="",
                    help="default: the package's layers/configs directory")
    ap.add_argument("--layout", choices=["packed", "row_major"], default="packed",
                    help="expert weight layout the table is for")
    ap.add_argument("--device-name", type=str, default="",
                    help="device_name field of the file name; default: the GPU architecture")
    return ap


def output_file_name(experts, intermediate, device_name, layout):
    """Name of the table this run writes: the one ``get_moe_configs`` looks up for the same
    (E, N), device name and weight layout."""
    suffix = "" if layout == "packed" else ",layout=row_major"
    return "E=%d,N=%d,device_name=%s%s.json" % (experts, intermediate, device_name, suffix)


def main():
    args = build_parser().parse_args()

    import torch
    from sarathi_amd import layers
    import importlib
    fm = importlib.import_module("sarathi_amd.layers.fused_moe")   # the module, not the function

    dev = torch.device("cuda:0")
    torch.manual_seed(0)
    E, k, H, I = args.experts, args.topk, args.hidden, args.intermediate
    bf = torch.bfloat16
    w1 = (torch.randn((E, 2 * I, H), device=dev, dtype=torch.float32) * H ** -0.5).to(bf)
    w2 = (torch.randn((E, H, I), device=dev, dtype=torch.float32) * I ** -0.5).to(bf)
    if args.layout == "packed":
        w1, w2 = layers.pack_expert_weights(w1), layers.pack_expert_weights(w2)

    def time_ms(fn):
        for _ in range(2):
            fn()
        torch.cuda.synchronize()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(args.iters):
            fn()
        b.record()
        torch.cuda.synchronize()
        return a.elapsed_time(b) / args.iters

    table, report = {}, {}
    for M in [int(v) for v in args.batch_sizes.split(",")]:
        x = torch.randn((M, H), device=dev, dtype=torch.float32).to(bf)
        gating = torch.randn((M, E), device=dev, dtype=torch.float32)
        tw, ti = layers.fused_topk(x, gating, k, True)
        best = None
        row = {}
        for bm in fm._BLOCK_SIZES:
            cfg = {"BLOCK_SIZE_M": bm, "BLOCK_SIZE_N": 256, "BLOCK_SIZE_K": 64, "GROUP_SIZE_M": 1}
            ms = time_ms(lambda: layers.fused_experts(x, w1, w2, tw, ti, override_config=cfg))
            row[bm] = round(ms, 4)
            if best is None or ms < best[0]:
                best = (ms, cfg)
        table[str(M)] = best[1]
        report[M] = row
        print("M=%5d  %s  -> BLOCK_SIZE_M=%d" % (M, row, best[1]["BLOCK_SIZE_M"]), flush=True)

    arch = torch.cuda.get_device_properties(0).gcnArchName.split(":")[0]
    name = args.device_name or arch
    out_dir = args.out_dir or fm.CONFIG_DIR
    os.makedirs(out_dir, exist_ok=True)
    path = os.path.join(out_dir, output_file_name(E, I, name, args.layout))
    with open(path, "w") as f:
        json.dump(table, f, indent=4)
        f.write("\n")
    print(json.dumps({"written": path, "ms_by_block": report}))


if __name__ == "__main__":
    main()
