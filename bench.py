"""Benchmark of the fused layer ops on the Llama-3-8B 2304-token hybrid batch (one MI355X).

A "step" is one pass of a decoder layer's element-wise chain over one hybrid batch
(2048 prefill tokens + 256 decode tokens), in layer order:

    fused_add_rms_norm [2304, 4096]            (input layernorm with the residual add fused in)
    rotary_embedding   q [2304, 32*128], k [2304, 8*128], views of a packed [2304, 6144] qkv
    fused_add_rms_norm [2304, 4096]            (post-attention layernorm)
    silu_and_mul       [2304, 2*14336] -> [2304, 14336]

All inputs are resident in HBM before the timed region.  Every step works on a different one of
several independent buffer sets whose total footprint exceeds 512 MB, so the 256 MB Infinity Cache
cannot serve the reads ("cold" numbers).  `value` is the step's algorithmic bytes divided by the
step time.  `per_op` carries, for every op (plus rms_norm alone and the Mixtral-shaped MoE routing
ops), µs per call, GB/s and fraction of the 8 TB/s HBM peak, cold and warm (same buffers every
call).  `roofline` describes the dominant kernel of the step, silu_and_mul: its algorithmic bytes
divided by its average launch duration over --steps back-to-back launches on cold buffers between
two HIP events on the launch stream.  `cpu_baseline` is the PyTorch CPU formulation of the same
step on this machine's host cores.  `moe_layer` times the MoE layer that the routing ops feed
(`fused_moe` forward with the grouped expert GEMMs, Mixtral-8x7B shape, row-major weights) at
three batch sizes; it is reported beside the headline, not in it.

--calibrate-copy additionally runs a plain device-to-device copy of a known size (256 MiB,
torch's copy kernel) so that a `rocprofv3 --pmc FETCH_SIZE` / `WRITE_SIZE` run of this script can
scale the counters by what they read for a known amount of traffic.

Prints ONE JSON line.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, "sarathi-serve_amd"), os.path.join(ROOT, "tests")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

HBM_PEAK_GBS = 8000.0

T, H, NQ, NKV, D, DFF = 2304, 4096, 32, 8, 128, 14336
PREFILL = 2048
BF16 = 2

# algorithmic (compulsory) bytes per call: every input element read once, every output element
# written once, in-place tensors counted read + write, weight / touched cache rows once
BYTES = {
    "fused_add_rms_norm": 4 * T * H * BF16 + H * BF16,
    "rms_norm": 2 * T * H * BF16 + H * BF16,
    # q and k read + written, int64 positions, one cos||sin cache row per token
    "rotary_embedding": 2 * (T * NQ * D + T * NKV * D) * BF16 + T * 8 + T * D * BF16,
    "silu_and_mul": (2 * T * DFF + T * DFF) * BF16,
}
# the step after rotary_embedding on the reference path: k and v rows go to their paged-cache
# entries (read once, written once; 16 index bytes per token) ...
PAGE = 16
BYTES["append_paged_kv_cache"] = 4 * T * NKV * D * BF16 + T * 16
# ... and the fusion of the two: q read + written, k and v read once, cache entries written once
BYTES["rotary_embedding_append_paged_kv"] = (2 * T * NQ * D + 4 * T * NKV * D) * BF16 + T * 24 + \
    T * D * BF16
BYTES["append_paged_kv_cache (slot mapping)"] = 4 * T * NKV * D * BF16 + T * 4
BYTES["rotary_embedding_append_paged_kv (slot mapping)"] = \
    BYTES["rotary_embedding_append_paged_kv"] - T * 12
# the reference's operation-metric names for the places these ops run at
# (sarathi/metrics/constants.py:9-34), so that reports line up with its own per-op timers
REFERENCE_LABELS = {
    "fused_add_rms_norm": "input_layernorm / post_attention_layernorm",
    "rms_norm": "input_layernorm / post_attention_layernorm",
    "rotary_embedding": "attn_rope",
    "silu_and_mul": "mlp_activation",
    "append_paged_kv_cache": "attn_kv_cache_save",
    "rotary_embedding_append_paged_kv": "attn_rope + attn_kv_cache_save",
    "topk_softmax": "moe_gating",
    "moe_align_block_size": "moe_linear (slot sort)",
    "fused_topk_align": "moe_gating + moe_linear (slot sort)",
}
MOE_T, MOE_E, MOE_K, MOE_B = 4096, 8, 2, 64
BYTES["topk_softmax"] = MOE_T * MOE_E * 4 + 3 * MOE_T * MOE_K * 4
_moe_sorted = MOE_T * MOE_K + MOE_E * (MOE_B - 1)
BYTES["moe_align_block_size"] = MOE_T * MOE_K * 4 + _moe_sorted * 4 + 4 * (
    (_moe_sorted + MOE_B - 1) // MOE_B) + 4
# both in one launch: the ids are written once and re-read from L2
BYTES["fused_topk_align"] = BYTES["topk_softmax"] + BYTES["moe_align_block_size"]


# HBM bytes per silu_and_mul launch at this shape as measured with rocprofv3 --pmc FETCH_SIZE and
# WRITE_SIZE (two runs), each counter scaled by what it reads for a plain 256 MiB copy:
# (64522.0 KiB * 1.99982 + 64512.0 KiB * 1.00000) * 1024.  Counters cannot be read from inside
# this script; the summary with the commands is profiles/kernels_llama3_8b_t2304_pmc_fetch_write.txt.
SILU_MEASURED_HBM_BYTES = 198189751


def make_set(torch, g, dev, cache_cpu):
    """One independent set of step inputs (seeded on the CPU, fp32 draw -> bf16)."""
    from helpers import hybrid_positions, randn
    s = {}
    s["x"] = randn((T, H), g).to(dev)
    s["res"] = randn((T, H), g).to(dev)
    s["w1"] = randn((H,), g, mean=1.0, std=0.1).to(dev)
    s["w2"] = randn((H,), g, mean=1.0, std=0.1).to(dev)
    s["qkv"] = randn((T, (NQ + 2 * NKV) * D), g).to(dev)
    s["q"], s["k"], _ = s["qkv"].split([NQ * D, NKV * D, NKV * D], dim=-1)
    s["pos"] = hybrid_positions(T, PREFILL, g).to(dev)
    s["cache"] = cache_cpu.to(dev)
    s["gate_up"] = randn((T, 2 * DFF), g).to(dev)
    s["act"] = torch.empty((T, DFF), dtype=torch.bfloat16, device=dev)
    s["norm_out"] = torch.empty((T, H), dtype=torch.bfloat16, device=dev)
    return s


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--sets", type=int, default=4, help="independent buffer sets to rotate through")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also launch a 256 MiB plain copy (counter calibration for --pmc runs)")
    ap.add_argument("--traffic", type=float, default=SILU_MEASURED_HBM_BYTES,
                    help="measured HBM bytes per silu_and_mul launch, reported verbatim as "
                         "roofline.traffic (default: the figure of the committed rocprofv3 --pmc "
                         "summary under profiles/)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this op library runs on one GPU; --gpus must be 1 "
                 "(the ops are per-token and never communicate)")

    import torch
    import sarathi_amd as ops          # raises if the HIP extension is missing
    from helpers import THETA_LLAMA3, cos_sin_cache, gen
    from oracle import torch_formulations as cpu_ops

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    LN, ACT, ROPE, MOE = ops.layernorm_ops, ops.activation_ops, ops.pos_encoding_ops, ops.moe_ops

    g = gen(1)
    cache_cpu = cos_sin_cache(8192, D, THETA_LLAMA3, torch.bfloat16)
    sets = [make_set(torch, g, dev, cache_cpu) for _ in range(args.sets)]
    set_bytes = sum(v.numel() * v.element_size() for k, v in sets[0].items() if k not in ("q", "k"))

    def step(s):
        LN.fused_add_rms_norm(s["x"], s["res"], s["w1"], 1e-5)
        ROPE.rotary_embedding(s["pos"], s["q"], s["k"], D, s["cache"], True)
        LN.fused_add_rms_norm(s["x"], s["res"], s["w2"], 1e-5)
        ACT.silu_and_mul(s["act"], s["gate_up"])

    step_bytes = 2 * BYTES["fused_add_rms_norm"] + BYTES["rotary_embedding"] + BYTES["silu_and_mul"]

    # ---- the timed region: exactly --steps steps, rotating buffer sets (cold) ----
    for i in range(args.warmup):
        step(sets[i % len(sets)])
    torch.cuda.synchronize()
    t0 = torch.cuda.Event(enable_timing=True)
    t1 = torch.cuda.Event(enable_timing=True)
    wall0 = time.perf_counter()
    t0.record()
    for i in range(args.steps):
        step(sets[i % len(sets)])
    t1.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - wall0
    gpu_ms = t0.elapsed_time(t1)
    ms_per_step = max(gpu_ms, wall * 1e3) / args.steps

    # ---- per-op tables: K back-to-back launches between two events ----
    # Every op gets its own ring of argument sets.  "cold": the ring's footprint exceeds
    # COLD_FOOTPRINT, so by the time a set comes round again the 256 MB Infinity Cache has been
    # flushed through twice over; "warm": the same set every call.
    COLD_FOOTPRINT = 640e6
    from helpers import hybrid_positions, randn

    def ring(name, make):
        n = max(4, int(COLD_FOOTPRINT // BYTES[name]) + 1)
        return [make() for _ in range(n)]          # a set may hold more than the op touches

    w_dev = sets[0]["w1"]
    cache_dev = sets[0]["cache"]
    pos_dev = sets[0]["pos"]

    torch.manual_seed(1)

    def dev_randn(shape):      # ring contents only feed timing loops: draw them on the device
        return torch.randn(shape, device=dev, dtype=torch.float32).to(torch.bfloat16)

    def mk_norm():
        return (dev_randn((T, H)), dev_randn((T, H)))

    def mk_rope():
        qkv = dev_randn((T, (NQ + 2 * NKV) * D))
        q, k, _ = qkv.split([NQ * D, NKV * D, NKV * D], dim=-1)
        return (qkv, q, k)

    def mk_silu():
        return (dev_randn((T, 2 * DFF)), torch.empty((T, DFF), dtype=torch.bfloat16, device=dev))

    # paged KV cache of the hybrid batch: one prompt chunk continuing a 4096-token request and
    # 256 decode requests with contexts of 1..3000 tokens, pages handed out in random order
    from sarathi_amd import kv_cache_ops as KV
    from sarathi_amd import layers as LAYERS
    import numpy as np
    rng = np.random.default_rng(5)
    lens = [(True, PREFILL, 4096 + PREFILL)] + [(False, 1, int(c))
                                                for c in rng.integers(1, 3000, size=T - PREFILL)]
    need = [(t + PAGE - 1) // PAGE for _, _, t in lens]
    perm = rng.permutation(sum(need))
    seqs, at = [], 0
    for (is_p, new, tot), n_pages in zip(lens, need):
        seqs.append(LAYERS.SequenceSlice(is_p, new, tot, perm[at:at + n_pages].tolist()))
        at += n_pages
    meta = LAYERS.build_append_metadata(seqs, PAGE, dev)
    assert meta.num_total_tokens == T
    # every ring set gets its own cache of just the pages that are written (plus the old ones'
    # numbers: entries are addressed through the page table, so the tensor must span them all)
    touched = torch.unique((meta.append_kv_page_indices[
        (meta.append_kv_page_indptr[meta.append_batch_indices.long()]
         + meta.append_positions // PAGE).long()]).long())
    remap = torch.zeros(sum(need), dtype=torch.int32, device=dev)
    remap[touched] = torch.arange(touched.numel(), dtype=torch.int32, device=dev)
    kv_indices_dense = remap[meta.append_kv_page_indices.long()]   # untouched pages alias page 0

    slots_dense = KV.get_kv_slot_mapping(meta.append_batch_indices, meta.append_positions,
                                         kv_indices_dense, meta.append_kv_page_indptr, PAGE)

    def mk_kv():
        qkv = dev_randn((T, (NQ + 2 * NKV) * D))
        q, k, v = qkv.split([NQ * D, NKV * D, NKV * D], dim=-1)
        cache = torch.empty((touched.numel(), 2, PAGE, NKV, D), dtype=torch.bfloat16, device=dev)
        return (qkv, q, k, v, (cache[:, 0], cache[:, 1]))   # K / V planes split once, not per call

    mg = gen(3)
    gating = torch.randn((MOE_T, MOE_E), generator=mg, dtype=torch.float32).to(dev)
    tw = torch.empty((MOE_T, MOE_K), dtype=torch.float32, device=dev)
    ti = torch.empty((MOE_T, MOE_K), dtype=torch.int32, device=dev)
    ts = torch.empty((MOE_T, MOE_K), dtype=torch.int32, device=dev)
    MOE.topk_softmax(tw, ti, ts, gating)
    sorted_ids = torch.empty((_moe_sorted,), dtype=torch.int32, device=dev)
    expert_ids = torch.empty(((_moe_sorted + MOE_B - 1) // MOE_B,), dtype=torch.int32, device=dev)
    post_pad = torch.empty((1,), dtype=torch.int32, device=dev)

    ops_table = {
        "fused_add_rms_norm": (ring("fused_add_rms_norm", mk_norm),
                               lambda a: LN.fused_add_rms_norm(a[0], a[1], w_dev, 1e-5)),
        "rms_norm": (ring("rms_norm", mk_norm), lambda a: LN.rms_norm(a[1], a[0], w_dev, 1e-5)),
        "rotary_embedding": (ring("rotary_embedding", mk_rope),
                             lambda a: ROPE.rotary_embedding(pos_dev, a[1], a[2], D, cache_dev, True)),
        "silu_and_mul": (ring("silu_and_mul", mk_silu), lambda a: ACT.silu_and_mul(a[1], a[0])),
        "append_paged_kv_cache": (ring("append_paged_kv_cache", mk_kv),
                                  lambda a: KV.append_paged_kv_cache(
                                      a[2], a[3], meta.append_batch_indices, meta.append_positions,
                                      a[4], kv_indices_dense, meta.append_kv_page_indptr)),
        "rotary_embedding_append_paged_kv": (
            ring("rotary_embedding_append_paged_kv", mk_kv),
            lambda a: KV.rotary_embedding_append_paged_kv(
                pos_dev, a[1], a[2], a[3], D, cache_dev, True, meta.append_batch_indices,
                meta.append_positions, a[4], kv_indices_dense, meta.append_kv_page_indptr)),
        "append_paged_kv_cache (slot mapping)": (
            ring("append_paged_kv_cache", mk_kv),
            lambda a: KV.append_paged_kv_cache(
                a[2], a[3], meta.append_batch_indices, meta.append_positions, a[4],
                kv_indices_dense, meta.append_kv_page_indptr, slot_mapping=slots_dense)),
        "rotary_embedding_append_paged_kv (slot mapping)": (
            ring("rotary_embedding_append_paged_kv", mk_kv),
            lambda a: KV.rotary_embedding_append_paged_kv(
                pos_dev, a[1], a[2], a[3], D, cache_dev, True, meta.append_batch_indices,
                meta.append_positions, a[4], kv_indices_dense, meta.append_kv_page_indptr,
                slot_mapping=slots_dense)),
        "topk_softmax": ([None], lambda a: MOE.topk_softmax(tw, ti, ts, gating)),
        "moe_align_block_size": ([None], lambda a: MOE.moe_align_block_size_filled(
            ti, MOE_E, MOE_B, sorted_ids, expert_ids, post_pad)),
        "fused_topk_align": ([None], lambda a: MOE.fused_topk_align(
            tw, ti, ts, gating, True, MOE_B, sorted_ids, expert_ids, post_pad, True)),
    }

    def time_op(fn, args, reps):
        n = len(args)
        for i in range(max(n, 5)):
            fn(args[i % n])
        torch.cuda.synchronize()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for i in range(reps):
            fn(args[i % n])
        b.record()
        torch.cuda.synchronize()
        return a.elapsed_time(b) * 1e3 / reps

    per_op = {}
    for name, (args_ring, fn) in ops_table.items():
        row = {"bytes": BYTES[name]}
        if name.split(" ")[0] in REFERENCE_LABELS:
            row["reference_label"] = REFERENCE_LABELS[name.split(" ")[0]]
        latency_bound = name in ("topk_softmax", "moe_align_block_size", "fused_topk_align")
        for label in ("cold", "warm"):
            if latency_bound and label == "cold":
                continue   # 0.07-0.2 MB working sets: launch-latency-bound, one (warm) figure
            use = args_ring if label == "cold" else args_ring[:1]
            us = time_op(fn, use, args.steps)
            gbs = BYTES[name] / us * 1e-3
            row[label] = {"us": round(us, 3), "GBps": round(gbs, 1),
                          "frac_of_peak": round(gbs / HBM_PEAK_GBS, 4)}
        if not latency_bound:
            row["ring_sets"] = len(args_ring)
        per_op[name] = row
        del args_ring
    del ops_table
    torch.cuda.empty_cache()

    # ---- context: a plain device-to-device copy that moves the same number of bytes ----
    # (torch's copy kernel, cold ring).  Half of an op's algorithmic bytes are read and half
    # written, which is exactly rms_norm's and rotary_embedding's mix; it shows what the memory
    # system gives a trivial kernel at each size.
    copy_ref = {}
    for name in ("rms_norm", "rotary_embedding", "fused_add_rms_norm", "silu_and_mul"):
        half = BYTES[name] // 2 // 2 * 2
        n = max(4, int(COLD_FOOTPRINT // BYTES[name]) + 1)
        pairs = [(torch.empty(half // 2, dtype=torch.bfloat16, device=dev).fill_(1.0),
                  torch.empty(half // 2, dtype=torch.bfloat16, device=dev)) for _ in range(n)]
        us = time_op(lambda a: a[1].copy_(a[0]), pairs, args.steps)
        gbs = 2 * half / us * 1e-3
        copy_ref[name] = {"bytes": 2 * half, "us": round(us, 3), "GBps": round(gbs, 1),
                          "frac_of_peak": round(gbs / HBM_PEAK_GBS, 4)}
        del pairs
    torch.cuda.empty_cache()

    if args.calibrate_copy:
        src = torch.empty((256 << 20) // 2, dtype=torch.bfloat16, device=dev).fill_(1.0)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    # ---- the other configurations of the same path (reported beside the headline workload) ----
    # C1: the fused norm at the 512-token shape that is also the CPU-sized case; C5: the four ops at
    # Llama-3-70B widths, T = 4608 (4096-token chunk + 512 decodes), one GPU, unsharded.
    def measure_shape(Tn, Hn, nq, nkv, dff, which):
        rows = {}
        wn = dev_randn((Hn,))
        table = cache_dev
        posn = hybrid_positions(Tn, Tn - Tn // 9, gen(4), prefill_start=4096,
                                max_pos=8192).to(dev) if "rotary_embedding" in which else None

        def sized_ring(nbytes, make):
            return [make() for _ in range(max(2, int(COLD_FOOTPRINT // nbytes) + 1))]
        plan = {
            "fused_add_rms_norm": (4 * Tn * Hn * BF16 + Hn * BF16,
                                   lambda: (dev_randn((Tn, Hn)), dev_randn((Tn, Hn))),
                                   lambda a: LN.fused_add_rms_norm(a[0], a[1], wn, 1e-5)),
            "rms_norm": (2 * Tn * Hn * BF16 + Hn * BF16,
                         lambda: (dev_randn((Tn, Hn)), dev_randn((Tn, Hn))),
                         lambda a: LN.rms_norm(a[1], a[0], wn, 1e-5)),
            "rotary_embedding": (2 * Tn * (nq + nkv) * D * BF16 + Tn * 8 + Tn * D * BF16,
                                 lambda: dev_randn((Tn, (nq + 2 * nkv) * D)),
                                 lambda a: ROPE.rotary_embedding(
                                     posn, *a.split([nq * D, nkv * D, nkv * D], dim=-1)[:2], D,
                                     table, True)),
            "silu_and_mul": (3 * Tn * dff * BF16,
                             lambda: (dev_randn((Tn, 2 * dff)),
                                      torch.empty((Tn, dff), dtype=torch.bfloat16, device=dev)),
                             lambda a: ACT.silu_and_mul(a[1], a[0])),
        }
        for name in which:
            nbytes, make, fn = plan[name]
            r = sized_ring(nbytes, make)
            us = time_op(fn, r, max(20, args.steps // 2))
            gbs = nbytes / us * 1e-3
            rows[name] = {"bytes": nbytes, "cold": {"us": round(us, 3), "GBps": round(gbs, 1),
                                                   "frac_of_peak": round(gbs / HBM_PEAK_GBS, 4)},
                          "ring_sets": len(r)}
            del r
            torch.cuda.empty_cache()
        return rows

    other_configs = {
        "fused_add_rms_norm [512, 4096] (CPU-sized case)":
            measure_shape(512, 4096, 32, 8, 14336, ["fused_add_rms_norm"]),
        "Llama-3-70B widths, T=4608: norm [4608, 8192], rope q[4608, 8192] k[4608, 1024], "
        "silu_and_mul [4608, 57344]":
            measure_shape(4608, 8192, 64, 8, 28672,
                          ["fused_add_rms_norm", "rms_norm", "rotary_embedding", "silu_and_mul"]),
    }

    # ---- the MoE layer either side of the routing ops: fused_moe forward (routing, slot sort, both
    # grouped expert GEMMs with the activation in the first one's epilogue, top-k sum) at the
    # Mixtral-8x7B layer shape with the reference's row-major [E, N, K] weights.  MFMA-bound at
    # large batches, weight-streaming-bound at decode sizes; not part of `value`.
    def measure_moe_layer():
        from sarathi_amd import layers
        E, k, H, I = 8, 2, 4096, 14336
        bf = torch.bfloat16
        w1 = (torch.randn((E, 2 * I, H), device=dev, dtype=torch.float32) * H ** -0.5).to(bf)
        w2 = (torch.randn((E, H, I), device=dev, dtype=torch.float32) * I ** -0.5).to(bf)
        rows = {}
        for Tn in (16, 1024, 4096):
            x = torch.randn((Tn, H), device=dev, dtype=torch.float32).to(bf)
            logits = torch.randn((Tn, E), device=dev, dtype=torch.float32)
            fn = lambda: layers.fused_moe(x, w1, w2, logits, k, True)  # noqa: E731
            for _ in range(3):
                fn()
            torch.cuda.synchronize()
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            reps = 20
            a.record()
            for _ in range(reps):
                fn()
            b.record()
            torch.cuda.synchronize()
            ms = a.elapsed_time(b) / reps
            flop = 2.0 * Tn * k * 3 * I * H
            rows["%d tokens" % Tn] = {
                "ms": round(ms, 4), "TFLOPs": round(flop / ms * 1e-9, 1),
                "frac_of_mfma_peak": round(flop / ms * 1e-9 / 2500.0, 4),
                "weight_stream_TBps": round((E * 3 * I * H * 2) / ms * 1e-9, 2)}
        del w1, w2
        torch.cuda.empty_cache()
        return {"shape": "Mixtral-8x7B MoE layer: 8 experts, top-2, hidden 4096, intermediate 14336, "
                         "bf16, row-major weights, back-to-back launches (weights warm in L2/MALL "
                         "as far as they fit)",
                "peak": "2500 TFLOP/s dense bf16 MFMA; 8 TB/s HBM", "fused_moe_forward": rows}

    moe_layer = measure_moe_layer()

    silu_us = per_op["silu_and_mul"]["cold"]["us"]
    silu_gbs = BYTES["silu_and_mul"] / silu_us * 1e-3
    roofline = {
        "kernel": "silu_and_mul_kernel (bf16, [2304, 28672] -> [2304, 14336])",
        "bound": "hbm", "achieved": round(silu_gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
        "frac": round(silu_gbs / HBM_PEAK_GBS, 4), "traffic": args.traffic,
        "bytes_per_launch": BYTES["silu_and_mul"], "avg_launch_us": round(silu_us, 3),
        "timing": "%d back-to-back launches between two HIP events on the launch stream, rotating "
                  "over %d cold buffer sets" % (args.steps, per_op["silu_and_mul"]["ring_sets"]),
    }

    # ---- CPU baseline: the PyTorch formulation of the same step on the host cores ----
    cpu = None
    if not args.no_cpu_baseline:
        cg = gen(1)
        cx, cr = randn((T, H), cg), randn((T, H), cg)
        cw = randn((H,), cg, mean=1.0, std=0.1)
        cqkv = randn((T, (NQ + 2 * NKV) * D), cg)
        cq, ck, _ = cqkv.split([NQ * D, NKV * D, NKV * D], dim=-1)
        cpos = hybrid_positions(T, PREFILL, cg)
        cgu = randn((T, 2 * DFF), cg)
        cact = torch.empty((T, DFF), dtype=torch.bfloat16)

        def cpu_step():
            cpu_ops.fused_add_rms_norm(cx, cr, cw, 1e-5)
            cpu_ops.rotary_embedding(cpos, cq, ck, D, cache_cpu, True)
            cpu_ops.fused_add_rms_norm(cx, cr, cw, 1e-5)
            cpu_ops.silu_and_mul(cact, cgu)

        cpu_step()
        t_start = time.perf_counter()
        cpu_step()
        one = time.perf_counter() - t_start
        reps = max(3, min(2000, int(12.0 / max(one, 1e-3))))      # about 12 s of CPU work
        times = []
        for _ in range(reps):
            t_start = time.perf_counter()
            cpu_step()
            times.append(time.perf_counter() - t_start)
        times.sort()
        med = times[len(times) // 2]

        # a CPU column for every op of the table (median of a few repetitions, same formulations)
        def cpu_us(fn, reps=5):
            fn()
            ts = []
            for _ in range(reps):
                t0 = time.perf_counter()
                fn()
                ts.append(time.perf_counter() - t0)
            return round(sorted(ts)[len(ts) // 2] * 1e6, 1)
        cnorm = torch.empty_like(cx)
        cgating = gating.cpu()
        ctw, cti, cts = tw.cpu(), ti.cpu(), ts.cpu()
        csorted, cexp, cpost = sorted_ids.cpu(), expert_ids.cpu(), post_pad.cpu()
        cpu_cols = {
            "fused_add_rms_norm": lambda: cpu_ops.fused_add_rms_norm(cx, cr, cw, 1e-5),
            "rms_norm": lambda: cpu_ops.rms_norm(cnorm, cx, cw, 1e-5),
            "rotary_embedding": lambda: cpu_ops.rotary_embedding(cpos, cq, ck, D, cache_cpu, True),
            "silu_and_mul": lambda: cpu_ops.silu_and_mul(cact, cgu),
            "topk_softmax": lambda: cpu_ops.topk_softmax(ctw, cti, cts, cgating),
            "moe_align_block_size": lambda: cpu_ops.moe_align_block_size(
                cti, MOE_E, MOE_B, csorted, cexp, cpost),
        }
        for name, fn in cpu_cols.items():
            per_op[name]["cpu_us"] = cpu_us(fn)
        c1x, c1r = randn((512, H), cg), randn((512, H), cg)
        other_configs["fused_add_rms_norm [512, 4096] (CPU-sized case)"]["fused_add_rms_norm"][
            "cpu_us"] = cpu_us(lambda: cpu_ops.fused_add_rms_norm(c1x, c1r, cw, 1e-5), reps=20)
        cpu = {
            "value": round(step_bytes / med * 1e-9, 2), "unit": "GB/s",
            "cores": torch.get_num_threads(), "kind": "port",
            "sample": "%d repetitions of the same 2304-token step (median %.1f ms/step) with the "
                      "PyTorch CPU formulation of the ops (oracle/torch_formulations.py), "
                      "os.cpu_count()=%d" % (reps, med * 1e3, os.cpu_count()),
            "ms_per_step": round(med * 1e3, 2),
        }

    value = step_bytes / (ms_per_step * 1e-3) * 1e-9
    out = {
        "metric": "achieved HBM GB/s (% of peak) per fused op at 2304-token hybrid batch",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms_per_step, 5), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {
            "workload": "Llama-3-8B hybrid batch, T=2304 (2048-token prefill chunk at positions "
                        "4096..6143 + 256 decode tokens): fused_add_rms_norm[2304,4096] -> neox "
                        "rotary_embedding(q[2304,4096], k[2304,1024], packed qkv, theta=5e5) -> "
                        "fused_add_rms_norm -> silu_and_mul[2304,28672]",
            "tokens": T, "bytes_per_step": step_bytes, "buffer_sets": len(sets),
            "buffer_set_bytes": set_bytes, "cache": "cold (rotating buffer sets)",
            "frac_of_hbm_peak": round(value / HBM_PEAK_GBS, 4),
            "gpu_ms_per_step_events": round(gpu_ms / args.steps, 5),
            "wall_ms_per_step": round(wall * 1e3 / args.steps, 5),
            "device": torch.cuda.get_device_name(0),
        },
        "roofline": roofline,
        "cpu_baseline": cpu,
        "per_op": per_op,
        "other_configs": other_configs,
        "moe_layer": moe_layer,
        "plain_copy_same_bytes_cold": copy_ref,
    }
    print(json.dumps(out))


if __name__ == "__main__":
    main()
