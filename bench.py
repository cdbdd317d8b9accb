"""Benchmark of the fused layer ops on the Llama-3-8B 2304-token hybrid batch (one MI355X).

A "step" is one pass of a decoder layer's element-wise chain over one hybrid batch
(2048 prefill tokens + 256 decode tokens), in layer order:

    fused_add_rms_norm [2304, 4096]            (input layernorm with the residual add fused in)
    rotary_embedding   q [2304, 32*128], k [2304, 8*128], views of a packed [2304, 6144] qkv
    fused_add_rms_norm [2304, 4096]            (post-attention layernorm)
    silu_and_mul       [2304, 2*14336] -> [2304, 14336]

All inputs are resident in HBM before the timed region.  Every step of the timed region (and of
the warm-up) has its own freshly drawn N(0, 1) buffers, up to 256 sets (beyond that they are
re-used in turn), so no value is fed through the chain twice and every read misses the 256 MB
Infinity Cache ("cold").  `value` is the step's algorithmic bytes divided by the step time.

Sections (--section, comma separated, default all):
  headline  the timed chain (`value`), `per_op` for the four ops of the chain plus rms_norm alone
            (cold ring and, unless --no-warm, warm = same buffers every call) and `roofline`
  ceiling   what the memory system gives a launch that only moves the same bytes: a plain copy in
            every launch shape of the streaming kernels (1 to 48 KiB per one-wave workgroup), the
            fastest shape taken as the ceiling, and the launch floor (back-to-back launches of a
            one-row rms_norm)
  kv        paged KV-cache append alone and fused with the rotary embedding
  routing   topk_softmax, moe_align_block_size, fused_topk_align at the Mixtral shape
  other     the rest of the module surface at T = 2304, token counts off the multiples of 256
            (T = 2248, 2560), the CPU-sized fused_add_rms_norm [512, 4096] and the Llama-3-70B
            widths at T = 4608
  moe       fused_moe forward and its grouped GEMMs at the Mixtral-8x7B layer shape (MFMA-bound;
            beside the headline, not in it)
  cpu       `cpu_baseline`: the PyTorch CPU formulation of the same step on the host cores, and a
            CPU column for the per-op tables
  models    (only when named; not part of "all") the four layer ops at the layer shapes of the model
            families the reference serves, full width and tensor-parallel shards, at 1024, 2304 and
            4608 tokens
Per-op figures: `us` is the average over >= 100 back-to-back launches between two HIP events on
the launch stream; `us_event_pair_median` is the median over the same number of launches with an
event pair around every single call (it includes the events' own cost, about 1 us).  `roofline`
describes the dominant kernel of the step, silu_and_mul; its `traffic` is read from the committed
rocprofv3 --pmc summary under profiles/ (counters cannot be read from inside this script) and is
null when that file is absent.

--calibrate-copy additionally runs a plain device-to-device copy of a known size (256 MiB,
torch's copy kernel) so that a `rocprofv3 --pmc FETCH_SIZE` / `WRITE_SIZE` run of this script can
scale the counters by what they read for a known amount of traffic.

Prints ONE JSON line.
"""
import argparse
import json
import os
import re
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, "sarathi-serve_amd"), os.path.join(ROOT, "tests")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

HBM_PEAK_GBS = 8000.0
MFMA_PEAK_TFLOPS = 2500.0
SECTIONS = ("headline", "ceiling", "kv", "routing", "other", "moe", "cpu")
EXTRA_SECTIONS = ("models",)   # run only when named

T, H, NQ, NKV, D, DFF = 2304, 4096, 32, 8, 128, 14336
PREFILL = 2048
BF16 = 2
MAX_STEP_SETS = 256           # own buffers for this many steps, then re-use
MIN_REPS = 100                # floor of the per-op timing loops, whatever --steps says
COLD_FOOTPRINT = 640e6        # a ring of argument sets is at least this large

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

# HBM bytes per launch of the dominant kernel, as the committed rocprofv3 --pmc summary states
# them (FETCH_SIZE and WRITE_SIZE, each scaled by what it reads for a plain 256 MiB copy)
TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "headline_kernels_llama3_8b_t2304_pmc_fetch_write.txt")


def measured_traffic(kernel):
    """`<kernel> ... hbm_bytes_per_launch=<int>` from the committed PMC summary, or None."""
    try:
        with open(TRAFFIC_PROFILE) as f:
            for line in f:
                if line.startswith(kernel):
                    m = re.search(r"hbm_bytes_per_launch=(\d+)", line)
                    if m:
                        return int(m.group(1))
    except OSError:
        pass
    return None


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--section", default="all",
                    help="comma-separated subset of: " + ", ".join(SECTIONS) + " (default all)")
    ap.add_argument("--no-warm", action="store_true",
                    help="skip the warm (same buffers every call) per-op loops, so that every "
                         "launch of a profiled run is a cold one")
    ap.add_argument("--no-cpu-baseline", action="store_true", help="same as leaving out 'cpu'")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also launch a 256 MiB plain copy (counter calibration for --pmc runs)")
    ap.add_argument("--moe-data", choices=["random", "constant"], default="random",
                    help="moe section: constant = every activation and weight holds the same value "
                         "(far fewer bits toggle per operation: shows how much of the gap to the "
                         "nominal MFMA peak is the clock the chip sustains under switching power)")
    ap.add_argument("--moe-routing", choices=["random", "balanced"], default="random",
                    help="moe section: random = N(0,1) router logits (experts get unequal shares, "
                         "as in a real batch); balanced = every expert gets exactly tokens * top_k / "
                         "experts slots (no partly filled slot blocks): shows what the imbalance costs")
    ap.add_argument("--moe-balance", choices=["on", "off"], default="off",
                    help="moe section: spread every expert's slots evenly over its slot blocks before "
                         "the GEMMs (layers.balance_blocks) or leave moe_align_block_size's greedy fill "
                         "(the library's default)")
    ap.add_argument("--moe-riders", choices=["on", "off"], default="on",
                    help="moe section, row-major weights at 256-slot blocks: the slots of an expert's "
                         "partly filled last block ride with the workgroups of its full blocks "
                         "and the other experts' slots are spread evenly over their blocks "
                         "(moe_ops.moe_plan_blocks; the library's default), or blocks stay as "
                         "moe_align_block_size fills them")
    ap.add_argument("--moe-block-m", type=int, default=0,
                    help="moe section: slot-block size of the grouped GEMMs (0 = the library's choice)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this op library runs on one GPU; --gpus must be 1 "
                 "(the ops are per-token and never communicate)")
    want = set(SECTIONS) if args.section == "all" else set(args.section.split(","))
    unknown = want - set(SECTIONS) - set(EXTRA_SECTIONS)
    if unknown:
        sys.exit("bench.py: unknown section(s) %s; choose from %s"
                 % (sorted(unknown), SECTIONS + EXTRA_SECTIONS))
    if args.no_cpu_baseline:
        want.discard("cpu")

    import torch
    import sarathi_amd as ops          # raises if the HIP extension is missing
    from helpers import THETA_LLAMA3, cos_sin_cache, gen, hybrid_positions, randn

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    LN, ACT, ROPE, MOE = ops.layernorm_ops, ops.activation_ops, ops.pos_encoding_ops, ops.moe_ops
    KV = ops.kv_cache_ops
    bf16 = torch.bfloat16
    torch.manual_seed(1)
    reps = max(args.steps, MIN_REPS)

    def dev_randn(shape):      # timing inputs: drawn on the device, N(0, 1) -> bf16
        return torch.randn(shape, device=dev, dtype=torch.float32).to(bf16)

    g = gen(1)
    cache_cpu = cos_sin_cache(8192, D, THETA_LLAMA3, bf16)
    cache_dev = cache_cpu.to(dev)
    pos_dev = hybrid_positions(T, PREFILL, g).to(dev)
    w_dev = randn((H,), g, mean=1.0, std=0.1).to(dev)
    w2_dev = randn((H,), g, mean=1.0, std=0.1).to(dev)

    def frac_row(nbytes, us):
        gbs = nbytes / us * 1e-3
        return {"us": round(us, 3), "GBps": round(gbs, 1), "frac_of_peak": round(gbs / HBM_PEAK_GBS, 4)}

    def time_op(fn, ring, n=None):
        """(avg us over back-to-back launches, median us of per-call event pairs)."""
        n = n or reps
        m = len(ring)
        for i in range(max(m, 5)):
            fn(ring[i % m])
        torch.cuda.synchronize()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for i in range(n):
            fn(ring[i % m])
        b.record()
        torch.cuda.synchronize()
        avg = a.elapsed_time(b) * 1e3 / n
        pairs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
                 for _ in range(n)]
        for i, (s, e) in enumerate(pairs):
            s.record()
            fn(ring[i % m])
            e.record()
        torch.cuda.synchronize()
        each = sorted(s.elapsed_time(e) * 1e3 for s, e in pairs)
        return avg, each[len(each) // 2]

    def ring_of(nbytes, make, least=4):
        return [make() for _ in range(max(least, int(COLD_FOOTPRINT // nbytes) + 1))]

    def op_rows(name, nbytes, ring, fn, latency_bound=False):
        row = {"bytes": nbytes}
        if name.split(" ")[0] in REFERENCE_LABELS:
            row["reference_label"] = REFERENCE_LABELS[name.split(" ")[0]]
        for label in ("cold", "warm"):
            if label == "cold" and latency_bound:
                continue   # 0.07-0.3 MB working sets: launch-latency-bound, one (warm) figure
            if label == "warm" and args.no_warm and not latency_bound:
                continue
            avg, med = time_op(fn, ring if label == "cold" else ring[:1])
            row[label] = frac_row(nbytes, avg)
            row[label]["us_event_pair_median"] = round(med, 3)
        if not latency_bound:
            row["ring_sets"] = len(ring)
        row["timed_launches"] = reps
        return row

    out = {
        "metric": "achieved HBM GB/s (% of peak) per fused op at 2304-token hybrid batch",
        "value": None, "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": None, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {
            "workload": "Llama-3-8B hybrid batch, T=2304 (2048-token prefill chunk at positions "
                        "4096..6143 + 256 decode tokens): fused_add_rms_norm[2304,4096] -> neox "
                        "rotary_embedding(q[2304,4096], k[2304,1024], packed qkv, theta=5e5) -> "
                        "fused_add_rms_norm -> silu_and_mul[2304,28672]",
            "tokens": T, "sections": sorted(want), "device": torch.cuda.get_device_name(0)},
        "roofline": None, "cpu_baseline": None,
    }
    per_op = {}
    step_bytes = 2 * BYTES["fused_add_rms_norm"] + BYTES["rotary_embedding"] + BYTES["silu_and_mul"]

    # =========================================================================== headline
    if "headline" in want:
        def make_set():
            s = {"x": dev_randn((T, H)), "res": dev_randn((T, H)),
                 "qkv": dev_randn((T, (NQ + 2 * NKV) * D)), "gate_up": dev_randn((T, 2 * DFF)),
                 "act": torch.empty((T, DFF), dtype=bf16, device=dev)}
            s["q"], s["k"], _ = s["qkv"].split([NQ * D, NKV * D, NKV * D], dim=-1)
            return s

        n_sets = min(args.steps + args.warmup, MAX_STEP_SETS)
        sets = [make_set() for _ in range(n_sets)]
        set_bytes = sum(v.numel() * v.element_size() for k, v in sets[0].items() if k not in ("q", "k"))

        def step(s):
            LN.fused_add_rms_norm(s["x"], s["res"], w_dev, 1e-5)
            ROPE.rotary_embedding(pos_dev, s["q"], s["k"], D, cache_dev, True)
            LN.fused_add_rms_norm(s["x"], s["res"], w2_dev, 1e-5)
            ACT.silu_and_mul(s["act"], s["gate_up"])

        # ---- the timed region: exactly --steps steps, each on its own buffers (cold) ----
        for i in range(args.warmup):
            step(sets[i % n_sets])
        torch.cuda.synchronize()
        t0 = torch.cuda.Event(enable_timing=True)
        t1 = torch.cuda.Event(enable_timing=True)
        wall0 = time.perf_counter()
        t0.record()
        for i in range(args.steps):
            step(sets[(args.warmup + i) % n_sets])
        t1.record()
        torch.cuda.synchronize()
        wall = time.perf_counter() - wall0
        gpu_ms = t0.elapsed_time(t1)
        ms_per_step = max(gpu_ms, wall * 1e3) / args.steps
        value = step_bytes / (ms_per_step * 1e-3) * 1e-9
        out["value"] = round(value, 1)
        out["ms_per_step"] = round(ms_per_step, 5)
        out["config"].update({
            "bytes_per_step": step_bytes, "buffer_sets": n_sets, "buffer_set_bytes": set_bytes,
            "cache": "cold (every step of warm-up and timed region on its own freshly drawn "
                     "N(0,1) buffers, up to %d sets)" % MAX_STEP_SETS,
            "frac_of_hbm_peak": round(value / HBM_PEAK_GBS, 4),
            "gpu_ms_per_step_events": round(gpu_ms / args.steps, 5),
            "wall_ms_per_step": round(wall * 1e3 / args.steps, 5)})
        del sets
        torch.cuda.empty_cache()

        # ---- per-op: >= 100 launches over a cold ring of argument sets, and warm ----
        def mk_norm():
            return (dev_randn((T, H)), dev_randn((T, H)))

        def mk_rope():
            qkv = dev_randn((T, (NQ + 2 * NKV) * D))
            q, k, _ = qkv.split([NQ * D, NKV * D, NKV * D], dim=-1)
            return (qkv, q, k)

        def mk_silu():
            return (dev_randn((T, 2 * DFF)), torch.empty((T, DFF), dtype=bf16, device=dev))

        # (the in-place ops re-use their ring sets: a set sees about reps / ring_sets calls)
        table = [
            ("fused_add_rms_norm", mk_norm, lambda a: LN.fused_add_rms_norm(a[0], a[1], w_dev, 1e-5)),
            ("rms_norm", mk_norm, lambda a: LN.rms_norm(a[1], a[0], w_dev, 1e-5)),
            ("rotary_embedding", mk_rope,
             lambda a: ROPE.rotary_embedding(pos_dev, a[1], a[2], D, cache_dev, True)),
            ("silu_and_mul", mk_silu, lambda a: ACT.silu_and_mul(a[1], a[0])),
        ]
        for name, make, fn in table:
            ring = ring_of(BYTES[name], make)
            per_op[name] = op_rows(name, BYTES[name], ring, fn)
            del ring
            torch.cuda.empty_cache()

        silu = per_op["silu_and_mul"]["cold"]
        traffic = measured_traffic("silu_and_mul_kernel")
        out["roofline"] = {
            "kernel": "silu_and_mul_kernel (bf16, [2304, 28672] -> [2304, 14336])",
            "bound": "hbm", "achieved": silu["GBps"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
            "frac": silu["frac_of_peak"], "traffic": traffic,
            "traffic_source": ("profiles/" + os.path.basename(TRAFFIC_PROFILE) + " (rocprofv3 --pmc "
                               "FETCH_SIZE / WRITE_SIZE, scaled by a 256 MiB copy)")
            if traffic is not None else None,
            "bytes_per_launch": BYTES["silu_and_mul"], "avg_launch_us": silu["us"],
            "timing": "%d back-to-back launches between two HIP events on the launch stream, rotating "
                      "over %d cold buffer sets" % (reps, per_op["silu_and_mul"]["ring_sets"]),
        }

    # =========================================================================== ceiling
    if "ceiling" in want:
        # What the memory system gives a launch that only moves the same number of bytes: a plain
        # copy (half the op's bytes in, half out, same cache policies) in every launch shape the
        # library's streaming kernels use, from 1 KiB per one-wave workgroup to 48 KiB; the fastest
        # shape is the ceiling of that launch size.  (moe_sum with top_k = 1, the library's own
        # copy-shaped kernel, is listed beside it.)
        from sarathi_amd import stream_ops
        ceiling = {}
        for name in ("rms_norm", "rotary_embedding", "fused_add_rms_norm", "silu_and_mul"):
            rows = BYTES[name] // 2 // (H * BF16)
            nbytes = 2 * rows * H * BF16
            ring = ring_of(nbytes, lambda: (dev_randn((rows, 1, H)),
                                            torch.empty((rows, H), dtype=bf16, device=dev)))
            shapes = {}
            for kib in stream_ops.COPY_SHAPES_KIB:
                avg, _ = time_op(lambda a: stream_ops.stream_copy(a[1], a[0], kib), ring)
                shapes["%d KiB per wave" % kib] = round(avg, 3)
            best = min(shapes, key=shapes.get)
            avg, med = time_op(lambda a: MOE.moe_sum(a[0], a[1]), ring)
            ceiling["copy of %s's bytes" % name] = dict(
                frac_row(nbytes, shapes[best]), bytes=nbytes, best_shape=best,
                kernel="stream_copy_kernel (one-wave workgroups, all loads before the first store)",
                us_by_shape=shapes,
                moe_sum_top1=dict(frac_row(nbytes, avg), us_event_pair_median=round(med, 3)))
            del ring
            torch.cuda.empty_cache()
        tiny_in, tiny_out = dev_randn((1, 64)), torch.empty((1, 64), dtype=bf16, device=dev)
        tiny_w = dev_randn((64,))
        avg, med = time_op(lambda a: LN.rms_norm(tiny_out, tiny_in, tiny_w, 1e-5), [None])
        ceiling["launch floor"] = {
            "us": round(avg, 3), "us_event_pair_median": round(med, 3),
            "kernel": "rms_norm on one row of 64 elements, back-to-back launches on one stream"}
        out["streaming_ceiling_cold"] = ceiling

    # =========================================================================== kv
    if "kv" in want:
        # paged KV cache of the hybrid batch: one prompt chunk continuing a 4096-token request and
        # 256 decode requests with contexts of 1..3000 tokens, pages handed out in random order
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
            cache = torch.empty((touched.numel(), 2, PAGE, NKV, D), dtype=bf16, device=dev)
            return (qkv, q, k, v, (cache[:, 0], cache[:, 1]))   # K / V planes split once, not per call

        kv_table = [
            ("append_paged_kv_cache",
             lambda a: KV.append_paged_kv_cache(
                 a[2], a[3], meta.append_batch_indices, meta.append_positions, a[4],
                 kv_indices_dense, meta.append_kv_page_indptr)),
            ("rotary_embedding_append_paged_kv",
             lambda a: KV.rotary_embedding_append_paged_kv(
                 pos_dev, a[1], a[2], a[3], D, cache_dev, True, meta.append_batch_indices,
                 meta.append_positions, a[4], kv_indices_dense, meta.append_kv_page_indptr)),
            ("append_paged_kv_cache (slot mapping)",
             lambda a: KV.append_paged_kv_cache(
                 a[2], a[3], meta.append_batch_indices, meta.append_positions, a[4],
                 kv_indices_dense, meta.append_kv_page_indptr, slot_mapping=slots_dense)),
            ("rotary_embedding_append_paged_kv (slot mapping)",
             lambda a: KV.rotary_embedding_append_paged_kv(
                 pos_dev, a[1], a[2], a[3], D, cache_dev, True, meta.append_batch_indices,
                 meta.append_positions, a[4], kv_indices_dense, meta.append_kv_page_indptr,
                 slot_mapping=slots_dense)),
        ]
        for name, fn in kv_table:
            ring = ring_of(BYTES[name], mk_kv)
            per_op[name] = op_rows(name, BYTES[name], ring, fn)
            del ring
            torch.cuda.empty_cache()

    # =========================================================================== routing
    gating = tw = ti = ts = sorted_ids = expert_ids = post_pad = None
    if "routing" in want or "cpu" in want:
        mg = gen(3)
        gating = torch.randn((MOE_T, MOE_E), generator=mg, dtype=torch.float32).to(dev)
        tw = torch.empty((MOE_T, MOE_K), dtype=torch.float32, device=dev)
        ti = torch.empty((MOE_T, MOE_K), dtype=torch.int32, device=dev)
        ts = torch.empty((MOE_T, MOE_K), dtype=torch.int32, device=dev)
        MOE.topk_softmax(tw, ti, ts, gating)
        sorted_ids = torch.empty((_moe_sorted,), dtype=torch.int32, device=dev)
        expert_ids = torch.empty(((_moe_sorted + MOE_B - 1) // MOE_B,), dtype=torch.int32, device=dev)
        post_pad = torch.empty((1,), dtype=torch.int32, device=dev)
    if "routing" in want:
        routing = [
            ("topk_softmax", lambda a: MOE.topk_softmax(tw, ti, ts, gating)),
            ("moe_align_block_size", lambda a: MOE.moe_align_block_size_filled(
                ti, MOE_E, MOE_B, sorted_ids, expert_ids, post_pad)),
            ("fused_topk_align", lambda a: MOE.fused_topk_align(
                tw, ti, ts, gating, True, MOE_B, sorted_ids, expert_ids, post_pad, True)),
        ]
        for name, fn in routing:
            per_op[name] = op_rows(name, BYTES[name], [None], fn, latency_bound=True)

    if args.calibrate_copy:
        src = torch.empty((256 << 20) // 2, dtype=bf16, device=dev).fill_(1.0)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    # =========================================================================== other
    other_configs = None
    if "other" in want or "models" in want:
        # C1: the fused norm at the 512-token shape that is also the CPU-sized case; C5: the four
        # ops at Llama-3-70B widths, T = 4608 (4096-token chunk + 512 decodes), one GPU, unsharded.
        def measure_shape(Tn, Hn, nq, nkv, dff, which, prefill=None, head=D):
            rows = {}
            wn = dev_randn((Hn,))
            posn = hybrid_positions(Tn, prefill or Tn - Tn // 9, gen(4), prefill_start=4096,
                                    max_pos=8192).to(dev) if any("rotary" in w for w in which) else None
            cache_n = cache_dev if head == D else cos_sin_cache(8192, head, THETA_LLAMA3, bf16).to(dev)
            if "rotary_embedding + KV append" in which:
                # one request that appends all Tn tokens to pages of 16 entries in shuffled order
                n_pages = (Tn + 15) // 16
                ap_b = torch.zeros(Tn, dtype=torch.int32, device=dev)
                ap_pos = torch.arange(Tn, dtype=torch.int32, device=dev)
                ap_pages = torch.randperm(n_pages, generator=gen(7)).to(torch.int32).to(dev)
                ap_indptr = torch.tensor([0, n_pages], dtype=torch.int32, device=dev)

                def mk_append():
                    q, k, v = dev_randn((Tn, (nq + 2 * nkv) * head)).split(
                        [nq * head, nkv * head, nkv * head], dim=-1)
                    cache = torch.empty((n_pages, 2, 16, nkv, head), dtype=bf16, device=dev)
                    return (q, k, v, (cache[:, 0], cache[:, 1]))
            plan = {
                "fused_add_rms_norm": (4 * Tn * Hn * BF16 + Hn * BF16,
                                       lambda: (dev_randn((Tn, Hn)), dev_randn((Tn, Hn))),
                                       lambda a: LN.fused_add_rms_norm(a[0], a[1], wn, 1e-5)),
                "rms_norm": (2 * Tn * Hn * BF16 + Hn * BF16,
                             lambda: (dev_randn((Tn, Hn)), dev_randn((Tn, Hn))),
                             lambda a: LN.rms_norm(a[1], a[0], wn, 1e-5)),
                "rotary_embedding": (2 * Tn * (nq + nkv) * head * BF16 + Tn * 8 + Tn * head * BF16,
                                     # q and k views of a packed qkv buffer, cut outside the timed call
                                     lambda: dev_randn((Tn, (nq + 2 * nkv) * head)).split(
                                         [nq * head, nkv * head, nkv * head], dim=-1)[:2],
                                     lambda a: ROPE.rotary_embedding(posn, a[0], a[1], head, cache_n,
                                                                     True)),
                "rotary_embedding + KV append": (
                    (2 * Tn * nq + 4 * Tn * nkv) * head * BF16 + 24 * Tn + Tn * head * BF16,
                    lambda: mk_append(),
                    lambda a: KV.rotary_embedding_append_paged_kv(
                        posn, a[0], a[1], a[2], head, cache_n, True, ap_b, ap_pos, a[3], ap_pages,
                        ap_indptr)),
                "silu_and_mul": (3 * Tn * dff * BF16,
                                 lambda: (dev_randn((Tn, 2 * dff)),
                                          torch.empty((Tn, dff), dtype=bf16, device=dev)),
                                 lambda a: ACT.silu_and_mul(a[1], a[0])),
                "gelu_new": (2 * Tn * dff * BF16,
                             lambda: (dev_randn((Tn, dff)),
                                      torch.empty((Tn, dff), dtype=bf16, device=dev)),
                             lambda a: ACT.gelu_new(a[1], a[0])),
                "gelu_fast": (2 * Tn * dff * BF16,
                              lambda: (dev_randn((Tn, dff)),
                                       torch.empty((Tn, dff), dtype=bf16, device=dev)),
                              lambda a: ACT.gelu_fast(a[1], a[0])),
                "rotary_embedding (GPT-J layout)": (
                    2 * Tn * (nq + nkv) * D * BF16 + Tn * 8 + Tn * D * BF16,
                    lambda: dev_randn((Tn, (nq + 2 * nkv) * D)).split([nq * D, nkv * D, nkv * D],
                                                                      dim=-1)[:2],
                    lambda a: ROPE.rotary_embedding(posn, a[0], a[1], D, cache_dev, False)),
            }
            for name in which:
                nbytes, make, fn = plan[name]
                r = ring_of(nbytes, make, least=2)
                avg, med = time_op(fn, r)
                rows[name] = {"bytes": nbytes, "cold": dict(frac_row(nbytes, avg),
                                                            us_event_pair_median=round(med, 3)),
                              "ring_sets": len(r), "timed_launches": reps}
                del r
                torch.cuda.empty_cache()
            return rows

    if "other" in want:
        other_configs = {
            "rest of the module surface at the Llama-3-8B batch, T=2304: gelu_new / gelu_fast "
            "[2304, 14336], rotary_embedding with interleaved (GPT-J) pairs":
                measure_shape(T, H, NQ, NKV, DFF,
                              ["gelu_new", "gelu_fast", "rotary_embedding (GPT-J layout)"]),
            "batches off the multiples of 256 tokens: 2048-token chunk + 200 decodes (T=2248)":
                measure_shape(2248, H, NQ, NKV, DFF,
                              ["fused_add_rms_norm", "rms_norm", "rotary_embedding"], prefill=PREFILL),
            "2048-token chunk + 512 decodes (T=2560)":
                measure_shape(2560, H, NQ, NKV, DFF,
                              ["fused_add_rms_norm", "rms_norm", "rotary_embedding"], prefill=PREFILL),
            "fused_add_rms_norm [512, 4096] (CPU-sized case)":
                measure_shape(512, 4096, 32, 8, 14336, ["fused_add_rms_norm"]),
            "Llama-3-70B widths, T=4608: norm [4608, 8192], rope q[4608, 8192] k[4608, 1024], "
            "silu_and_mul [4608, 57344]":
                measure_shape(4608, 8192, 64, 8, 28672,
                              ["fused_add_rms_norm", "rms_norm", "rotary_embedding", "silu_and_mul"]),
        }
        out["other_configs"] = other_configs

    # =========================================================================== models
    if "models" in want:
        # Layer shapes of the model families the reference serves (sarathi/model_executor/models/):
        # hidden, query + key heads of head_size, intermediate size (0: no gated activation); "tp N"
        # is one GPU's share under the reference's tensor parallelism, whose norms see the full
        # hidden size.  A 2048-token chunk (or all but a ninth of the batch) plus decodes.
        shapes = [
            ("Llama-3-8B / Mistral-7B / Mixtral-8x7B", 4096, 32, 8, 128, 14336),
            ("Llama-2-7B", 4096, 32, 32, 128, 11008),
            ("Llama-2-13B / InternLM-20B", 5120, 40, 40, 128, 13824),
            ("Yi-34B", 7168, 56, 8, 128, 20480),
            ("Llama-3-70B", 8192, 64, 8, 128, 28672),
            ("Qwen-72B", 8192, 64, 64, 128, 24576),
            ("Falcon-7B", 4544, 71, 1, 64, 0),
            ("Falcon-40B", 8192, 128, 8, 64, 0),
            ("Llama-3-70B tp 4", 8192, 16, 2, 128, 7168),
            ("Llama-3-70B tp 8", 8192, 8, 1, 128, 3584),
        ]
        models = {}
        for name, Hn, nq, nkv, head, dff in shapes:
            which = (["rms_norm", "fused_add_rms_norm", "rotary_embedding", "rotary_embedding + KV append"]
                     + (["silu_and_mul"] if dff else []))
            models[name] = {
                "hidden": Hn, "heads": [nq, nkv], "head_size": head, "intermediate": dff,
                "tokens": {str(Tn): measure_shape(Tn, Hn, nq, nkv, dff, which,
                                                  prefill=min(2048, Tn - Tn // 9), head=head)
                           for Tn in (1024, 2304, 4608)}}
        out["model_shapes"] = models

    # =========================================================================== moe
    if "moe" in want:
        # The MoE layer either side of the routing ops: fused_moe forward (routing, slot sort, both
        # grouped expert GEMMs with the activation in the first one's epilogue, top-k sum) at the
        # Mixtral-8x7B layer shape, and the GEMMs on their own at 4096 tokens for both weight
        # layouts.  MFMA-bound at large batches, weight-streaming-bound at decode sizes.
        import importlib
        from sarathi_amd import layers
        importlib.import_module("sarathi_amd.layers.fused_moe").BALANCE_BLOCKS = args.moe_balance == "on"
        importlib.import_module("sarathi_amd.layers.fused_moe").RIDERS = args.moe_riders == "on"
        E, k, Hm, I = 8, 2, 4096, 14336

        def timeit_ms(fn, n=20):
            for _ in range(3):
                fn()
            torch.cuda.synchronize()
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            for _ in range(n):
                fn()
            b.record()
            torch.cuda.synchronize()
            return a.elapsed_time(b) / n

        def tflops(flop, ms):
            return {"ms": round(ms, 4), "TFLOPs": round(flop / ms * 1e-9, 1),
                    "frac_of_mfma_peak": round(flop / ms * 1e-9 / MFMA_PEAK_TFLOPS, 4)}

        def router_logits(Tn):
            if args.moe_routing == "random":
                return torch.randn((Tn, E), device=dev, dtype=torch.float32)
            t = torch.arange(Tn, device=dev)
            lg = torch.zeros((Tn, E), device=dev, dtype=torch.float32)
            for j in range(k):                      # token t -> experts (k t + j) mod E
                lg[t, (k * t + j) % E] = float(k - j)
            return lg

        w1 = (torch.randn((E, 2 * I, Hm), device=dev, dtype=torch.float32) * Hm ** -0.5).to(bf16)
        w2 = (torch.randn((E, Hm, I), device=dev, dtype=torch.float32) * I ** -0.5).to(bf16)
        if args.moe_data == "constant":
            w1.fill_(0.0078125)
            w2.fill_(0.0078125)
        forward = {}
        for Tn in (16, 1024, 2048, 2304, 4096):
            x = torch.randn((Tn, Hm), device=dev, dtype=torch.float32).to(bf16)
            if args.moe_data == "constant":
                x.fill_(0.0078125)
            logits = router_logits(Tn)
            ms = timeit_ms(lambda: layers.fused_moe(x, w1, w2, logits, k, True))
            row = tflops(2.0 * Tn * k * 3 * I * Hm, ms)
            row["weight_stream_TBps"] = round((E * 3 * I * Hm * 2) / ms * 1e-9, 2)
            forward["%d tokens" % Tn] = row

        Tn = 4096
        x = torch.randn((Tn, Hm), device=dev, dtype=torch.float32).to(bf16)
        if args.moe_data == "constant":
            x.fill_(0.0078125)
        logits = router_logits(Tn)
        tw_m, ti_m = layers.fused_topk(x, logits, k, True)
        c1 = torch.empty((Tn, k, 2 * I), device=dev, dtype=bf16)
        c2 = torch.empty((Tn * k, I), device=dev, dtype=bf16)
        c3 = torch.empty((Tn, k, Hm), device=dev, dtype=bf16)
        f1, f2 = 2.0 * Tn * k * Hm * 2 * I, 2.0 * Tn * k * I * Hm
        gemms = {}
        for label in ("row_major", "packed"):
            config = dict(layers.try_get_optimal_moe_config((E, 2 * I, Hm), (E, Hm, I), k, Tn,
                                                            packed=label == "packed"))
            if args.moe_block_m:
                config["BLOCK_SIZE_M"] = args.moe_block_m
            bm = config["BLOCK_SIZE_M"]
            s_ids, e_ids, p_pad = layers.moe_align_block_size(ti_m, bm, E)
            if args.moe_balance == "on":
                s_ids = layers.balance_blocks(s_ids, e_ids, p_pad, bm, E, Tn * k, packed=label == "packed")
            if label == "packed":      # re-tile once, then drop the row-major copies
                p1, p2 = layers.pack_expert_weights(w1), layers.pack_expert_weights(w2)
                b1, b2, pk, wa, wb = p1.data, p2.data, True, p1, p2
                del w1, w2
                torch.cuda.empty_cache()
            else:
                b1, b2, pk, wa, wb = w1, w2, False, w1, w2
            rd = None
            if args.moe_riders == "on" and label == "row_major" and bm == 256 and args.moe_balance != "on":
                rd = torch.empty((e_ids.numel(),), dtype=torch.int32, device=dev)
                planned = torch.empty_like(s_ids)     # what fused_experts does: riders, even fill for the rest
                MOE.moe_plan_blocks(s_ids, planned, e_ids, p_pad, E, bm, Tn * k, rd)
                s_ids = planned
            ms1 = timeit_ms(lambda: MOE.moe_grouped_gemm(
                x, b1, c1, tw_m, s_ids, e_ids, p_pad, Tn * k, bm, k, False, pk, 2 * I, False, rd))
            ms_act = timeit_ms(lambda: ACT.silu_and_mul(c2, c1.view(-1, 2 * I)))
            ms1s = timeit_ms(lambda: MOE.moe_grouped_gemm(
                x, b1, c2, tw_m, s_ids, e_ids, p_pad, Tn * k, bm, k, False, pk, 2 * I, True, rd))
            ACT.silu_and_mul(c2, c1.view(-1, 2 * I))
            ms2 = timeit_ms(lambda: MOE.moe_grouped_gemm(
                c2, b2, c3, tw_m, s_ids, e_ids, p_pad, Tn * k, bm, 1, True, pk, Hm, False, rd))
            ms_all = timeit_ms(lambda: layers.fused_moe(x, wa, wb, logits, k, True,
                                                        override_config=config))
            gemms[label] = {
                "block_m": bm, "gemm_w1": tflops(f1, ms1), "silu_and_mul": {"ms": round(ms_act, 4)},
                "gemm_w1_with_silu_and_mul_epilogue": tflops(f1, ms1s), "gemm_w2": tflops(f2, ms2),
                "fused_moe_forward": tflops(f1 + f2, ms_all)}
        del b1, b2, wa, wb
        torch.cuda.empty_cache()
        out["moe_layer"] = {
            "shape": "Mixtral-8x7B MoE layer: 8 experts, top-2, hidden 4096, intermediate 14336, "
                     "bf16, %s data, %s routing, slot blocks %s, back-to-back launches (weights "
                     "warm in L2/MALL as far as they fit)"
                     % (args.moe_data, args.moe_routing,
                        "filled evenly per expert" if args.moe_balance == "on"
                        else "planned per expert (riders or even fill)" if args.moe_riders == "on" else "filled greedily"),
            "peak": "2500 TFLOP/s dense bf16 MFMA; 8 TB/s HBM",
            "fused_moe_forward_row_major": forward, "at_4096_tokens": gemms}

    # =========================================================================== cpu
    if "cpu" in want:
        from oracle import torch_formulations as cpu_ops
        cg = gen(1)
        cx, cr = randn((T, H), cg), randn((T, H), cg)
        cw = randn((H,), cg, mean=1.0, std=0.1)
        cqkv = randn((T, (NQ + 2 * NKV) * D), cg)
        cq, ck, _ = cqkv.split([NQ * D, NKV * D, NKV * D], dim=-1)
        cpos = hybrid_positions(T, PREFILL, cg)
        cgu = randn((T, 2 * DFF), cg)
        cact = torch.empty((T, DFF), dtype=bf16)
        # the CPU chain would feed its own output back in on every repetition: restore the
        # in-place tensors from pristine copies outside the timed part of each repetition
        cx0, cr0, cqkv0 = cx.clone(), cr.clone(), cqkv.clone()

        def cpu_step():
            cpu_ops.fused_add_rms_norm(cx, cr, cw, 1e-5)
            cpu_ops.rotary_embedding(cpos, cq, ck, D, cache_cpu, True)
            cpu_ops.fused_add_rms_norm(cx, cr, cw, 1e-5)
            cpu_ops.silu_and_mul(cact, cgu)

        def restore():
            cx.copy_(cx0)
            cr.copy_(cr0)
            cqkv.copy_(cqkv0)

        cpu_step()
        restore()
        t_start = time.perf_counter()
        cpu_step()
        one = time.perf_counter() - t_start
        n_cpu = max(3, min(2000, int(12.0 / max(one, 1e-3))))      # about 12 s of CPU work
        times = []
        for _ in range(n_cpu):
            restore()
            t_start = time.perf_counter()
            cpu_step()
            times.append(time.perf_counter() - t_start)
        times.sort()
        med = times[len(times) // 2]

        # a CPU column for every op of the tables (median of a few repetitions, same formulations)
        def cpu_us(fn, n=5):
            fn()
            tt = []
            for _ in range(n):
                t_a = time.perf_counter()
                fn()
                tt.append(time.perf_counter() - t_a)
            return round(sorted(tt)[len(tt) // 2] * 1e6, 1)
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
            if name in per_op:
                per_op[name]["cpu_us"] = cpu_us(fn)
        if other_configs is not None:
            c1x, c1r = randn((512, H), cg), randn((512, H), cg)
            other_configs["fused_add_rms_norm [512, 4096] (CPU-sized case)"]["fused_add_rms_norm"][
                "cpu_us"] = cpu_us(lambda: cpu_ops.fused_add_rms_norm(c1x, c1r, cw, 1e-5), n=20)
        out["cpu_baseline"] = {
            "value": round(step_bytes / med * 1e-9, 2), "unit": "GB/s",
            "cores": torch.get_num_threads(), "kind": "port",
            "sample": "%d repetitions of the same 2304-token step (median %.1f ms/step) with the "
                      "PyTorch CPU formulation of the ops (oracle/torch_formulations.py), "
                      "os.cpu_count()=%d" % (n_cpu, med * 1e3, os.cpu_count()),
            "ms_per_step": round(med * 1e3, 2),
        }

    out["per_op"] = per_op
    print(json.dumps(out))


if __name__ == "__main__":
    main()
