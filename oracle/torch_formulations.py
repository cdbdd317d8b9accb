"""The ops as ordinary CPU PyTorch tensor code.  TEST INFRASTRUCTURE ONLY.

The reference ships no PyTorch fallback for its csrc ops; these are the plain
tensor-level formulations of what the kernels compute, with the model dtype
kept wherever the kernels' ``scalar_t`` arithmetic rounds
(csrc/layernorm_kernels.cu:18-34, csrc/activation_kernels.cu:9-24,
csrc/pos_encoding_kernels.cu:16-35, csrc/moe_topk_softmax_kernels.cu:261-378,
csrc/moe_align_block_size_kernels.cu:30-108).  Same positional signatures as
the reference's pybind modules; results through out-parameters / in place.
They serve two purposes: an independent check of the C oracle, and the
multi-threaded CPU baseline timed by the benchmark.
"""
import torch
import torch.nn.functional as F


def rms_norm(out, input, weight, epsilon):
    xf = input.float()
    var = xf.pow(2).mean(dim=-1, keepdim=True)
    normed = (xf * torch.rsqrt(var + epsilon)).to(input.dtype)   # first rounding
    out.copy_(normed * weight)                                    # second rounding


def fused_add_rms_norm(input, residual, weight, epsilon):
    # sarathi/model_executor/models/llama.py:248-252
    z = residual + input
    residual.copy_(z)
    rms_norm(input, z, weight, epsilon)


def silu_and_mul(out, input):
    d = input.shape[-1] // 2
    out.copy_(F.silu(input[..., :d]) * input[..., d:])


def gelu_new(out, input):
    x = input
    c = 0.79788456
    out.copy_(0.5 * x * (1.0 + torch.tanh(c * (x + 0.044715 * x * x * x))))


def gelu_fast(out, input):
    x = input
    out.copy_(0.5 * x * (1.0 + torch.tanh(x * 0.79788456 * (1.0 + 0.044715 * x * x))))


def rotary_embedding(positions, query, key, head_size, cos_sin_cache, is_neox):
    rot = cos_sin_cache.shape[1]
    cos, sin = cos_sin_cache[positions].chunk(2, dim=-1)          # [T, rot/2] each
    cos, sin = cos.unsqueeze(1), sin.unsqueeze(1)
    for a in (query, key):
        T = a.shape[0]
        v = a.view(T, -1, head_size) if a.is_contiguous() else a.unflatten(1, (-1, head_size))
        r = v[..., :rot]
        if is_neox:
            x, y = r[..., : rot // 2], r[..., rot // 2:]
        else:
            x, y = r[..., 0::2], r[..., 1::2]
        nx = x * cos - y * sin        # each tensor op rounds once to the dtype
        ny = y * cos + x * sin
        x.copy_(nx)
        y.copy_(ny)


def topk_softmax(topk_weights, topk_indices, token_expert_indices, gating_output):
    k = topk_weights.shape[-1]
    T = gating_output.shape[0]
    p = torch.softmax(gating_output.float(), dim=-1)
    # a stable descending sort gives "larger value first, lower index on ties"
    order = torch.sort(p, dim=-1, descending=True, stable=True)
    topk_weights.copy_(order.values[:, :k])
    topk_indices.copy_(order.indices[:, :k].to(torch.int32))
    j = torch.arange(k, dtype=torch.int32).unsqueeze(0)
    t = torch.arange(T, dtype=torch.int32).unsqueeze(1)
    token_expert_indices.copy_(j * T + t)


def moe_align_block_size(topk_ids, num_experts, block_size, sorted_token_ids, experts_ids,
                         num_tokens_post_pad):
    flat = topk_ids.reshape(-1).to(torch.int64)
    counts = torch.bincount(flat, minlength=num_experts)
    padded = (counts + block_size - 1) // block_size * block_size
    cumsum = torch.zeros(num_experts + 1, dtype=torch.int64)
    cumsum[1:] = torch.cumsum(padded, 0)
    order = torch.argsort(flat, stable=True)                       # ascending index per expert
    starts = torch.zeros(num_experts + 1, dtype=torch.int64)
    starts[1:] = torch.cumsum(counts, 0)
    sorted_e = flat[order]
    dest = cumsum[sorted_e] + (torch.arange(flat.numel()) - starts[sorted_e])
    sorted_token_ids[dest] = order.to(torch.int32)
    nblk = int(cumsum[-1]) // block_size
    blk_start = torch.arange(nblk, dtype=torch.int64) * block_size
    experts_ids[:nblk] = (torch.searchsorted(cumsum, blk_start, right=True) - 1).to(torch.int32)
    num_tokens_post_pad[0] = int(cumsum[-1])


def moe_balance_blocks(topk_ids, num_experts, block_size, granule, rows_per_block=1):
    """Expected output of the library's moe_balance_blocks (no counterpart in the reference), built
    from the ids directly rather than from moe_align_block_size's output: expert e with cnt slots
    gets nb = ceil(cnt / block) blocks; its ceil(cnt / granule) tiles of ``granule`` slots are dealt
    to them as evenly as they go (the first blocks take the odd tiles), slots in ascending order,
    padding (numel) elsewhere.  With rows_per_block = R the tiles are dealt to the expert's nb * R
    ranges of block_size / R slots instead, each range filled from its own start.  Returns (sorted_token_ids, expert_ids, num_tokens_post_pad) as
    Python lists / int, lengths as the reference's caller sizes them
    (sarathi/model_executor/layers/fused_moe/fused_moe.py:191-200)."""
    flat = [int(v) for v in topk_ids.reshape(-1).tolist()]
    numel = len(flat)
    sorted_len = numel + num_experts * (block_size - 1)
    sorted_ids, expert_ids = [], []
    for e in range(num_experts):
        mine = [i for i, v in enumerate(flat) if v == e]
        if not mine:
            continue
        nb = -(-len(mine) // block_size)
        tiles = -(-len(mine) // granule)
        ranges, width = nb * rows_per_block, block_size // rows_per_block
        at = 0
        for j in range(ranges):
            take = (tiles // ranges + (1 if j < tiles % ranges else 0)) * granule
            part = mine[at:at + take]
            at += take
            sorted_ids += part + [numel] * (width - len(part))
        expert_ids += [e] * nb
        assert at >= len(mine)
    post_pad = len(sorted_ids)
    sorted_ids += [numel] * (sorted_len - post_pad)
    return sorted_ids, expert_ids, post_pad


def moe_grouped_gemm(A, B, C, topk_weights, sorted_token_ids, expert_ids, num_tokens_post_padded,
                     num_valid_tokens, block_m, top_k, mul_routed_weight):
    """What the reference's Triton fused_moe_kernel computes
    (sarathi/model_executor/layers/fused_moe/fused_moe.py:84-147): per block of block_m sorted slots,
    rows A[slot // top_k] times B[expert]^T with fp32 accumulation, optionally times the slot's
    routing weight (in fp32), cast to the kernel's compute type — bfloat16 for bfloat16 tensors,
    float16 for everything else, float32 tensors included (fused_moe.py:142, 466) — and stored at
    row `slot` of C."""
    compute_type = torch.bfloat16 if C.dtype == torch.bfloat16 else torch.float16
    n_post = int(num_tokens_post_padded.item())
    Cf = C.view(-1, B.shape[1])
    wflat = topk_weights.reshape(-1)
    for blk in range(n_post // block_m):
        slots = sorted_token_ids[blk * block_m:(blk + 1) * block_m].long()
        slots = slots[slots < num_valid_tokens]
        if slots.numel() == 0:
            continue
        e = int(expert_ids[blk].item())
        acc = A[slots // top_k].float() @ B[e].float().t()
        if mul_routed_weight:
            acc = acc * wflat[slots].float().unsqueeze(1)
        Cf[slots] = acc.to(compute_type).to(C.dtype)


def fused_moe(hidden_states, w1, w2, gating_output, topk, renormalize, topk_weights=None,
              topk_ids=None):
    """Dense statement of the MoE layer the reference's fused_moe computes (fused_moe.py:411-622),
    keeping its intermediate tensors in the model dtype: out[t] = sum_j T(w_j * (h_j @ W2[e_j]^T))
    with h_j = silu_and_mul(T(x_t @ W1[e_j]^T)).  T rounds to the kernel's compute type, which is
    float16 for float32 tensors (fused_moe.py:466)."""
    T, _ = hidden_states.shape
    dt = hidden_states.dtype
    ct = torch.bfloat16 if dt == torch.bfloat16 else torch.float16
    if topk_ids is not None:      # routing decided by the caller (e.g. grouped_topk)
        tw, ti = topk_weights, topk_ids
    else:
        tw = torch.empty((T, topk), dtype=torch.float32)
        ti = torch.empty((T, topk), dtype=torch.int32)
        ts = torch.empty((T, topk), dtype=torch.int32)
        topk_softmax(tw, ti, ts, gating_output.float())
        if renormalize:
            tw = tw / tw.sum(dim=-1, keepdim=True)
    inter = w1.shape[1] // 2
    parts = torch.zeros((T, topk, w2.shape[1]), dtype=dt)
    for e in range(w1.shape[0]):
        tok, j = torch.nonzero(ti == e, as_tuple=True)
        if tok.numel() == 0:
            continue
        gate_up = (hidden_states[tok].float() @ w1[e].float().t()).to(ct).to(dt)
        act = torch.empty((tok.numel(), inter), dtype=dt)
        silu_and_mul(act, gate_up)
        down = (act.float() @ w2[e].float().t()) * tw[tok, j].unsqueeze(1)
        parts[tok, j] = down.to(ct).to(dt)
    return parts.sum(dim=1)


def grouped_topk(gating_output, topk, renormalize, num_expert_group, topk_group):
    """Group-limited routing as the reference states it with tensor ops
    (sarathi/model_executor/layers/fused_moe/fused_moe.py:377-408): softmax; a group's score is
    its best member; the topk_group best groups stay, all other experts' scores become 0; top-k.
    The reference's torch.topk(sorted=False) leaves output order and ties open; this restatement
    (and the kernel) return descending scores with the lower index first among equals, which is
    one of the outcomes the reference allows.  Returns (weights f32 [T, k], ids i32 [T, k])."""
    scores = torch.softmax(gating_output.float(), dim=-1)
    T, E = scores.shape
    per_group = E // num_expert_group
    weights = torch.empty((T, topk), dtype=torch.float32)
    ids = torch.empty((T, topk), dtype=torch.int32)
    for t in range(T):
        row = scores[t]
        best_of_group = [float(row[g * per_group:(g + 1) * per_group].max())
                         for g in range(num_expert_group)]
        order = sorted(range(num_expert_group), key=lambda g: (-best_of_group[g], g))
        kept = set(order[:topk_group])
        masked = [float(row[e]) if (e // per_group) in kept else 0.0 for e in range(E)]
        pick = sorted(range(E), key=lambda e: (-masked[e], e))[:topk]
        for j, e in enumerate(pick):
            weights[t, j] = row[e] if (e // per_group) in kept else 0.0
            ids[t, j] = e
    if renormalize:
        weights = weights / weights.sum(dim=-1, keepdim=True)
    return weights, ids
