"""Eager PyTorch reference implementations of every custom op.

These are the numerics oracle for the HIP/CDNA4 kernels (tests compare the HIP
kernel against these in fp32) and the CPU execution path for GPU-less plumbing
tests. They are NOT the GPU serving path — on a GPU box the HIP extension is
required and ops fail loudly if it is missing (see ops/__init__.py).

Op inventory mirrors the reference's src/parallax_extensions/ops.py kernel set
(paged_attention v1/v2, reshape_and_cache, mla_paged_attention, ...) re-designed
for the [num_blocks, num_kv_heads, block_size, head_dim] MI355X layout.
"""

from __future__ import annotations

from typing import List, Optional, Tuple

import torch


# -- normalization -----------------------------------------------------------------


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float = 1e-6) -> torch.Tensor:
    xf = x.float()
    var = xf.pow(2).mean(dim=-1, keepdim=True)
    out = xf * torch.rsqrt(var + eps) * weight.float()
    return out.to(x.dtype)


def fused_add_rmsnorm(
    x: torch.Tensor, residual: torch.Tensor, weight: torch.Tensor, eps: float = 1e-6
) -> Tuple[torch.Tensor, torch.Tensor]:
    """residual' = x + residual; out = rmsnorm(residual')."""
    new_residual = (x.float() + residual.float()).to(x.dtype)
    return rmsnorm(new_residual, weight, eps), new_residual


# -- rotary embedding ----------------------------------------------------------------


def build_rope_cache(
    max_positions: int,
    rot_dim: int,
    base: float = 10000.0,
    scaling_factor: float = 1.0,
    device: torch.device = torch.device("cpu"),
    inv_freq: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """[max_positions, rot_dim] fp32 cache: cos in [:, :rot_dim//2], sin in [:, rot_dim//2:].
    Precomputed on host per CDNA guide (on-device trig turns RoPE VALU-bound)."""
    if inv_freq is None:
        inv_freq = 1.0 / (
            base ** (torch.arange(0, rot_dim, 2, dtype=torch.float32) / rot_dim)
        )
    t = torch.arange(max_positions, dtype=torch.float32) / scaling_factor
    freqs = torch.outer(t, inv_freq)  # [P, rot_dim/2]
    return torch.cat([freqs.cos(), freqs.sin()], dim=-1).to(device)


def rope_inplace(
    q: torch.Tensor,           # [T, Hq, D]
    k: torch.Tensor,           # [T, Hk, D]
    positions: torch.Tensor,   # [T] int
    cos_sin: torch.Tensor,     # [P, rot_dim] fp32
    is_neox: bool = True,
) -> None:
    rot_dim = cos_sin.shape[-1]
    half = rot_dim // 2
    cs = cos_sin[positions.long()]          # [T, rot_dim]
    cos = cs[:, :half].unsqueeze(1)         # [T, 1, half]
    sin = cs[:, half:].unsqueeze(1)

    def _apply(t: torch.Tensor) -> None:
        # clone: .float() on an fp32 tensor is a VIEW — without the clone the
        # first store below would clobber x1/x2 before o2 is evaluated
        rot = t[..., :rot_dim].clone().float()
        if is_neox:
            x1, x2 = rot[..., :half], rot[..., half:]
            o1 = x1 * cos - x2 * sin
            o2 = x2 * cos + x1 * sin
            t[..., :half] = o1.to(t.dtype)
            t[..., half:rot_dim] = o2.to(t.dtype)
        else:  # interleaved (GPT-J style)
            x1, x2 = rot[..., 0::2], rot[..., 1::2]
            o1 = x1 * cos - x2 * sin
            o2 = x2 * cos + x1 * sin
            t[..., 0:rot_dim:2] = o1.to(t.dtype)
            t[..., 1:rot_dim:2] = o2.to(t.dtype)

    _apply(q)
    if k is not None:
        _apply(k)


# -- KV cache scatter ------------------------------------------------------------------


def reshape_and_cache(
    k: torch.Tensor,             # [T, Hk, D]
    v: torch.Tensor,             # [T, Hk, D]
    k_cache: torch.Tensor,       # [num_blocks, Hk, block_size, D]
    v_cache: torch.Tensor,       # [num_blocks, Hk, D, block_size] (transposed)
    slot_mapping: torch.Tensor,  # [T] int (block*bs + off); -1 = skip (padding)
) -> None:
    block_size = k_cache.shape[2]
    valid = slot_mapping >= 0
    slots = slot_mapping[valid].long()
    blk = slots // block_size
    off = slots % block_size
    k_cache[blk, :, off] = k[valid].to(k_cache.dtype)
    v_cache[blk, :, :, off] = v[valid].to(v_cache.dtype)


def mla_reshape_and_cache(
    kv_latent: torch.Tensor,     # [T, lora_rank]
    k_rope: torch.Tensor,        # [T, rope_dim]
    cache: torch.Tensor,         # [num_blocks, block_size, lora_rank + rope_dim]
    slot_mapping: torch.Tensor,
) -> None:
    block_size = cache.shape[1]
    lora_rank = kv_latent.shape[-1]
    valid = slot_mapping >= 0
    slots = slot_mapping[valid].long()
    blk, off = slots // block_size, slots % block_size
    cache[blk, off, :lora_rank] = kv_latent[valid].to(cache.dtype)
    cache[blk, off, lora_rank:] = k_rope[valid].to(cache.dtype)


# -- attention ---------------------------------------------------------------------------


def _gather_kv(
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    block_table: torch.Tensor,  # [max_blocks] int
    seq_len: int,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Gather one request's KV as [seq_len, Hk, D] (V cache is transposed)."""
    block_size = k_cache.shape[2]
    nb = (seq_len + block_size - 1) // block_size
    blocks = block_table[:nb].long()
    k = k_cache[blocks].transpose(1, 2).reshape(nb * block_size, *k_cache.shape[1:2], k_cache.shape[3])
    v = v_cache[blocks].permute(0, 3, 1, 2).reshape(nb * block_size, *v_cache.shape[1:2], v_cache.shape[2])
    return k[:seq_len], v[:seq_len]


def paged_attention_decode(
    q: torch.Tensor,             # [B, Hq, D]
    k_cache: torch.Tensor,       # [num_blocks, Hk, bs, D]
    v_cache: torch.Tensor,
    block_tables: torch.Tensor,  # [B, max_blocks] int
    seq_lens: torch.Tensor,      # [B] int  (context INCLUDING the current token)
    scale: float,
    sliding_window: int = -1,
    softcap: float = 0.0,
    sinks: Optional[torch.Tensor] = None,  # [Hq] attention-sink logits
) -> torch.Tensor:
    B, Hq, D = q.shape
    Hk = k_cache.shape[1]
    group = Hq // Hk
    out = torch.empty_like(q, dtype=q.dtype)
    for i in range(B):
        L = int(seq_lens[i])
        k, v = _gather_kv(k_cache, v_cache, block_tables[i], L)  # [L, Hk, D]
        qi = q[i].float()                                        # [Hq, D]
        kf = k.float().transpose(0, 1)                           # [Hk, L, D]
        vf = v.float().transpose(0, 1)
        kf = kf.repeat_interleave(group, dim=0)                  # [Hq, L, D]
        vf = vf.repeat_interleave(group, dim=0)
        logits = torch.einsum("hd,hld->hl", qi, kf) * scale      # [Hq, L]
        if softcap > 0:
            logits = softcap * torch.tanh(logits / softcap)
        if sliding_window > 0:
            first_valid = max(0, L - sliding_window)
            logits[:, :first_valid] = float("-inf")
        if sinks is not None:
            logits = torch.cat([sinks.float().unsqueeze(-1), logits], dim=-1)
        p = torch.softmax(logits, dim=-1)
        if sinks is not None:
            p = p[:, 1:]
        out[i] = torch.einsum("hl,hld->hd", p, vf).to(q.dtype)
    return out


def prefill_attention(
    q: torch.Tensor,             # [T, Hq, D] packed varlen new tokens
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    block_tables: torch.Tensor,  # [B, max_blocks]
    seq_lens: torch.Tensor,      # [B] total context length (prefix + new)
    query_lens: torch.Tensor,    # [B] new-token count per request
    scale: float,
    sliding_window: int = -1,
    softcap: float = 0.0,
    sinks: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """Causal varlen prefill over paged KV (new tokens attend to full prefix +
    causally to each other). KV for the new tokens must already be scattered
    into the cache (reshape_and_cache runs first)."""
    T, Hq, D = q.shape
    Hk = k_cache.shape[1]
    group = Hq // Hk
    out = torch.empty_like(q)
    t0 = 0
    for i in range(len(query_lens)):
        QL = int(query_lens[i])
        L = int(seq_lens[i])
        prefix = L - QL
        k, v = _gather_kv(k_cache, v_cache, block_tables[i], L)
        qi = q[t0 : t0 + QL].float().transpose(0, 1)       # [Hq, QL, D]
        kf = k.float().transpose(0, 1).repeat_interleave(group, dim=0)  # [Hq, L, D]
        vf = v.float().transpose(0, 1).repeat_interleave(group, dim=0)
        logits = torch.einsum("hqd,hld->hql", qi, kf) * scale
        if softcap > 0:
            logits = softcap * torch.tanh(logits / softcap)
        # causal mask: query t0+j (absolute pos prefix+j) sees keys <= prefix+j
        qpos = torch.arange(prefix, L, device=q.device).unsqueeze(-1)   # [QL,1]
        kpos = torch.arange(0, L, device=q.device).unsqueeze(0)          # [1,L]
        mask = kpos > qpos
        if sliding_window > 0:
            mask |= kpos <= (qpos - sliding_window)
        logits.masked_fill_(mask.unsqueeze(0), float("-inf"))
        if sinks is not None:
            logits = torch.cat(
                [sinks.float().view(Hq, 1, 1).expand(Hq, QL, 1), logits], dim=-1
            )
        p = torch.softmax(logits, dim=-1)
        if sinks is not None:
            p = p[..., 1:]
        out[t0 : t0 + QL] = torch.einsum("hql,hld->hqd", p, vf).transpose(0, 1).to(q.dtype)
        t0 += QL
    return out


def mla_paged_attention_decode(
    q_latent: torch.Tensor,      # [B, Hq, lora_rank]  (q absorbed into latent space)
    q_rope: torch.Tensor,        # [B, Hq, rope_dim]
    cache: torch.Tensor,         # [num_blocks, bs, lora_rank + rope_dim]
    block_tables: torch.Tensor,
    seq_lens: torch.Tensor,
    scale: float,
) -> torch.Tensor:
    """DeepSeek MLA decode over the compressed cache:
    softmax(scale * (q_latent . latent^T + q_rope . rope^T)) . latent
    (reference ops.py:73-121). Output is [B, Hq, lora_rank] — the caller applies
    the out-projection from latent space."""
    B, Hq, R = q_latent.shape
    bs = cache.shape[1]
    out = torch.empty_like(q_latent)
    for i in range(B):
        L = int(seq_lens[i])
        nb = (L + bs - 1) // bs
        entries = cache[block_tables[i, :nb].long()].reshape(nb * bs, -1)[:L].float()
        latent, rope = entries[:, :R], entries[:, R:]
        logits = (
            q_latent[i].float() @ latent.T + q_rope[i].float() @ rope.T
        ) * scale                                            # [Hq, L]
        p = torch.softmax(logits, dim=-1)
        out[i] = (p @ latent).to(q_latent.dtype)
    return out


# -- activations ------------------------------------------------------------------------


def silu_and_mul(x: torch.Tensor) -> torch.Tensor:
    """x = [gate | up] on the last dim; returns silu(gate) * up."""
    half = x.shape[-1] // 2
    gate, up = x[..., :half].float(), x[..., half:].float()
    return (torch.nn.functional.silu(gate) * up).to(x.dtype)


def gelu_and_mul(x: torch.Tensor) -> torch.Tensor:
    half = x.shape[-1] // 2
    gate, up = x[..., :half].float(), x[..., half:].float()
    return (torch.nn.functional.gelu(gate, approximate="tanh") * up).to(x.dtype)


# -- sampling -----------------------------------------------------------------------------


def sample_tokens(
    logits: torch.Tensor,        # [B, vocab] (any device)
    temperatures,                # [B] floats (list or CPU tensor)
    top_ps,
    top_ks,                      # ints, -1 = off
    min_ps,
    generator: Optional[torch.Generator] = None,
) -> torch.Tensor:
    """Batched temperature / top-k / top-p / min-p filtering + sampling.

    Fully vectorized — sampling params are HOST values (never .item()'d off the
    device), so the hot path issues no device syncs. Greedy rows
    (temperature == 0) take argmax."""
    B, V = logits.shape
    temps = [float(t) for t in temperatures]
    tps = [float(p) for p in top_ps]
    tks = [int(k) for k in top_ks]
    mps = [float(m) for m in min_ps]
    dev = logits.device
    logits = logits.float()

    greedy = [t <= 0.0 for t in temps]
    need_filter = any(
        (not g) and (0 < k < V or p < 1.0 or m > 0.0)
        for g, k, p, m in zip(greedy, tks, tps, mps)
    )
    if all(greedy):
        return logits.argmax(dim=-1)

    t_gpu = torch.tensor(
        [max(t, 1e-6) for t in temps], dtype=torch.float32, device=dev
    ).unsqueeze(-1)
    if not need_filter:
        # gumbel-max: argmax(logits/T + G), G ~ Gumbel(0,1). Identical
        # distribution to softmax+multinomial but pure elementwise+argmax —
        # torch.multinomial over a [B, 128k] prob matrix is the single most
        # expensive sampler kernel on ROCm
        u = torch.rand(B, V, device=dev, generator=generator)
        gumbel = -torch.log(
            (-torch.log(u.clamp_min(1e-20))).clamp_min(1e-20)
        )
        sampled = (logits / t_gpu + gumbel).argmax(dim=-1)
        if not any(greedy):
            return sampled
        greedy_mask = torch.tensor(greedy, dtype=torch.bool, device=dev)
        return torch.where(greedy_mask, logits.argmax(dim=-1), sampled)

    out = logits.argmax(dim=-1)  # greedy default for every row
    probs = torch.softmax(logits / t_gpu, dim=-1)
    if need_filter:
        sorted_p, idx = torch.sort(probs, dim=-1, descending=True)
        cum = torch.cumsum(sorted_p, dim=-1)
        tp_g = torch.tensor(tps, dtype=torch.float32, device=dev).unsqueeze(-1)
        keep = (cum - sorted_p) < tp_g                       # top-p (first always kept)
        tk = torch.tensor(
            [k if 0 < k < V else V for k in tks], dtype=torch.long, device=dev
        ).unsqueeze(-1)
        keep &= torch.arange(V, device=dev).unsqueeze(0) < tk  # top-k
        mp_g = torch.tensor(mps, dtype=torch.float32, device=dev).unsqueeze(-1)
        keep &= sorted_p >= mp_g * sorted_p[:, :1]             # min-p
        keep[:, 0] = True
        sorted_p = torch.where(keep, sorted_p, torch.zeros_like(sorted_p))
        sorted_p = sorted_p / sorted_p.sum(dim=-1, keepdim=True)
        picked = torch.multinomial(sorted_p, 1, generator=generator)
        sampled = idx.gather(-1, picked).squeeze(-1)
    else:
        sampled = torch.multinomial(probs, 1, generator=generator).squeeze(-1)

    greedy_mask = torch.tensor(greedy, dtype=torch.bool, device=dev)
    return torch.where(greedy_mask, out, sampled)


def apply_penalties(
    logits: torch.Tensor,            # [B, vocab]
    output_token_ids: List[List[int]],
    prompt_token_ids: List[List[int]],
    repetition_penalties: torch.Tensor,
    presence_penalties: torch.Tensor,
    frequency_penalties: torch.Tensor,
) -> torch.Tensor:
    logits = logits.clone()
    for i in range(logits.shape[0]):
        rp = float(repetition_penalties[i])
        if rp != 1.0:
            seen = torch.tensor(
                sorted(set(prompt_token_ids[i]) | set(output_token_ids[i])),
                dtype=torch.long, device=logits.device,
            )
            if seen.numel():
                vals = logits[i, seen]
                logits[i, seen] = torch.where(vals > 0, vals / rp, vals * rp)
        pp, fp = float(presence_penalties[i]), float(frequency_penalties[i])
        if (pp != 0.0 or fp != 0.0) and output_token_ids[i]:
            ids = torch.tensor(output_token_ids[i], dtype=torch.long, device=logits.device)
            counts = torch.bincount(ids, minlength=logits.shape[1]).to(logits.dtype)
            logits[i] -= pp * (counts > 0).to(logits.dtype) + fp * counts
    return logits


# -- sparse attention (DSA: DeepSeek V3.2 top-k tokens; MSA: MiniMax block top-k) --


def dsa_paged_attention_decode(
    q_latent: torch.Tensor,      # [B, Hq, lora_rank]
    q_rope: torch.Tensor,        # [B, Hq, rope_dim]
    cache: torch.Tensor,         # [num_blocks, bs, lora_rank + rope_dim]
    block_tables: torch.Tensor,
    seq_lens: torch.Tensor,
    topk_indices: torch.Tensor,  # [B, index_topk] int; -1 padded; row starting
                                 # with -1 => dense fallback (reference ops.py:182)
    scale: float,
) -> torch.Tensor:
    B, Hq, R = q_latent.shape
    bs = cache.shape[1]
    out = torch.empty_like(q_latent)
    for i in range(B):
        L = int(seq_lens[i])
        nb = (L + bs - 1) // bs
        entries = cache[block_tables[i, :nb].long()].reshape(nb * bs, -1)[:L].float()
        idx = topk_indices[i]
        if int(idx[0]) >= 0:
            keep = idx[(idx >= 0) & (idx < L)].long()
            entries = entries[keep]
        latent, rope = entries[:, :R], entries[:, R:]
        logits = (
            q_latent[i].float() @ latent.T + q_rope[i].float() @ rope.T
        ) * scale
        p = torch.softmax(logits, dim=-1)
        out[i] = (p @ latent).to(q_latent.dtype)
    return out


def dsa_indexer_scores(
    q_index: torch.Tensor,       # [B, index_heads, index_dim]
    index_cache: torch.Tensor,   # [nb, bs, index_heads, index_dim] or
                                 # [nb, bs, index_dim] (keys shared across
                                 # heads, as in DeepSeek-V3.2 where only the
                                 # indexer query is multi-headed)
    head_weights: torch.Tensor,  # [B, index_heads] per-head score weights
    block_tables: torch.Tensor,
    seq_lens: torch.Tensor,
) -> torch.Tensor:
    """Weighted q.k scores over the full context for top-k selection
    (reference dsa_indexer, ops.py:325-367). Returns [B, max_ctx] with -inf
    past each row's length; top-k itself is torch.topk on the result."""
    B, Hi, Di = q_index.shape
    bs = index_cache.shape[1]
    shared_k = index_cache.dim() == 3
    max_ctx = int(seq_lens.max())
    scores = torch.full((B, max_ctx), float("-inf"), dtype=torch.float32,
                        device=q_index.device)
    for i in range(B):
        L = int(seq_lens[i])
        nb = (L + bs - 1) // bs
        keys = index_cache[block_tables[i, :nb].long()].reshape(nb * bs, -1, Di)[:L]
        if shared_k:
            s = torch.einsum("hd,ld->hl", q_index[i].float(),
                             keys.squeeze(1).float())
        else:
            s = torch.einsum("hd,lhd->hl", q_index[i].float(), keys.float())
        s = torch.relu(s)  # per DeepSeek-V3.2 indexer: ReLU before head-weighting
        scores[i, :L] = torch.einsum("h,hl->l", head_weights[i].float(), s)
    return scores


def store_indexer_cache(
    index_keys: torch.Tensor,    # [T, index_heads, index_dim] or [T, index_dim]
    index_cache: torch.Tensor,   # [num_blocks(+1 trash), bs, ...]
    slot_mapping: torch.Tensor,
) -> None:
    """Scatter indexer keys by slot. hipGraph-capture safe: instead of
    boolean compaction (data-dependent shapes) pad tokens (slot -1) are
    redirected into the cache's LAST block, which the engine over-allocates
    as a trash row (MLAKVCache/PagedKVCache index_caches)."""
    bs = index_cache.shape[1]
    slots = slot_mapping.long()
    trash = (index_cache.shape[0] - 1) * bs
    slots = torch.where(slots >= 0, slots, torch.full_like(slots, trash))
    index_cache[slots // bs, slots % bs] = index_keys.to(index_cache.dtype)


def msa_block_scores(
    q: torch.Tensor,             # [B, Hq, D]
    k_cache: torch.Tensor,       # [num_blocks, Hk, bs, D]
    block_tables: torch.Tensor,
    seq_lens: torch.Tensor,
    sparse_block: int,
) -> torch.Tensor:
    """Mean-pooled K per sparse block scored against the mean query
    (reference msa_indexer phase 1). Returns [B, max_sparse_blocks] (-inf pad)."""
    B, Hq, D = q.shape
    Hk = k_cache.shape[1]
    bs = k_cache.shape[2]
    max_blocks = (int(seq_lens.max()) + sparse_block - 1) // sparse_block
    out = torch.full((B, max_blocks), float("-inf"), dtype=torch.float32)
    qm = q.float().mean(dim=1)  # [B, D]
    for i in range(B):
        L = int(seq_lens[i])
        nb = (L + bs - 1) // bs
        k = (
            k_cache[block_tables[i, :nb].long()]
            .transpose(1, 2).reshape(nb * bs, Hk, D)[:L]
            .float().mean(dim=1)
        )  # [L, D]
        nsb = (L + sparse_block - 1) // sparse_block
        for sb in range(nsb):
            seg = k[sb * sparse_block : min((sb + 1) * sparse_block, L)]
            out[i, sb] = seg.mean(dim=0) @ qm[i]
    return out


def msa_topk_tokens(
    block_scores: torch.Tensor,  # [B, max_sparse_blocks]
    seq_lens: torch.Tensor,
    sparse_block: int,
    topk_blocks: int,
    init_blocks: int = 1,
    local_blocks: int = 2,
) -> torch.Tensor:
    """Top-k sparse blocks per sequence expanded to token positions, always
    keeping the first `init_blocks` and last `local_blocks` (reference
    msa_block_topk_tokens). Returns [B, max_positions] int64, -1 padded."""
    B = block_scores.shape[0]
    rows = []
    for i in range(B):
        L = int(seq_lens[i])
        nsb = (L + sparse_block - 1) // sparse_block
        keep = set(range(min(init_blocks, nsb)))
        keep |= set(range(max(0, nsb - local_blocks), nsb))
        remaining = [b for b in range(nsb) if b not in keep]
        if remaining and topk_blocks > 0:
            sc = block_scores[i, remaining]
            take = min(topk_blocks, len(remaining))
            top = torch.topk(sc, take).indices.tolist()
            keep |= {remaining[t] for t in top}
        pos = []
        for b in sorted(keep):
            pos.extend(range(b * sparse_block, min((b + 1) * sparse_block, L)))
        rows.append(torch.tensor(sorted(pos), dtype=torch.int64))
    max_p = max(r.numel() for r in rows)
    out = torch.full((B, max_p), -1, dtype=torch.int64)
    for i, r in enumerate(rows):
        out[i, : r.numel()] = r
    return out


def msa_paged_attention_decode(
    q: torch.Tensor,             # [B, Hq, D]
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    block_tables: torch.Tensor,
    seq_lens: torch.Tensor,
    token_positions: torch.Tensor,  # [B, max_positions] int, -1 padded; or
                                    # [B, Hk, max_positions] for one selection
                                    # per kv head (minimax-m3)
    scale: float,
) -> torch.Tensor:
    """Exact attention over explicit token positions mapped through block
    tables (reference msa_paged_attention, ops.py:594-662)."""
    B, Hq, D = q.shape
    Hk = k_cache.shape[1]
    group = Hq // Hk
    per_head = token_positions.dim() == 3
    out = torch.empty_like(q)
    for i in range(B):
        L = int(seq_lens[i])
        k, v = _gather_kv(k_cache, v_cache, block_tables[i], L)
        for h in range(Hk):
            pos = token_positions[i, h] if per_head else token_positions[i]
            keep = pos[(pos >= 0) & (pos < L)].long()
            kf = k.float()[keep, h]                      # [P, D]
            vf = v.float()[keep, h]
            qh = q[i, h * group:(h + 1) * group].float() # [G, D]
            logits = (qh @ kf.T) * scale
            p = torch.softmax(logits, dim=-1)
            out[i, h * group:(h + 1) * group] = (p @ vf).to(q.dtype)
    return out


# -- sequence mixers: fp32-residual layer norm, latent window attention, GLA ----
# Eager torch versions of the _mix extension's kernels (CPU engine, oracles of
# the kernel tests). Same signatures as the wrappers in ops/mix.py.


def add_layernorm(resid, y, scale, mult, weight, bias, eps, out_dtype):
    """resid [T, W] fp32 += mult * scale * y (in place; skipped when y is
    None); returns layer_norm(resid) * weight + bias in out_dtype (None when
    weight is None)."""
    if y is not None:
        resid.add_(mult * (scale.float() * y.float()))
    if weight is None:
        return None
    mean = resid.mean(-1, keepdim=True)
    var = ((resid - mean) ** 2).mean(-1, keepdim=True)
    out = (resid - mean) / torch.sqrt(var + eps) * weight.float() + bias.float()
    return out.to(out_dtype)


def _rotate_rows(x, positions, freq, mult, rot_dims, interleaved=False,
                 sign=1.0):
    """x [T, ..., >=rot_dims] fp32; pair (i, i + rot_dims/2), or (2i, 2i+1)
    when interleaved; sign -1 turns the other way."""
    half = rot_dims // 2
    ang = positions.float().unsqueeze(-1) * freq.float()          # [T, half]
    shape = [x.shape[0]] + [1] * (x.dim() - 2) + [half]
    c = (torch.cos(ang) * mult).view(shape)
    s = (torch.sin(ang) * (mult * sign)).view(shape)
    out = x.clone()
    if interleaved:
        u, v = x[..., 0:rot_dims:2], x[..., 1:rot_dims:2]
        out[..., 0:rot_dims:2] = u * c - v * s
        out[..., 1:rot_dims:2] = v * c + u * s
    else:
        u, v = x[..., :half], x[..., half:rot_dims]
        out[..., :half] = u * c - v * s
        out[..., half:rot_dims] = v * c + u * s
    return out


def latent_kv_store(dkv, norm_w, eps, freq, mult, rot_dims, positions,
                    slot_mapping, cache, rank):
    x = dkv.float()
    lat = x[:, :rank]
    lat = lat / torch.sqrt((lat * lat).mean(-1, keepdim=True) + eps) * norm_w.float()
    kr = x[:, rank:]
    if rot_dims > 0:
        kr = _rotate_rows(kr, positions, freq, mult, rot_dims)
    entry = torch.cat([lat, kr], dim=-1).to(cache.dtype)
    keep = slot_mapping >= 0
    flat = cache.view(-1, cache.shape[-1])
    flat[slot_mapping[keep]] = entry[keep]


def rope_rows(q, col0, rot_w, freq, mult, rot_dims, positions):
    return _rotate_rows(q[..., col0 : col0 + rot_w].float(), positions, freq,
                        mult, rot_dims).contiguous()


def latent_window_attention(q_lat, q_rot, cache, block_tables, token_seq,
                            positions, window, scale):
    T, H, rank = q_lat.shape
    bs = cache.shape[1]
    out = torch.empty_like(q_lat)
    pos = positions.tolist()
    seq = token_seq.tolist() if token_seq is not None else list(range(T))
    for t in range(T):
        p = pos[t]
        lo = max(0, p - window + 1)
        j = torch.arange(lo, p + 1)
        bt = block_tables[seq[t]].long()
        rows = cache[bt[j // bs], j % bs].float()                  # [n, E]
        s = (q_lat[t] @ rows[:, :rank].T + q_rot[t] @ rows[:, rank:].T) * scale
        out[t] = torch.softmax(s, dim=-1) @ rows[:, :rank]
    return out


def gla_recurrence(q, k, v, z, z_bias, state, slots, cu, positions, inv_tau,
                   q_scale):
    T = q.shape[0]
    _, H, dk, dv = state.shape
    qf = q.float().view(T, H, dk) * q_scale
    kf = k.float().view(T, H, dk)
    vf = v.float().view(T, H, dv)
    zf = z.float().view(T, H, dk) + z_bias.float().view(H, dk)
    alpha = torch.exp(torch.nn.functional.logsigmoid(zf) * inv_tau)
    o = torch.empty(T, H, dv, dtype=torch.float32)
    bounds = cu.tolist() if cu is not None else list(range(T + 1))
    pos = positions.tolist()
    for b, slot in enumerate(slots.tolist()):
        t0, t1 = bounds[b], bounds[b + 1]
        if t0 >= t1:
            continue
        S = torch.zeros(H, dk, dv) if pos[t0] == 0 else state[slot].clone()
        for t in range(t0, t1):
            S = alpha[t].unsqueeze(-1) * S + kf[t].unsqueeze(-1) * vf[t].unsqueeze(-2)
            o[t] = torch.einsum("hkv,hk->hv", S, qf[t])
        state[slot] = S
    return o


def gated_rmsnorm(o, gate, weight, eps, out_dtype):
    T, H, dv = o.shape
    x = o / torch.sqrt((o * o).mean(-1, keepdim=True) + eps) * weight.float()
    g = gate.float().view(T, H, dv)
    return (x * torch.nn.functional.silu(g)).view(T, H * dv).to(out_dtype)


# -- row-cache attention mixers: sandwich RMS norm with depth averaging,
# differential / pooled-window softmax attention over [keys | values] rows,
# xIELU ---------------------------------------------------------------------


def sandwich_rmsnorm(x, y, w_branch, hist, n_hist, dwa, w_next, eps, offset,
                     out_dtype, add_table=None, add_index=None):
    """One residual step of a stack that norms a branch before AND after it.
    x [T, W] fp32, in place:
      x += add_table[add_index]                       (when add_table is given)
      x += y / rms(y) * (offset + w_branch)           (when y is given)
      hist[n_hist - 1] = x                            (when hist is given)
      x = sum_j dwa[j] * hist[j], j < n_hist          (when dwa is given)
    and returns x / rms(x) * (offset + w_next) in out_dtype (None when w_next
    is None). rms(v) = sqrt(mean(v^2) + eps); everything in fp32."""
    if add_table is not None:
        x.add_(add_table[add_index.long()].float())
    if y is not None:
        yf = y.float()
        r = yf / torch.sqrt((yf * yf).mean(-1, keepdim=True) + eps)
        x.add_(r * (offset + w_branch.float()))
    if hist is not None:
        hist[n_hist - 1].copy_(x)
    if dwa is not None:
        acc = torch.zeros_like(x)
        for j in range(n_hist):
            acc = acc + dwa[j].float() * hist[j]
        x.copy_(acc)
    if w_next is None:
        return None
    out = x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) \
        * (offset + w_next.float())
    return out.to(out_dtype)


def _segment_rms(x, seg, eps):
    T = x.shape[0]
    v = x.view(T, -1, seg)
    return (v / torch.sqrt((v * v).mean(-1, keepdim=True) + eps)).reshape(T, -1)


def _segment_rotate(x, seg, positions, freq, mult, rot_dims, interleaved=False):
    T = x.shape[0]
    return _rotate_rows(x.view(T, -1, seg), positions, freq, mult,
                        rot_dims, interleaved).reshape(T, -1)


def qkv_store(q, k, v, positions, slot_mapping, cache, seg_dim, norm_eps,
              temp_coef, temp_every, q_weight=None, k_weight=None,
              rot_freq=None, rot_mult=1.0, rot_dims=0, norm_whole=False,
              rot_interleaved=False, v_seg=0, v_rot_freq=None, v_cs_out=None):
    """Queries to fp32 (each seg_dim-wide segment divided by its RMS when
    norm_eps is given, times q_weight [seg_dim] when given; with norm_whole
    the RMS runs over the token's WHOLE query row and q_weight has the row's
    width; then each segment's first rot_dims dimensions rotated by position,
    dimension i paired with i + rot_dims / 2 (or 2i with 2i + 1 when
    rot_interleaved) at angle pos * rot_freq[i], cos and sin times rot_mult,
    when rot_freq is given; multiplied by 1 + temp_coef * ln(floor((pos + 1)
    / temp_every) + 1) when temp_every > 0), keys (normed, weighted by
    k_weight and rotated alike) and values into one cache row [keys | values]
    per token. v_rot_freq [v_seg / 2] given: every v_seg-wide segment of the
    values is rotated by position over its whole width (same pairing, angles
    pos * v_rot_freq[m]) before it is stored; v_cs_out [T, v_seg] fp32 then
    receives every token's (cos, sin) pairs of that rotation. v None: the values are the keys
    as they came in, before the norm. k None: nothing is stored (the layer
    reads another layer's rows). Slot -1 skips the token."""

    def prepare(x, weight):
        if norm_eps is not None:
            x = _segment_rms(x, x.shape[1] if norm_whole else seg_dim, norm_eps)
        if weight is not None:
            if norm_whole:
                x = x * weight.float()
            else:
                x = (x.view(x.shape[0], -1, seg_dim) * weight.float()).reshape(x.shape)
        if rot_freq is not None:
            x = _segment_rotate(x, seg_dim, positions, rot_freq, rot_mult,
                                rot_dims, rot_interleaved)
        return x

    qf = prepare(q.float(), q_weight)
    if v_rot_freq is not None and v_cs_out is not None:
        ang = positions.float().unsqueeze(-1) * v_rot_freq.float()
        v_cs_out.copy_(torch.stack([torch.cos(ang), torch.sin(ang)], -1)
                       .reshape(v_cs_out.shape))
    if temp_every > 0:
        p = positions.float()
        temp = 1.0 + temp_coef * torch.log(torch.floor((p + 1.0) / temp_every) + 1.0)
        qf = qf * temp.unsqueeze(-1)
    if k is not None:
        kf = k.float()
        vals = kf if v is None else v.float()
        kf = prepare(kf, k_weight)
        if v_rot_freq is not None:
            vals = _segment_rotate(vals, v_seg, positions, v_rot_freq, 1.0,
                                   v_seg, rot_interleaved)
        entry = torch.cat([kf, vals], dim=-1).to(cache.dtype)
        keep = slot_mapping >= 0
        flat = cache.view(-1, cache.shape[-1])
        flat[slot_mapping[keep]] = entry[keep]
    return qf.contiguous()


def rotate_heads(x, positions, freq, interleaved, sign, out_dtype):
    """x [T, H, D] fp32: every head turned by its token's position over the
    whole width D (pair m: dimensions m and m + D/2, or 2m and 2m + 1 when
    interleaved) by sign * pos * freq[m]. Returns [T, H * D] of out_dtype."""
    T, H, D = x.shape
    return _rotate_rows(x.float(), positions, freq, 1.0, D, interleaved,
                        sign).reshape(T, H * D).to(out_dtype)


def pool_cache_update(cache, pool, block_tables, token_seq, positions,
                      slot_mapping, pool_tokens):
    """For every token of the step that completes a block of `pool_tokens`
    positions: the fp32 mean of the block's cache rows (as the cache holds
    them) into the pooled rows of its sequence."""
    T = positions.shape[0]
    bs, per_page = cache.shape[1], pool.shape[1]
    pos = positions.tolist()
    seq = token_seq.tolist() if token_seq is not None else list(range(T))
    slots = slot_mapping.tolist()
    P = pool_tokens
    for t in range(T):
        p = pos[t]
        if slots[t] < 0 or (p + 1) % P != 0:
            continue
        bt = block_tables[seq[t]].long()
        j = torch.arange(p + 1 - P, p + 1)
        rows = cache[bt[j // bs], j % bs].float()
        acc = torch.zeros_like(rows[0])
        for r in rows:          # in position order, as the kernel adds them
            acc = acc + r
        b = p // P
        pool[bt[b // per_page], b % per_page] = acc / P


def row_attention(q, cache, pool, block_tables, token_seq, positions, heads,
                  kv_heads, maps, dim, vdim, window, pool_tokens, scale,
                  softcap, lam, norm_eps, out_mult, out_dtype, head_bias=None,
                  gate=None, shared_kv=False, out_rot_cs=None,
                  out_rot_interleaved=False, value_col=0):
    """Attention over cache rows [keys (kv_heads x maps x dim) |
    values (kv_heads x vdim)]; shared_kv: a row holds the keys only (one kv
    head, one map) and the values are its columns value_col .. value_col +
    vdim (vdim == dim: the values ARE the keys). q [T, heads * maps * dim] fp32. window 0: every
    key up to the token's position; window > 0: keys j with 0 <= pos - j <
    window plus, when pool_tokens > 0, the pooled row of every block of
    pool_tokens positions that ends at or before pos - window, in the same
    softmax. softcap > 0: s <- softcap * tanh(s / softcap). maps == 2: the
    two maps' results (same values) combine as a1 - lam * a2. norm_eps given:
    the head's result is divided by its RMS and multiplied by out_mult.
    head_bias [heads] given: no softmax; a visible key weighs sigmoid(s +
    head_bias[h]) and the weights are not normalised over the keys. gate
    [T, heads] given: head h's result is multiplied by sigmoid(gate[t, h]).
    out_rot_cs [T, vdim / 2, 2] (cos, sin per token and pair) given: every
    head's result is turned BACK by its token's angles over the whole value
    width (pair m = dimensions m, m + vdim / 2, or 2m, 2m + 1 when
    out_rot_interleaved): (u, w) -> (u cos + w sin, w cos - u sin).
    Returns [T, heads * vdim] in out_dtype."""
    T = q.shape[0]
    bs = cache.shape[1]
    H, G, M = heads, kv_heads, maps
    wk = G * M * dim
    rep = H // G
    pos = positions.tolist()
    seq = token_seq.tolist() if token_seq is not None else list(range(T))
    out = torch.empty(T, H, vdim, dtype=torch.float32)
    qv = q.view(T, G, rep, M, dim)
    for t in range(T):
        p = pos[t]
        bt = block_tables[seq[t]].long()
        lo = max(0, p - window + 1) if window > 0 else 0
        j = torch.arange(lo, p + 1)
        rows = cache[bt[j // bs], j % bs].float()
        if window > 0 and pool_tokens > 0 and p - window + 1 >= pool_tokens:
            nb = (p - window + 1) // pool_tokens
            b = torch.arange(nb)
            per_page = pool.shape[1]
            rows = torch.cat([pool[bt[b // per_page], b % per_page], rows], 0)
        k = rows[:, :wk].view(-1, G, M, dim)
        v = (rows[:, value_col:value_col + vdim] if shared_kv
             else rows[:, wk:]).reshape(-1, G, vdim)
        s = torch.einsum("grmd,ngmd->grmn", qv[t], k) * scale
        if softcap > 0:
            s = softcap * torch.tanh(s / softcap)
        if head_bias is not None:
            wts = torch.sigmoid(s + head_bias.float().view(G, rep, 1, 1))
        else:
            wts = torch.softmax(s, dim=-1)
        a = torch.einsum("grmn,ngv->grmv", wts, v)
        o = a[:, :, 0] - lam * a[:, :, 1] if M == 2 else a[:, :, 0]
        if norm_eps is not None:
            o = o / torch.sqrt((o * o).mean(-1, keepdim=True) + norm_eps) * out_mult
        if gate is not None:
            o = o * torch.sigmoid(gate[t].float()).view(G, rep, 1)
        out[t] = o.reshape(H, vdim)
    if out_rot_cs is not None:
        cs = out_rot_cs.view(T, 1, vdim // 2, 2).float()
        c, sn = cs[..., 0], cs[..., 1]
        if out_rot_interleaved:
            u, w = out[..., 0::2].clone(), out[..., 1::2].clone()
            out[..., 0::2] = u * c + w * sn
            out[..., 1::2] = w * c - u * sn
        else:
            hv = vdim // 2
            u, w = out[..., :hv].clone(), out[..., hv:].clone()
            out[..., :hv] = u * c + w * sn
            out[..., hv:] = w * c - u * sn
    return out.view(T, H * vdim).to(out_dtype)


def xielu(x, a_pos, a_neg):
    """z > 0: a_pos z^2 + z / 2; z <= 0: (1/2 + a_neg)(exp(z) - 1 - z) + z / 2."""
    z = x.float()
    neg = torch.clamp(z, max=0.0)
    out = torch.where(z > 0, a_pos * z * z + 0.5 * z,
                      (0.5 + a_neg) * (torch.expm1(neg) - neg) + 0.5 * z)
    return out.to(x.dtype)


# -- post-norm residual stream, minGRU, clamped gated linear unit ----------------


def branch_rmsnorm_add(x, y1, y2, a, b, weight, eps, out_dtype, keep_stream=True):
    """One step of a residual stream that norms a sublayer's OUTPUT:
      y = a * y1 (+ b * y2),  n = y / sqrt(mean(y^2) + eps) * weight,
      x <- x + n   (x None: x = n)
    all in fp32; x [T, W] fp32 is updated in place. Returns (x, x in
    out_dtype); keep_stream False: (None, the sum in out_dtype) and x is
    left as it was."""
    y = a * y1.float()
    if y2 is not None:
        y = y + b * y2.float()
    n = y / torch.sqrt((y * y).mean(-1, keepdim=True) + eps) * weight.float()
    if x is not None:
        n = n + x
    if not keep_stream:
        return None, n.to(out_dtype)
    if x is None:
        x = n.contiguous()
    else:
        x.copy_(n)
    return x, x.to(out_dtype)


def mingru_scan(zug, z_bias, u_bias, state, slots, cu, positions, out_dtype):
    """minGRU over packed sequences. zug [T, 3 * width]: pre-activations of
    the update gate z, the candidate u and the output gate g of every token.
      f = sigma(z_pre + z_bias),    p = u_pre + u_bias,
      c = p + 1/2 where p >= 0, sigma(p) below,
      S_t = S_(t-1) + f (c - S_(t-1))   per channel,
    fp32 throughout; the state [slots, width] fp32 is read (or started from
    zero when the portion begins at position 0) and written back. cu [B+1]
    int32 token bounds (None: one token each). Returns S_t * silu(g_pre) as
    [T, width] of out_dtype."""
    T = zug.shape[0]
    width = state.shape[1]
    f = zug.float()
    z = torch.sigmoid(f[:, :width] + z_bias.float())
    u = f[:, width : 2 * width] + u_bias.float()
    cand = torch.where(u >= 0, u + 0.5, torch.sigmoid(u))
    g = f[:, 2 * width :]
    g = g * torch.sigmoid(g)
    out = torch.empty(T, width, dtype=torch.float32)
    bounds = cu.tolist() if cu is not None else list(range(T + 1))
    pos = positions.tolist()
    for b, slot in enumerate(slots.tolist()):
        t0, t1 = bounds[b], bounds[b + 1]
        if t0 >= t1:
            continue
        S = torch.zeros(width) if pos[t0] == 0 else state[slot].clone()
        for t in range(t0, t1):
            S = (1.0 - z[t]) * S + z[t] * cand[t]
            out[t] = S * g[t]
        state[slot] = S
    return out.to(out_dtype)


def clamped_glu(gate_up, limit, alpha=1.702):
    """gate_up [T, 2 I] = [gate | up] -> [T, I]: a sigma(alpha a) (1 + b) with
    a = gate cut off above at `limit`, b = up cut off at -limit and +limit
    (fp32 inside)."""
    I = gate_up.shape[-1] // 2
    f = gate_up.float()
    g = f[..., :I].clamp(max=limit)
    u = f[..., I:].clamp(min=-limit, max=limit)
    return (g * torch.sigmoid(alpha * g) * (u + 1.0)).to(gate_up.dtype)


# -- grouped RMS norm over a parallel residual, hashed pair embedding, relu^2 ----


def group_rmsnorm_add(x, y1, y2, weight, groups, eps, out_dtype):
    """One step of a residual stream whose sublayers all read ONE norm:
      x <- x + (y1 + y2)     (fp32, in place; y1 None: no update; y2 None: y1 only)
      h = x split into `groups` equal consecutive parts, each divided by its
          own sqrt(mean(part^2) + eps), the whole times weight
    Returns h in out_dtype (None when weight is None)."""
    if y1 is not None:
        y = y1.float()
        if y2 is not None:
            y = y + y2.float()
        x.add_(y)
    if weight is None:
        return None
    T, W = x.shape
    v = x.view(T, groups, W // groups)
    h = (v / torch.sqrt((v * v).mean(-1, keepdim=True) + eps)).reshape(T, W)
    return (h * weight.float()).to(out_dtype)


def pair_hash_embedding(ids, prev_ids, table, scale, pair_table, buckets,
                        mul_prev, mul_cur):
    """fp32 [T, W]: table[id] * scale + pair_table[r], r = (prev * mul_prev +
    id * mul_cur) mod buckets, or r = buckets (the table's last row) where a
    token has no predecessor (prev < 0)."""
    ids = ids.long()
    prev = prev_ids.long()
    r = (prev.clamp(min=0) * int(mul_prev) + ids * int(mul_cur)) % int(buckets)
    r = torch.where(prev < 0, torch.full_like(r, int(buckets)), r)
    return table[ids].float() * float(scale) + pair_table[r].float()


def relu_squared(x):
    """max(x, 0)^2 (fp32 inside, result in the input dtype)."""
    z = x.float().clamp(min=0.0)
    return (z * z).to(x.dtype)
