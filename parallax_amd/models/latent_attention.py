"""Attention over a compressed latent cache: with a sliding window and a
rotated key part (LatentWindowAttention), or without positions, over the whole
context, with an output gate per head (GatedLatentAttention).

Per token the cache holds one row [latent c (RMS-normed) | rotated key part]
shared by all heads; a head's key is [W_uk c | rotated part] and its value
W_uv c. Attention runs absorbed, as the DeepSeek MLA path of this package
does: queries are folded through W_uk into the latent space (fp32), scores and
softmax are fp32 over the cache rows, and the weighted latent sum is expanded
through W_uv afterwards. Differences from models/deepseek_v3.MLAAttention,
all parameters: a sliding window (a token sees itself and window - 1 tokens
before it), separate W_uk / W_uv, rotate-half pairing on the first rot_dims
dimensions of the rotated part with a YaRN frequency ramp whose softmax scale
is left untouched, and a layer may read ANOTHER layer's cache rows
(`cache_layer_idx` of the owner) with its own queries and up-projections.
"""

from __future__ import annotations

from typing import Optional

import torch
import torch.nn as nn

from .. import ops
from ..parallel.layers import MergedColumnParallelLinear, RowParallelLinear
from .forward_meta import ForwardMeta
from .rope import yarn_ramp_frequencies


class LatentWindowAttention(nn.Module):
    def __init__(self, hidden_size: int, heads: int, nope_dim: int, rot_width: int,
                 value_dim: int, rank: int, window: int, scale: float,
                 norm_eps: float, cache_layer_idx: int, owns_cache: bool,
                 rot_dims: Optional[int] = None, rot_base: float = 10000.0,
                 rot_scaling: Optional[dict] = None):
        super().__init__()
        self.heads, self.dn, self.dr, self.dv = heads, nope_dim, rot_width, value_dim
        self.rank, self.window, self.scale = rank, int(window), float(scale)
        self.eps = norm_eps
        self.cache_layer_idx = cache_layer_idx
        self.owns_cache = owns_cache
        self.rot_dims = rot_dims if rot_dims is not None else rot_width
        sc = rot_scaling or {}
        self._freq, self._mult = yarn_ramp_frequencies(
            self.rot_dims, rot_base, float(sc.get("factor", 1.0)),
            float(sc.get("original", 0.0)), float(sc.get("fast", 32.0)),
            float(sc.get("slow", 1.0)),
        )
        sizes = [heads * (nope_dim + rot_width)]
        if owns_cache:
            sizes.append(rank + rot_width)
            self.latent_norm = nn.Parameter(torch.empty(rank), requires_grad=False)
        # queries (and, for a layer with a cache of its own, the down
        # projection to latent + rotated key part) in one GEMM
        self.in_proj = MergedColumnParallelLinear(hidden_size, sizes)
        self.w_uk = nn.Parameter(torch.empty(heads, nope_dim, rank), requires_grad=False)
        self.w_uv = nn.Parameter(torch.empty(heads, value_dim, rank), requires_grad=False)
        self.o_proj = RowParallelLinear(heads * value_dim, hidden_size)
        self._f32 = None  # (freq, w_uk fp32, w_uv fp32) on the run device

    def _constants(self, device):
        if self._f32 is None or self._f32[0].device != device:
            self._f32 = (self._freq.to(device), self.w_uk.float().contiguous(),
                         self.w_uv.float().contiguous())
        return self._f32

    def invalidate_constants(self) -> None:
        self._f32 = None

    def forward(self, x: torch.Tensor, meta: ForwardMeta) -> torch.Tensor:
        T, H = x.shape[0], self.heads
        freq, w_uk, w_uv = self._constants(x.device)
        parts = self.in_proj.split_output(self.in_proj(x))
        q = parts[0].view(T, H, self.dn + self.dr)
        cache = meta.mla_cache.layer(self.cache_layer_idx)
        if self.owns_cache:
            ops.latent_kv_store(parts[1], self.latent_norm, self.eps, freq,
                                self._mult, self.rot_dims, meta.positions,
                                meta.slot_mapping, cache, self.rank)
        q_rot = ops.rope_rows(q, self.dn, self.dr, freq, self._mult,
                              self.rot_dims, meta.positions)
        q_lat = torch.einsum("thd,hdr->thr", q[..., : self.dn].float(), w_uk)
        out_lat = ops.latent_window_attention(
            q_lat.contiguous(), q_rot, cache, meta.block_tables,
            meta.token_seq(), meta.positions, self.window, self.scale,
            max_seq_len=meta.max_seq_len,
        )
        attn = torch.einsum("thr,hvr->thv", out_lat, w_uv).to(x.dtype)
        return self.o_proj(attn.reshape(T, H * self.dv))


class GatedLatentAttention(nn.Module):
    """Latent attention without positions. Per token the cache holds the
    RMS-normed latent c = norm(W_dkv x) alone; head h has the key W_uk,h c and
    the value W_uv,h c, the score q_h . k_h * scale, a full causal mask and an
    ordinary softmax; the head's result is multiplied by sigmoid(w_g,h . x),
    a gate that reads the mixer's input. Runs absorbed: the queries are folded
    through W_uk into the latent space (fp32), ops.row_attention treats the
    latent row as the one shared key AND value row of all heads (scores,
    softmax and sums fp32), and the weighted latent sum is expanded through
    W_uv afterwards; the gate, a scalar per head, commutes with that
    expansion and is applied inside the attention kernel. own_proj False: a
    caller merges the input projections (widths `proj_sizes`: queries, latent,
    gate pre-activations) with others of the same input and calls mix()."""

    VALUE_COLS = 256   # value columns a head sums in one attention call

    def __init__(self, hidden_size: int, heads: int, dim: int, value_dim: int,
                 rank: int, scale: float, norm_eps: float, cache_layer_idx: int,
                 own_proj: bool = True):
        super().__init__()
        self.heads, self.dim, self.vdim, self.rank = heads, dim, value_dim, rank
        self.scale, self.eps = float(scale), float(norm_eps)
        self.cache_layer_idx = cache_layer_idx
        self.proj_sizes = [heads * dim, rank, heads]
        self.in_proj = MergedColumnParallelLinear(hidden_size, self.proj_sizes) \
            if own_proj else None
        self.latent_norm = nn.Parameter(torch.empty(rank), requires_grad=False)
        self.w_uk = nn.Parameter(torch.empty(heads, dim, rank), requires_grad=False)
        self.w_uv = nn.Parameter(torch.empty(heads, value_dim, rank), requires_grad=False)
        self.o_proj = RowParallelLinear(heads * value_dim, hidden_size)
        self._f32 = None

    def _constants(self, device):
        if self._f32 is None or self._f32[0].device != device:
            self._f32 = (self.w_uk.float().contiguous(),
                         self.w_uv.float().contiguous(),
                         torch.empty(0, dtype=torch.float32, device=device))
        return self._f32

    def invalidate_constants(self) -> None:
        self._f32 = None

    def mix(self, parts, meta: ForwardMeta, out_dtype) -> torch.Tensor:
        """parts: [q, latent pre-norm, gate pre-activations] of the step's
        tokens (strided views are fine) -> [T, heads * value_dim]."""
        q, dkv, gate = parts
        T, H = q.shape[0], self.heads
        w_uk, w_uv, no_freq = self._constants(q.device)
        cache = meta.mla_cache.layer(self.cache_layer_idx)
        ops.latent_kv_store(dkv, self.latent_norm, self.eps, no_freq, 1.0, 0,
                            meta.positions, meta.slot_mapping, cache, self.rank)
        q_lat = torch.einsum("thd,hdr->thr", q.view(T, H, self.dim).float(), w_uk)
        q_lat = q_lat.reshape(T, H * self.rank)
        # the attention kernels sum at most VALUE_COLS value columns per
        # head: a wider latent is summed in column shares (the scores are
        # worked out again for every share)
        shares = []
        for c0 in range(0, self.rank, self.VALUE_COLS):
            cols = min(self.VALUE_COLS, self.rank - c0)
            shares.append(ops.row_attention(
                q_lat, cache, None, meta.block_tables, meta.token_seq(),
                meta.positions, H, 1, 1, self.rank, cols, 0, 0, self.scale,
                0.0, 0.0, None, 1.0, torch.float32,
                max_seq_len=meta.max_seq_len, query_bounds=meta.query_bounds(),
                gate=gate, shared_kv=True, value_col=c0,
            ).view(T, H, cols))
        o_lat = shares[0] if len(shares) == 1 else torch.cat(shares, dim=-1)
        attn = torch.einsum("thr,hvr->thv", o_lat, w_uv)
        return attn.to(out_dtype).reshape(T, H * self.vdim)

    def forward(self, x: torch.Tensor, meta: ForwardMeta) -> torch.Tensor:
        parts = self.in_proj.split_output(self.in_proj(x))
        return self.o_proj(self.mix(parts, meta, x.dtype))
