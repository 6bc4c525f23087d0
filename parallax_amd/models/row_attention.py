"""Grouped-head softmax attention over a row-per-token cache: every token
owns one paged cache row [keys of all kv heads | values of all kv heads], and
one kernel (ops.row_attention) serves prompt portions and decode rows alike,
reading keys and values from the cache only, so a position's result does not
depend on how its prompt was cut or batched. Queries are prepared in fp32 by
ops.qkv_store, which also scatters the step's keys and values; scores,
softmax and the per-head post-processing are fp32.

Four mixers are built on it:

DifferentialAttention — every head has TWO query/key maps over the same
values. With a1, a2 the two softmax results, o = a1 - lambda * a2, then o is
divided by its RMS over the value width and multiplied by (1 - diff);
lambda = exp(lq1 . lk1) - exp(lq2 . lk2) + diff is one learned number per
layer. Full causal mask, no rotation; the queries are multiplied by a
position-dependent temperature 1 + coef * ln(floor((p + 1) / every) + 1).
Biases on q, k, v.

PooledWindowAttention — queries and keys are divided by their per-head RMS
(no weight), the values ARE the keys as projected (before that norm), scores
pass a tanh soft cap, and the mask is a sliding window plus pooled blocks:
beyond the window a token sees one mean key / mean value per block of `pool`
consecutive positions that lies wholly outside the window, in the same
softmax. The means are kept in the cache's pooled rows (fp32), written by
ops.pool_cache_update when a block's last token is stored.

GatedSigmoidAttention — no softmax: a visible key j weighs sigmoid(q . k_j *
scale + b_h) with a learned number b_h per head, and the weights are not
normalised over the keys. Queries and keys pass a per-head RMS norm with a
learned weight (shared by the heads) and then a rotation by position on their
first rot_dims dimensions (pairs i, i + rot_dims/2, YaRN frequency ramp);
full causal mask; head h's result is multiplied by sigmoid(w_g,h . x), an
output gate that reads the mixer's input.

RotaryRowAttention — a configurable mixer: softmax, or sigmoid(score +
b_h) key weights; full causal mask or a sliding window; rotation of the
first rot_dims dimensions of every query and key head in either pairing
(i with i + rot_dims/2, or 2i with 2i + 1) at frequencies the caller hands
in; optionally an RMS norm over the WHOLE query projection and the whole key
projection (before the split into heads) with weights as wide as those; and
optionally rotated values: the value of position j is turned by j over its
whole width before it is cached, and a head's result at position i is turned
back by i, so that the result depends on i - j only.

Any of them may read ANOTHER layer's cache rows (`owns_cache=False`) with
its own queries. All sizes and constants are constructor arguments.
"""

from __future__ import annotations

import math
from typing import Optional

import torch
import torch.nn as nn

from .. import ops
from ..parallel.comm import get_comm
from ..parallel.layers import MergedColumnParallelLinear, RowParallelLinear
from .forward_meta import ForwardMeta
from .rope import yarn_ramp_frequencies


class _RowAttentionBase(nn.Module):
    maps = 1

    def __init__(self, hidden_size: int, heads: int, kv_heads: int, dim: int,
                 value_dim: int, scale: float, norm_eps: float,
                 cache_layer_idx: int, owns_cache: bool, bias: bool,
                 separate_values: bool, extra_sizes=(), own_proj: bool = True):
        super().__init__()
        if get_comm().tp_size != 1:
            raise NotImplementedError(
                "row-cache attention keeps all kv heads of a token in one "
                "cache row; tensor parallelism is not wired up for it")
        if heads % kv_heads != 0:
            raise ValueError(f"{heads} query heads do not divide into "
                             f"{kv_heads} key/value heads")
        self.heads, self.kv_heads = heads, kv_heads
        self.dim, self.vdim = dim, value_dim
        self.scale, self.eps = float(scale), float(norm_eps)
        self.cache_layer_idx, self.owns_cache = cache_layer_idx, owns_cache
        sizes = [heads * self.maps * dim]
        if owns_cache:
            sizes.append(kv_heads * self.maps * dim)
            if separate_values:
                sizes.append(kv_heads * value_dim)
        # widths of the input projections, in order: queries, (keys, values,)
        # then whatever the mixer adds (e.g. gate pre-activations). own_proj
        # False: a caller merges them with other projections of the same
        # input and hands the parts to the mixer's mix()
        self.proj_sizes = sizes + list(extra_sizes)
        self.in_proj = MergedColumnParallelLinear(
            hidden_size, self.proj_sizes, bias=bias) if own_proj else None
        self.o_proj = RowParallelLinear(heads * value_dim, hidden_size)

    def _project(self, x: torch.Tensor):
        parts = self.in_proj.split_output(self.in_proj(x))
        return parts + [None] * (3 - len(parts))


class DifferentialAttention(_RowAttentionBase):
    maps = 2

    def __init__(self, hidden_size: int, heads: int, kv_heads: int, dim: int,
                 value_dim: int, scale: float, diff: float, temp_coef: float,
                 temp_every: int, norm_eps: float, cache_layer_idx: int,
                 owns_cache: bool = True, bias: bool = True):
        super().__init__(hidden_size, heads, kv_heads, dim, value_dim, scale,
                         norm_eps, cache_layer_idx, owns_cache, bias, True)
        self.diff = float(diff)
        self.temp_coef, self.temp_every = float(temp_coef), int(temp_every)
        for name in ("lq1", "lk1", "lq2", "lk2"):
            setattr(self, name, nn.Parameter(torch.empty(dim), requires_grad=False))
        self._lam: Optional[float] = None

    @property
    def lam(self) -> float:
        if self._lam is None:
            d1 = float((self.lq1.double() * self.lk1.double()).sum())
            d2 = float((self.lq2.double() * self.lk2.double()).sum())
            self._lam = math.exp(d1) - math.exp(d2) + self.diff
        return self._lam

    def invalidate_constants(self) -> None:
        self._lam = None

    def forward(self, x: torch.Tensor, meta: ForwardMeta) -> torch.Tensor:
        q, k, v = self._project(x)
        cache = meta.mla_cache.layer(self.cache_layer_idx)
        q32 = ops.qkv_store(q, k, v, meta.positions, meta.slot_mapping, cache,
                            self.dim, None, self.temp_coef, self.temp_every)
        o = ops.row_attention(
            q32, cache, None, meta.block_tables, meta.token_seq(),
            meta.positions, self.heads, self.kv_heads, 2, self.dim, self.vdim,
            0, 0, self.scale, 0.0, self.lam, self.eps, 1.0 - self.diff,
            x.dtype, max_seq_len=meta.max_seq_len,
            query_bounds=meta.query_bounds(),
        )
        return self.o_proj(o)


class PooledWindowAttention(_RowAttentionBase):
    maps = 1

    def __init__(self, hidden_size: int, heads: int, kv_heads: int, dim: int,
                 value_dim: int, scale: float, softcap: float, window: int,
                 pool: int, norm_eps: float, cache_layer_idx: int,
                 owns_cache: bool = True):
        if value_dim != dim:
            raise ValueError("the values are the projected keys: value width "
                             f"{value_dim} must equal the key width {dim}")
        super().__init__(hidden_size, heads, kv_heads, dim, value_dim, scale,
                         norm_eps, cache_layer_idx, owns_cache, False, False)
        self.softcap = float(softcap)
        self.window, self.pool = int(window), int(pool)
        if self.window < 1:
            raise ValueError("window size must be at least 1")

    def invalidate_constants(self) -> None:
        pass

    def forward(self, x: torch.Tensor, meta: ForwardMeta) -> torch.Tensor:
        q, k, _ = self._project(x)
        cache = meta.mla_cache.layer(self.cache_layer_idx)
        pool = meta.mla_cache.pool_layer(self.cache_layer_idx) \
            if self.pool > 0 else None
        q32 = ops.qkv_store(q, k, None, meta.positions, meta.slot_mapping,
                            cache, self.dim, self.eps, 0.0, 0)
        if pool is not None and self.owns_cache:
            ops.pool_cache_update(cache, pool, meta.block_tables,
                                  meta.token_seq(), meta.positions,
                                  meta.slot_mapping, self.pool)
        o = ops.row_attention(
            q32, cache, pool, meta.block_tables, meta.token_seq(),
            meta.positions, self.heads, self.kv_heads, 1, self.dim, self.vdim,
            self.window, self.pool, self.scale, self.softcap, 0.0, None, 1.0,
            x.dtype, max_seq_len=meta.max_seq_len,
            query_bounds=meta.query_bounds(),
        )
        return self.o_proj(o)


class GatedSigmoidAttention(_RowAttentionBase):
    maps = 1

    def __init__(self, hidden_size: int, heads: int, kv_heads: int, dim: int,
                 value_dim: int, scale: float, norm_eps: float,
                 cache_layer_idx: int, owns_cache: bool = True,
                 rot_dims: int = 0, rot_base: float = 10000.0,
                 rot_scaling: Optional[dict] = None, own_proj: bool = True):
        super().__init__(hidden_size, heads, kv_heads, dim, value_dim, scale,
                         norm_eps, cache_layer_idx, owns_cache, False, True,
                         extra_sizes=[heads], own_proj=own_proj)
        if rot_dims % 2 or rot_dims > dim:
            raise ValueError(f"cannot rotate {rot_dims} of {dim} dimensions")
        self.rot_dims = int(rot_dims)
        sc = rot_scaling or {}
        self._freq, self._mult = (None, 1.0)
        if self.rot_dims:
            self._freq, self._mult = yarn_ramp_frequencies(
                self.rot_dims, rot_base, float(sc.get("factor", 1.0)),
                float(sc.get("original", 0.0)), float(sc.get("fast", 32.0)),
                float(sc.get("slow", 1.0)))
        self.q_norm = nn.Parameter(torch.empty(dim), requires_grad=False)
        self.k_norm = nn.Parameter(torch.empty(dim), requires_grad=False)
        self.score_bias = nn.Parameter(torch.empty(heads), requires_grad=False)
        self._f32 = None

    def invalidate_constants(self) -> None:
        self._f32 = None

    def _constants(self, device):
        if self._f32 is None or self._f32[0].device != device:
            self._f32 = (
                self.q_norm.detach().float().contiguous().to(device),
                self.k_norm.detach().float().contiguous().to(device),
                self.score_bias.detach().float().contiguous().to(device),
                self._freq.to(device) if self._freq is not None else None,
            )
        return self._f32

    def mix(self, parts, meta: ForwardMeta, out_dtype) -> torch.Tensor:
        """parts: the projections [q, (k, v,) gate pre-activations] of the
        step's tokens (strided views are fine) -> [T, heads * value_dim]."""
        q, gate = parts[0], parts[-1]
        k, v = (parts[1], parts[2]) if self.owns_cache else (None, None)
        wq, wk, bias, freq = self._constants(q.device)
        cache = meta.mla_cache.layer(self.cache_layer_idx)
        q32 = ops.qkv_store(q, k, v, meta.positions, meta.slot_mapping, cache,
                            self.dim, self.eps, 0.0, 0, q_weight=wq,
                            k_weight=wk, rot_freq=freq, rot_mult=self._mult,
                            rot_dims=self.rot_dims)
        return ops.row_attention(
            q32, cache, None, meta.block_tables, meta.token_seq(),
            meta.positions, self.heads, self.kv_heads, 1, self.dim, self.vdim,
            0, 0, self.scale, 0.0, 0.0, None, 1.0, out_dtype,
            max_seq_len=meta.max_seq_len, query_bounds=meta.query_bounds(),
            head_bias=bias, gate=gate,
        )

    def forward(self, x: torch.Tensor, meta: ForwardMeta) -> torch.Tensor:
        parts = self.in_proj.split_output(self.in_proj(x))
        return self.o_proj(self.mix(parts, meta, x.dtype))


class RotaryRowAttention(_RowAttentionBase):
    maps = 1

    def __init__(self, hidden_size: int, heads: int, kv_heads: int, dim: int,
                 value_dim: int, scale: float, norm_eps: float,
                 cache_layer_idx: int, owns_cache: bool = True, *,
                 rot_dims: int = 0, rot_freq: Optional[torch.Tensor] = None,
                 rot_interleaved: bool = False, qk_norm_whole: bool = False,
                 value_rot_freq: Optional[torch.Tensor] = None,
                 window: int = 0, sigmoid_weights: bool = False,
                 own_proj: bool = True):
        super().__init__(hidden_size, heads, kv_heads, dim, value_dim, scale,
                         norm_eps, cache_layer_idx, owns_cache, False, True,
                         own_proj=own_proj)
        if rot_dims % 2 or rot_dims > dim:
            raise ValueError(f"cannot rotate {rot_dims} of {dim} dimensions")
        if rot_dims and (rot_freq is None or rot_freq.numel() != rot_dims // 2):
            raise ValueError("one frequency per rotated pair is needed")
        if value_rot_freq is not None and (
                value_dim % 2 or value_rot_freq.numel() != value_dim // 2):
            raise ValueError("rotated values need an even width and one "
                             "frequency per pair")
        if window < 0:
            raise ValueError("window size must not be negative")
        self.rot_dims = int(rot_dims)
        self.rot_interleaved = bool(rot_interleaved)
        self.window = int(window)
        self._freq = rot_freq.float().contiguous() if self.rot_dims else None
        self._vfreq = value_rot_freq.float().contiguous() \
            if value_rot_freq is not None else None
        self.qk_norm_whole = bool(qk_norm_whole)
        if self.qk_norm_whole:
            self.q_norm = nn.Parameter(torch.empty(heads * dim), requires_grad=False)
            self.k_norm = nn.Parameter(torch.empty(kv_heads * dim), requires_grad=False)
        self.sigmoid_weights = bool(sigmoid_weights)
        if self.sigmoid_weights:
            self.score_bias = nn.Parameter(torch.empty(heads), requires_grad=False)
        self._f32 = None

    def invalidate_constants(self) -> None:
        self._f32 = None

    def _constants(self, device):
        if self._f32 is None or self._f32[4] != device:
            def f32(p):
                return p.detach().float().contiguous().to(device)
            self._f32 = (
                f32(self.q_norm) if self.qk_norm_whole else None,
                f32(self.k_norm) if self.qk_norm_whole else None,
                f32(self.score_bias) if self.sigmoid_weights else None,
                (self._freq.to(device) if self._freq is not None else None,
                 self._vfreq.to(device) if self._vfreq is not None else None),
                device,
            )
        return self._f32

    def mix(self, parts, meta: ForwardMeta, out_dtype) -> torch.Tensor:
        """parts: the projections [q, (k, v)] of the step's tokens (strided
        views are fine) -> [T, heads * value_dim]."""
        q = parts[0]
        k, v = (parts[1], parts[2]) if self.owns_cache else (None, None)
        wq, wk, bias, (freq, vfreq), _ = self._constants(q.device)
        cache = meta.mla_cache.layer(self.cache_layer_idx)
        # the tokens' cos/sin of the value rotation: the store turns the
        # values by them, the attention kernel turns its results back
        v_cs = torch.empty(q.shape[0], self.vdim, dtype=torch.float32,
                           device=q.device) if vfreq is not None else None
        q32 = ops.qkv_store(
            q, k, v, meta.positions, meta.slot_mapping, cache, self.dim,
            self.eps if self.qk_norm_whole else None, 0.0, 0, q_weight=wq,
            k_weight=wk, rot_freq=freq, rot_mult=1.0, rot_dims=self.rot_dims,
            norm_whole=self.qk_norm_whole, rot_interleaved=self.rot_interleaved,
            v_seg=self.vdim, v_rot_freq=vfreq, v_cs_out=v_cs)
        return ops.row_attention(
            q32, cache, None, meta.block_tables, meta.token_seq(),
            meta.positions, self.heads, self.kv_heads, 1, self.dim, self.vdim,
            self.window, 0, self.scale, 0.0, 0.0, None, 1.0, out_dtype,
            max_seq_len=meta.max_seq_len, query_bounds=meta.query_bounds(),
            head_bias=bias, out_rot_cs=v_cs,
            out_rot_interleaved=self.rot_interleaved,
        )

    def forward(self, x: torch.Tensor, meta: ForwardMeta) -> torch.Tensor:
        parts = self.in_proj.split_output(self.in_proj(x))
        return self.o_proj(self.mix(parts, meta, x.dtype))
