"""Pudizen: a decoder whose config lists its layers one by one, like Vurizen's,
Sogidra's and Zabusun's, with these pieces:

* embedding: the token's row times `embedding.scale`, plus a row of a second
  table picked by a hash of the (previous token, token) pair
  (parallel.layers.PairHashEmbedding); the previous token comes from the
  request's own token list (ForwardMeta.prev_ids), so it survives any cut of a
  prompt into portions;
* one norm per layer, read by BOTH sublayers, which run side by side:
  h = norm(x), x <- x + (mixer(h) + ff(h)). The norm is an RMS norm taken in
  `norm.groups` equal consecutive parts of the width, each divided by its own
  root mean square, the whole times a learned weight;
* mixer 'attention': grouped heads, RMS norm over the WHOLE query projection
  and the whole key projection (weights that wide), rotation of the first
  rot.dims dimensions of every head (dimension i with i + dims/2, frequencies
  scaled by wavelength), VALUES rotated by their position over their whole
  width and the head's result rotated back by the query's position, full
  causal mask, softmax (row_attention.RotaryRowAttention);
* mixer 'attention_2': grouped heads, rotation of pairs (2i, 2i + 1), sliding
  window, key weights sigmoid(score + b_h) without normalisation over the
  keys (the same class, other switches);
* mixer 'latent_attention': keys and values expanded from a cached RMS-normed
  latent, no positions, full causal mask, softmax, a sigmoid output gate per
  head (latent_attention.GatedLatentAttention);
* feed-forward: W_down relu(W_up h)^2, or none;
* logits: the same grouped norm, then a separate output matrix.

The residual stream and every norm are fp32 whatever the activation dtype;
one kernel per layer (ops.group_rmsnorm_add) adds both sublayers' results to
the stream and norms it for the next layer. One merged GEMM projects the
layer's input for the mixer AND the feed-forward. Every size and constant
comes from the config or a tensor's shape; layers shard by range (pipeline
stages), the fp32 stream travels between stages.

Checkpoint tensor names: 'embed', 'bigram', 'final.norm', 'head',
'l<i>.norm1', 'l<i>.mix.{q,k,v,o}' with '{q.norm,k.norm}' ('attention') or
'pb' ('attention_2'), 'l<i>.mix.{q,dkv,dkv.norm,uk,uv,g,o}'
('latent_attention'), 'l<i>.mlp.{up,down}'.
"""

from __future__ import annotations

import math
from typing import Callable, List, Optional

import torch
import torch.nn as nn

from .. import ops
from ..parallel.comm import get_comm
from ..parallel.layers import (
    ColumnParallelLinear, MergedColumnParallelLinear, PairHashEmbedding,
    RowParallelLinear,
)
from .config import ModelConfig
from .forward_meta import ForwardMeta
from .latent_attention import GatedLatentAttention
from .registry import register_model
from .rope import wavelength_scaled_frequencies
from .row_attention import RotaryRowAttention


def _rot_frequencies(rot: dict) -> Optional[torch.Tensor]:
    dims = int(rot.get("dims", 0))
    if not dims:
        return None
    sc = rot.get("scaling") or {}
    return wavelength_scaled_frequencies(
        dims, float(rot.get("base", 10000.0)), float(sc.get("factor", 1.0)),
        float(sc.get("low", 1.0)), float(sc.get("high", 4.0)),
        float(sc.get("original", 0.0)))


def build_mixer(kind: str, mx: dict, hidden_size: int, eps: float,
                cache_layer_idx: int) -> nn.Module:
    """The mixer of one layer from its config entry; its input projections
    are left to the layer (own_proj False)."""
    if kind == "latent_attention":
        return GatedLatentAttention(
            hidden_size, int(mx["heads"]), int(mx["dim"]),
            int(mx.get("vdim", mx["dim"])), int(mx["kv_rank"]),
            float(mx["scale"]), eps, cache_layer_idx, own_proj=False)
    rot = mx.get("rot") or {}
    heads = int(mx["heads"])
    dim, vdim = int(mx["dim"]), int(mx.get("vdim", mx["dim"]))
    window = int((mx.get("mask") or {}).get("size", 0))
    common = dict(rot_dims=int(rot.get("dims", 0)), rot_freq=_rot_frequencies(rot),
                  window=window, own_proj=False)
    if kind == "attention":
        # values turn by their position at unscaled frequencies over vdim
        vfreq = wavelength_scaled_frequencies(vdim, float(rot.get("base", 10000.0)))
        return RotaryRowAttention(
            hidden_size, heads, int(mx.get("kv_heads", heads)), dim, vdim,
            float(mx["scale"]), eps, cache_layer_idx, True,
            rot_interleaved=False, qk_norm_whole=True, value_rot_freq=vfreq,
            sigmoid_weights=False, **common)
    if kind == "attention_2":
        return RotaryRowAttention(
            hidden_size, heads, int(mx.get("kv_heads", heads)), dim, vdim,
            float(mx["scale"]), eps, cache_layer_idx, True,
            rot_interleaved=True, qk_norm_whole=False, value_rot_freq=None,
            sigmoid_weights=True, **common)
    raise ValueError(f"layer type {kind!r} is not part of this design")


class PudizenLayer(nn.Module):
    """norm -> (mixer, feed-forward) side by side. The up projection of the
    feed-forward and the mixer's input projections are ONE GEMM over the
    normed input; forward returns the two results apart, the caller's
    residual kernel adds them in fp32."""

    def __init__(self, cfg: ModelConfig, spec: dict, mixer: nn.Module):
        super().__init__()
        W = cfg.hidden_size
        self.kind = spec["type"]
        self.mixer = mixer
        self.norm1 = nn.Parameter(torch.empty(W), requires_grad=False)
        mlp = spec.get("mlp")
        self.ff = int(mlp["ff"]) if mlp is not None else 0
        # [feed-forward up | the mixer's projections]
        sizes = ([self.ff] if self.ff else []) + list(mixer.proj_sizes)
        self.in_proj = MergedColumnParallelLinear(W, sizes)
        self.down = RowParallelLinear(self.ff, W) if self.ff else None

    def forward(self, h: torch.Tensor, meta: ForwardMeta):
        parts = self.in_proj.split_output(self.in_proj(h))
        first = 1 if self.ff else 0
        a = self.mixer.o_proj(self.mixer.mix(parts[first:], meta, h.dtype))
        b = self.down(ops.relu_squared(parts[0])) if self.ff else None
        return a, b


@register_model("Pudizen")
class PudizenShardModel(nn.Module):
    """Layers [start_layer, end_layer) of a Pudizen stack. The first shard
    owns the embedding tables, the last one the final norm and the output
    matrix. Between shards the hidden state IS the fp32 residual stream
    (`hidden_dtype`)."""

    hidden_dtype = torch.float32
    # the engine hands embed() each token's predecessor in its sequence
    uses_prev_tokens = True
    graph_safe = True

    def __init__(self, cfg: ModelConfig, start_layer: int = 0,
                 end_layer: Optional[int] = None):
        super().__init__()
        if cfg.layer_specs is None:
            raise ValueError("Pudizen needs a config with a 'layers' list")
        if get_comm().tp_size != 1:
            raise NotImplementedError(
                "Pudizen shards by layer range (pipeline stages); tensor "
                "parallelism inside a layer is not wired up for it")
        self.cfg = cfg
        self.start_layer = start_layer
        self.end_layer = end_layer if end_layer is not None else cfg.num_layers
        self.is_first = start_layer == 0
        self.is_last = self.end_layer == cfg.num_layers
        self.eps = cfg.rms_norm_eps
        self.groups = int(cfg.norm_groups)
        W = cfg.hidden_size
        if self.is_first:
            # a config without a pair table: one bucket whose rows stay zero
            ph = cfg.pair_hash or {"buckets": 1, "mul_prev": 0, "mul_cur": 0}
            self.embed_tokens = PairHashEmbedding(
                cfg.vocab_size, W, ph["buckets"], ph["mul_prev"], ph["mul_cur"],
                cfg.embed_scale)
            self.embed_tokens.pair.data.zero_()
        self.layers = nn.ModuleList(
            PudizenLayer(cfg, cfg.layer_specs[g],
                         build_mixer(cfg.layer_specs[g]["type"],
                                     cfg.layer_specs[g]["mixer"], W, self.eps, n))
            for n, g in enumerate(range(self.start_layer, self.end_layer)))
        if self.is_last:
            self.norm = nn.Parameter(torch.empty(W), requires_grad=False)
            self.lm_head = ColumnParallelLinear(W, cfg.vocab_size)
        self.rope_cache = None  # angles are computed inside the kernels
        # debugging aid: called with (global layer index, fp32 residual after
        # that layer) when set
        self.tap: Optional[Callable[[int, torch.Tensor], None]] = None

    @property
    def num_local_layers(self) -> int:
        return len(self.layers)

    def embed(self, input_ids: torch.Tensor,
              prev_ids: Optional[torch.Tensor] = None) -> torch.Tensor:
        assert self.is_first, "only the first shard embeds tokens"
        if prev_ids is None:
            raise ValueError("this design's embedding needs every token's "
                             "predecessor (ForwardMeta.prev_ids)")
        return self.embed_tokens(input_ids, prev_ids)

    def forward(self, hidden: torch.Tensor, meta: ForwardMeta) -> torch.Tensor:
        """hidden [T, width]: the embedding sum (first shard) or the previous
        shard's fp32 residual. Returns the final-normed activations on the
        last shard, the fp32 residual elsewhere."""
        x = hidden.float().contiguous()
        n = len(self.layers)
        tail = self.norm if self.is_last else None
        if n == 0:
            out = ops.group_rmsnorm_add(x, None, None, tail, self.groups,
                                        self.eps, tail.dtype) if tail is not None else None
            return out if self.is_last else x
        dt = self.layers[0].norm1.dtype
        h = ops.group_rmsnorm_add(x, None, None, self.layers[0].norm1,
                                  self.groups, self.eps, dt)
        for i, layer in enumerate(self.layers):
            a, b = layer(h, meta)
            w_next = self.layers[i + 1].norm1 if i + 1 < n else tail
            h = ops.group_rmsnorm_add(x, a, b, w_next, self.groups, self.eps, dt)
            if self.tap is not None:
                self.tap(self.start_layer + i, x)
        return h if self.is_last else x

    def compute_logits(self, hidden: torch.Tensor) -> torch.Tensor:
        assert self.is_last, "only the last shard computes logits"
        return self.lm_head(hidden.contiguous()).float()

    def finalize_weights(self) -> None:
        for layer in self.layers:
            layer.mixer.invalidate_constants()

    # -- weight loading ---------------------------------------------------------

    def map_global_layer(self, name: str) -> Optional[str]:
        """Checkpoint name -> 'layers.<local>.<rest>' or the name itself when
        this shard holds the tensor, else None."""
        if name in ("embed", "bigram"):
            return name if self.is_first else None
        if name in ("final.norm", "head"):
            return name if self.is_last else None
        if name.startswith("l"):
            first, _, rest = name.partition(".")
            if first[1:].isdigit() and rest:
                g = int(first[1:])
                if self.start_layer <= g < self.end_layer:
                    return f"layers.{g - self.start_layer}.{rest}"
        return None

    def load_hf_weight(self, name: str, tensor: torch.Tensor) -> bool:
        local = self.map_global_layer(name)
        if local is None:
            return False
        t = tensor.to(torch.bfloat16) if tensor.is_floating_point() else tensor
        if local == "embed":
            self.embed_tokens.weight.data.copy_(t)
        elif local == "bigram":
            self.embed_tokens.pair.data.copy_(t)
        elif local == "final.norm":
            self.norm.data.copy_(t)
        elif local == "head":
            self.lm_head.load_full_weight(t)
        else:
            parts = local.split(".")
            layer: PudizenLayer = self.layers[int(parts[1])]
            key = ".".join(parts[3:])
            if parts[2] == "norm1" and len(parts) == 3:
                layer.norm1.data.copy_(t)
            elif parts[2] == "mix":
                return self._load_mixer(layer, key, t)
            elif parts[2] == "mlp" and layer.ff:
                if key == "up":
                    layer.in_proj.load_full_weight_part(0, t)
                elif key == "down":
                    layer.down.load_full_weight(t)
                else:
                    return False
            else:
                return False
        return True

    @staticmethod
    def _load_mixer(layer: PudizenLayer, key: str, t: torch.Tensor) -> bool:
        m = layer.mixer
        first = 1 if layer.ff else 0
        if isinstance(m, GatedLatentAttention):
            slot = {"q": 0, "dkv": 1, "g": 2}.get(key)
            if slot is not None:
                layer.in_proj.load_full_weight_part(first + slot, t)
            elif key == "dkv.norm":
                m.latent_norm.data.copy_(t)
            elif key == "uk":
                m.w_uk.data.copy_(t.view(m.heads, m.dim, m.rank))
            elif key == "uv":
                m.w_uv.data.copy_(t.view(m.heads, m.vdim, m.rank))
            elif key == "o":
                m.o_proj.load_full_weight(t)
            else:
                return False
            return True
        slot = {"q": 0, "k": 1, "v": 2}.get(key)
        if slot is not None:
            layer.in_proj.load_full_weight_part(first + slot, t)
        elif key == "q.norm" and m.qk_norm_whole:
            m.q_norm.data.copy_(t)
        elif key == "k.norm" and m.qk_norm_whole:
            m.k_norm.data.copy_(t)
        elif key == "pb" and m.sigmoid_weights:
            m.score_bias.data.copy_(t)
        elif key == "o":
            m.o_proj.load_full_weight(t)
        else:
            return False
        return True

    @torch.no_grad()
    def init_random(self, seed: int = 1234) -> None:
        """Synthetic weights for benchmarking: projections ~ N(0, 1/fan_in),
        norm weights 1, score biases negative (so that the unnormalised key
        weights stay small over long windows)."""
        g = torch.Generator().manual_seed(seed)
        for name, p in self.named_parameters():
            leaf = name.rsplit(".", 1)[-1]
            if leaf in ("norm", "norm1", "q_norm", "k_norm", "latent_norm"):
                p.data.fill_(1.0)
            elif leaf == "score_bias":
                p.data.fill_(-4.0)
            else:
                p.data.copy_(
                    torch.randn(p.shape, generator=g, dtype=torch.float32)
                    .mul_(1.0 / math.sqrt(p.shape[-1])).to(p.dtype))
        self.finalize_weights()
