"""Zabusun: a decoder whose config lists its layers one by one, like Vurizen's
and Sogidra's, with these pieces:

* the embedding passes an RMS norm before the first layer; the logits reuse
  the embedding table after a final norm and are multiplied by `logit_scale`;
* layer type 'parallel': TWO mixers read the same input side by side and
  their results add up with one scale each: sigmoid-weighted attention with
  grouped heads, q/k norm, partial rotation, a per-head score bias and a
  per-head output gate (row_attention.GatedSigmoidAttention), and a minGRU
  (linear_attention.MinGRU);
* feed-forward: a clamped gated linear unit: with a = W_gate h cut off above
  at L and b = W_up h cut off at -L and L, W_down (a sigma(1.702 a) (1 + b)),
  either dense or as sigmoid-routed experts whose routing weight (the chosen
  expert's own score, not renormalised) multiplies the expert's INPUT;
* the norm sits on a sublayer's OUTPUT only: x += norm(sublayer(x)); the
  sublayers read the residual stream itself.

The residual stream and every norm are fp32 whatever the activation dtype;
each residual step (scale and add the two mixers, norm, add, round the next
sublayer's input) is ONE kernel, ops.branch_rmsnorm_add. One merged GEMM
projects the layer input for both mixers. Every size and constant comes from
the config or a tensor's shape; layers shard by range (pipeline stages), the
fp32 stream travels between stages.

Checkpoint tensor names: 'embed', 'embed.norm', 'final.norm', 'l<i>.norm1',
'l<i>.norm2', 'l<i>.mix.left.{q,k,v,q.norm,k.norm,pb,g,o}',
'l<i>.mix.right.{z,z.b,x,x.b,g,o}', 'l<i>.mlp.{gate,up,down}' (dense),
'l<i>.mlp.{router,e<j>.{gate,up,down}}' (experts).
"""

from __future__ import annotations

import dataclasses
import math
from typing import Callable, List, Optional

import torch
import torch.nn as nn

from .. import ops
from ..parallel.comm import get_comm
from ..parallel.layers import (
    MergedColumnParallelLinear, RowParallelLinear, VocabEmbedding,
)
from .config import ModelConfig
from .forward_meta import ForwardMeta
from .linear_attention import MinGRU
from .moe import FusedMoE
from .registry import register_model
from .row_attention import GatedSigmoidAttention


class ParallelMixer(nn.Module):
    """Two mixers over the same input: out = left_scale * left(h) +
    right_scale * right(h). The input projections of both are one GEMM; the
    two results stay apart (forward returns both) so that the caller's
    residual kernel scales and adds them in fp32."""

    def __init__(self, hidden_size: int, left: nn.Module, right: nn.Module,
                 left_scale: float, right_scale: float):
        super().__init__()
        self.left, self.right = left, right
        self.left_scale, self.right_scale = float(left_scale), float(right_scale)
        self.n_left = len(left.proj_sizes)
        self.in_proj = MergedColumnParallelLinear(
            hidden_size, list(left.proj_sizes) + list(right.proj_sizes))
        self._right_width = sum(right.proj_sizes)

    def invalidate_constants(self) -> None:
        self.left.invalidate_constants()
        self.right.invalidate_constants()

    def forward(self, h: torch.Tensor, meta: ForwardMeta):
        y = self.in_proj(h)
        parts = self.in_proj.split_output(y)
        a = self.left.o_proj(self.left.mix(parts[: self.n_left], meta, h.dtype))
        # the right mixer's pre-activations are adjacent columns of y
        b = self.right.o_proj(
            self.right.mix(y[:, y.shape[1] - self._right_width:], meta))
        return a, b


class ClampedGluMLP(nn.Module):
    """W_down (a sigma(alpha a) (1 + b)) with a = W_gate h cut off above at
    `limit` and b = W_up h cut off at -limit and +limit."""

    alpha = 1.702

    def __init__(self, hidden_size: int, ff: int, limit: float):
        super().__init__()
        self.intermediate_size = ff
        self.limit = float(limit)
        self.gate_up = MergedColumnParallelLinear(hidden_size, [ff, ff])
        self.down = RowParallelLinear(ff, hidden_size)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return self.down(ops.clamped_glu(self.gate_up(x), self.limit, self.alpha))


def _expert_config(cfg: ModelConfig, mlp: dict) -> ModelConfig:
    """The flat MoE fields of ModelConfig for ONE layer's experts: sigmoid
    scores, the best `top`, weights = the chosen scores as they are."""
    router = mlp["router"]
    return dataclasses.replace(
        cfg,
        num_experts=int(router["experts"]),
        num_experts_per_tok=int(router["top"]),
        moe_intermediate_size=int(mlp["expert"]["ff"]),
        scoring_func="sigmoid",
        norm_topk_prob=False,
        routed_scaling_factor=1.0,
        n_group=1,
        topk_group=1,
    )


def _mlp_kind(mlp: dict) -> str:
    return mlp.get("kind", "moe" if "router" in mlp else "dense")


class ZabusunLayer(nn.Module):
    def __init__(self, cfg: ModelConfig, spec: dict, mixer: nn.Module):
        super().__init__()
        W = cfg.hidden_size
        self.kind = spec["type"]
        self.mixer = mixer
        self.norm1 = nn.Parameter(torch.empty(W), requires_grad=False)
        self.mlp = None
        mlp = spec.get("mlp")
        if mlp is not None:
            if _mlp_kind(mlp) == "dense":
                self.mlp = ClampedGluMLP(W, int(mlp["ff"]), float(mlp["limit"]))
            else:
                self.mlp = FusedMoE(_expert_config(cfg, mlp),
                                    act_limit=float(mlp["expert"]["limit"]))
                self.mlp.fp32_output = True
                self.mlp.weight_on_input = True
            self.norm2 = nn.Parameter(torch.empty(W), requires_grad=False)


@register_model("Zabusun")
class ZabusunShardModel(nn.Module):
    """Layers [start_layer, end_layer) of a Zabusun stack. The first shard
    owns the embedding and its norm, the last one the final norm and the
    logits (it keeps the embedding table for them). Between shards the hidden
    state IS the fp32 residual stream (`hidden_dtype`)."""

    hidden_dtype = torch.float32

    def __init__(self, cfg: ModelConfig, start_layer: int = 0,
                 end_layer: Optional[int] = None):
        super().__init__()
        if cfg.layer_specs is None:
            raise ValueError("Zabusun needs a config with a 'layers' list")
        if get_comm().tp_size != 1:
            raise NotImplementedError(
                "Zabusun shards by layer range (pipeline stages); tensor "
                "parallelism inside a layer is not wired up for it")
        self.cfg = cfg
        self.start_layer = start_layer
        self.end_layer = end_layer if end_layer is not None else cfg.num_layers
        self.is_first = start_layer == 0
        self.is_last = self.end_layer == cfg.num_layers
        self.eps = cfg.rms_norm_eps
        self.logit_scale = float(cfg.logit_scale)
        W = cfg.hidden_size
        if self.is_first or self.is_last:
            self.embed_tokens = VocabEmbedding(cfg.vocab_size, W)
        if self.is_first:
            self.embed_norm = nn.Parameter(torch.empty(W), requires_grad=False)
        self.layers = nn.ModuleList(self._build_layers(cfg))
        if self.is_last:
            self.norm = nn.Parameter(torch.empty(W), requires_grad=False)
        self.rope_cache = None  # angles are computed inside the kernels
        # debugging aid: called with (global layer index, fp32 residual after
        # that layer) when set
        self.tap: Optional[Callable[[int, torch.Tensor], None]] = None

    def _build_layers(self, cfg: ModelConfig) -> List[ZabusunLayer]:
        layers = []
        W, eps = cfg.hidden_size, cfg.rms_norm_eps
        for n, g in enumerate(range(self.start_layer, self.end_layer)):
            spec = cfg.layer_specs[g]
            if spec["type"] != "parallel":
                raise ValueError(f"layer type {spec['type']!r} is not part of "
                                 "this design")
            mx = spec["mixer"]
            lf, rt = mx["left"], mx["right"]
            rot = lf.get("rot") or {}
            # every layer owns cache entry n and state entry n of this shard
            left = GatedSigmoidAttention(
                W, int(lf["heads"]), int(lf.get("kv_heads", lf["heads"])),
                int(lf["dim"]), int(lf.get("vdim", lf["dim"])),
                float(lf["scale"]), eps, n, True,
                rot_dims=int(rot.get("dims", 0)),
                rot_base=float(rot.get("base", 10000.0)),
                rot_scaling=rot.get("scaling"), own_proj=False,
            )
            right = MinGRU(W, int(rt["width"]), n, own_proj=False)
            mixer = ParallelMixer(W, left, right,
                                  float(mx.get("left_scale", 1.0)),
                                  float(mx.get("right_scale", 1.0)))
            layers.append(ZabusunLayer(cfg, spec, mixer))
        return layers

    @property
    def graph_safe(self) -> bool:
        """Whether a decode forward can be captured into a hipGraph: the
        per-expert loop that serves expert sizes outside the grouped-GEMM
        kernel's tiling reads routing results on the host."""
        W = self.cfg.hidden_size
        return all(
            not isinstance(layer.mlp, FusedMoE)
            or FusedMoE.grouped_kernel_fits(W, layer.mlp.intermediate_size)
            for layer in self.layers
        )

    @property
    def num_local_layers(self) -> int:
        return len(self.layers)

    def embed(self, input_ids: torch.Tensor) -> torch.Tensor:
        assert self.is_first, "only the first shard embeds tokens"
        return self.embed_tokens(input_ids)

    def forward(self, hidden: torch.Tensor, meta: ForwardMeta) -> torch.Tensor:
        """hidden [T, width]: embedding rows (first shard) or the previous
        shard's fp32 residual. Returns the final-normed activations on the
        last shard, the fp32 residual elsewhere."""
        dt = self.layers[0].norm1.dtype if len(self.layers) else hidden.dtype
        eps = self.eps
        if self.is_first:
            x, h = ops.branch_rmsnorm_add(None, hidden, None, 1.0, 0.0,
                                          self.embed_norm, eps, dt)
        else:
            x = hidden.float().contiguous()
            h = x.to(dt)
        for i, layer in enumerate(self.layers):
            mixer = layer.mixer
            a, b = mixer(h, meta)
            x, h = ops.branch_rmsnorm_add(x, a, b, mixer.left_scale,
                                          mixer.right_scale, layer.norm1, eps, dt)
            if layer.mlp is not None:
                x, h = ops.branch_rmsnorm_add(x, layer.mlp(h), None, 1.0, 0.0,
                                              layer.norm2, eps, dt)
            if self.tap is not None:
                self.tap(self.start_layer + i, x)
        if not self.is_last:
            return x
        return ops.branch_rmsnorm_add(None, x, None, 1.0, 0.0, self.norm, eps,
                                      dt, keep_stream=False)[1]

    def compute_logits(self, hidden: torch.Tensor) -> torch.Tensor:
        assert self.is_last, "only the last shard computes logits"
        w = self.embed_tokens.weight
        return ops.linear(hidden.to(w.dtype).contiguous(), w).float() \
            * self.logit_scale

    def finalize_weights(self) -> None:
        for layer in self.layers:
            layer.mixer.invalidate_constants()

    # -- weight loading ---------------------------------------------------------

    def map_global_layer(self, name: str) -> Optional[str]:
        """Checkpoint name -> 'layers.<local>.<rest>' or the name itself when
        this shard holds the tensor, else None."""
        if name == "embed":
            return name if (self.is_first or self.is_last) else None
        if name == "embed.norm":
            return name if self.is_first else None
        if name == "final.norm":
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
            return True
        if local == "embed.norm":
            self.embed_norm.data.copy_(t)
            return True
        if local == "final.norm":
            self.norm.data.copy_(t)
            return True
        parts = local.split(".")
        layer: ZabusunLayer = self.layers[int(parts[1])]
        key = ".".join(parts[2:])
        if key == "norm1":
            layer.norm1.data.copy_(t)
        elif key == "norm2":
            if layer.mlp is None:
                return False  # a layer without feed-forward has no use for it
            layer.norm2.data.copy_(t)
        elif parts[2] == "mix" and len(parts) > 4:
            return self._load_mixer(layer.mixer, parts[3], ".".join(parts[4:]), t)
        elif parts[2] == "mlp" and layer.mlp is not None:
            return self._load_mlp(layer.mlp, parts[3:], t)
        else:
            return False
        return True

    @staticmethod
    def _load_mixer(mixer: ParallelMixer, side: str, key: str,
                    t: torch.Tensor) -> bool:
        if side == "left":
            m = mixer.left
            slot = {"q": 0, "k": 1, "v": 2, "g": 3}.get(key)
            if slot is not None:
                mixer.in_proj.load_full_weight_part(slot, t)
            elif key == "q.norm":
                m.q_norm.data.copy_(t)
            elif key == "k.norm":
                m.k_norm.data.copy_(t)
            elif key == "pb":
                m.score_bias.data.copy_(t)
            elif key == "o":
                m.o_proj.load_full_weight(t)
            else:
                return False
            return True
        if side == "right":
            m = mixer.right
            slot = {"z": 0, "x": 1, "g": 2}.get(key)
            if slot is not None:
                mixer.in_proj.load_full_weight_part(mixer.n_left + slot, t)
            elif key == "z.b":
                m.z_bias.data.copy_(t)
            elif key == "x.b":
                m.x_bias.data.copy_(t)
            elif key == "o":
                m.o_proj.load_full_weight(t)
            else:
                return False
            return True
        return False

    @staticmethod
    def _load_mlp(mlp: nn.Module, parts: List[str], t: torch.Tensor) -> bool:
        if isinstance(mlp, ClampedGluMLP):
            if parts == ["gate"]:
                mlp.gate_up.load_full_weight_part(0, t)
            elif parts == ["up"]:
                mlp.gate_up.load_full_weight_part(1, t)
            elif parts == ["down"]:
                mlp.down.load_full_weight(t)
            else:
                return False
            return True
        if parts == ["router"]:
            mlp.router.weight.data.copy_(t)
        elif len(parts) == 2 and parts[0][:1] == "e" and parts[0][1:].isdigit():
            e = int(parts[0][1:])
            if parts[1] == "gate":
                mlp.load_expert_gate(e, t)
            elif parts[1] == "up":
                mlp.load_expert_up(e, t)
            elif parts[1] == "down":
                mlp.load_expert_down(e, t)
            else:
                return False
        else:
            return False
        return True

    @torch.no_grad()
    def init_random(self, seed: int = 1234) -> None:
        """Synthetic weights for benchmarking: projections ~ N(0, 1/fan_in),
        norm weights 1, biases small, score biases negative (so that the
        unnormalised key weights stay small over long contexts)."""
        g = torch.Generator().manual_seed(seed)
        for name, p in self.named_parameters():
            leaf = name.rsplit(".", 1)[-1]
            if leaf in ("norm", "norm1", "norm2", "embed_norm", "q_norm", "k_norm"):
                p.data.fill_(1.0)
            elif leaf == "score_bias":
                p.data.fill_(-4.0)
            elif leaf == "e_score_correction_bias":
                p.data.zero_()
            elif leaf in ("z_bias", "x_bias"):
                p.data.copy_(torch.randn(p.shape, generator=g).mul_(0.1).to(p.dtype))
            else:
                p.data.copy_(
                    torch.randn(p.shape, generator=g, dtype=torch.float32)
                    .mul_(1.0 / math.sqrt(p.shape[-1])).to(p.dtype))
        self.finalize_weights()
