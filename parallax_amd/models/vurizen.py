"""Vurizen: a pre-norm decoder whose config lists its layers one by one. Each
layer names its sequence mixer — gated linear attention ('gla') or
sliding-window latent attention ('latent_attention', optionally reading the
cache rows of an earlier layer through `kv_from`) — with that mixer's sizes,
and a sigmoid-routed, group-limited mixture of experts as feed-forward (or
none). Layer norms carry a bias, every branch is multiplied by a per-channel
layer scale and a global residual multiplier, and the residual stream is fp32
from the embedding to the final norm whatever the activation dtype is.

Nothing here is specific to one checkpoint: every size and constant comes
from the config (per layer) or from a tensor's shape (the decay rank of the
GLA layers). The mechanisms live beside their relatives and take their
constants as arguments: models/linear_attention.GatedLinearAttention,
models/latent_attention.LatentWindowAttention, llama.ResidualLayerNorm,
moe.MoERouter / FusedMoE; the kernels are ops/mix.py.

Checkpoint tensor names: 'embed', 'l<i>.norm1[.b]', 'l<i>.norm2[.b]',
'l<i>.ls1', 'l<i>.ls2', 'l<i>.mix.{q,k,v,g,o,norm,a1,a2,a2.b}' (gla),
'l<i>.mix.{q,dkv,dkv.norm,uk,uv,o}' (latent attention),
'l<i>.mlp.{router,correction,e<j>.{gate,up,down}}', 'final.norm[.b]', 'head'.
"""

from __future__ import annotations

import dataclasses
import math
from typing import Callable, List, Optional

import torch
import torch.nn as nn

from .. import ops
from ..parallel.comm import get_comm
from ..parallel.layers import ColumnParallelLinear, VocabEmbedding
from .config import ModelConfig
from .forward_meta import ForwardMeta
from .latent_attention import LatentWindowAttention
from .linear_attention import GatedLinearAttention
from .llama import ResidualLayerNorm
from .moe import FusedMoE
from .registry import register_model


def _moe_config(cfg: ModelConfig, mlp: dict) -> ModelConfig:
    """The flat MoE fields of ModelConfig for ONE layer's feed-forward."""
    router = mlp["router"]
    groups = router.get("groups") or {}
    return dataclasses.replace(
        cfg,
        num_experts=int(router["experts"]),
        num_experts_per_tok=int(router["top"]),
        moe_intermediate_size=int(mlp["expert"]["ff"]),
        scoring_func="sigmoid",
        norm_topk_prob=True,
        routed_scaling_factor=float(router.get("scale", 1.0)),
        n_group=int(groups.get("count", 1)),
        topk_group=int(groups.get("keep", 1)),
    )


class VurizenLayer(nn.Module):
    def __init__(self, cfg: ModelConfig, spec: dict, mixer: nn.Module):
        super().__init__()
        W = cfg.hidden_size
        self.kind = spec["type"]
        self.mixer = mixer
        self.norm1 = ResidualLayerNorm(W, cfg.rms_norm_eps)
        self.ls1 = nn.Parameter(torch.empty(W), requires_grad=False)
        self.mlp = None
        if spec.get("mlp") is not None:
            self.mlp = FusedMoE(_moe_config(cfg, spec["mlp"]))
            self.mlp.fp32_output = True
            self.norm2 = ResidualLayerNorm(W, cfg.rms_norm_eps)
            self.ls2 = nn.Parameter(torch.empty(W), requires_grad=False)


@register_model("Vurizen")
class VurizenShardModel(nn.Module):
    """Layers [start_layer, end_layer) of a Vurizen stack. The first shard owns
    the embedding, the last one the final norm and the head. Between shards
    the hidden state IS the fp32 residual stream (`hidden_dtype`)."""

    hidden_dtype = torch.float32

    def __init__(self, cfg: ModelConfig, start_layer: int = 0,
                 end_layer: Optional[int] = None):
        super().__init__()
        if cfg.layer_specs is None:
            raise ValueError("Vurizen needs a config with a 'layers' list")
        if get_comm().tp_size != 1:
            raise NotImplementedError(
                "Vurizen shards by layer range (pipeline stages); tensor "
                "parallelism inside a layer is not wired up for it")
        self.cfg = cfg
        self.start_layer = start_layer
        self.end_layer = end_layer if end_layer is not None else cfg.num_layers
        self.is_first = start_layer == 0
        self.is_last = self.end_layer == cfg.num_layers
        self.residual_mult = cfg.residual_mult
        W = cfg.hidden_size
        if self.is_first:
            self.embed_tokens = VocabEmbedding(cfg.vocab_size, W)
        self.layers = nn.ModuleList(self._build_layers(cfg))
        if self.is_last:
            self.norm = ResidualLayerNorm(W, cfg.rms_norm_eps)
            self.lm_head = ColumnParallelLinear(W, cfg.vocab_size, gather_output=True)
        self.rope_cache = None  # angles are computed inside the kernels
        # debugging aid: called with (global layer index, fp32 residual after
        # that layer) when set
        self.tap: Optional[Callable[[int, torch.Tensor], None]] = None

    def _build_layers(self, cfg: ModelConfig) -> List[VurizenLayer]:
        layers = []
        cache_of = {}   # global index of a cache-owning latent layer -> local cache idx
        n_state = 0
        eps = cfg.rms_norm_eps
        W = cfg.hidden_size
        for g in range(self.start_layer, self.end_layer):
            spec = cfg.layer_specs[g]
            mx = spec["mixer"]
            if spec["type"] == "gla":
                mixer = GatedLinearAttention(
                    W, int(mx["heads"]), int(mx["dim"]), int(mx["vdim"]),
                    float(mx["tau"]), eps, n_state,
                    decay_rank=int(mx.get("decay_rank", 32)),
                )
                n_state += 1
            else:
                src = mx.get("kv_from")
                owns = src is None
                if owns:
                    cache_of[g] = len(cache_of)
                    idx = cache_of[g]
                else:
                    if int(src) not in cache_of:
                        raise ValueError(
                            f"layer {g} reads the cache of layer {src}, which "
                            f"is not a cache-owning latent layer of this "
                            f"shard [{self.start_layer}, {self.end_layer})")
                    idx = cache_of[int(src)]
                rot = mx.get("rot") or {}
                mixer = LatentWindowAttention(
                    W, int(mx["heads"]), int(mx["dim"]), int(mx["rot_dim"]),
                    int(mx["vdim"]), int(mx["kv_rank"]), int(mx["mask"]["size"]),
                    float(mx["scale"]), eps, idx, owns,
                    rot_dims=int(rot.get("dims", mx["rot_dim"])),
                    rot_base=float(rot.get("base", 10000.0)),
                    rot_scaling=rot.get("scaling"),
                )
            layers.append(VurizenLayer(cfg, spec, mixer))
        return layers

    @property
    def graph_safe(self) -> bool:
        """Whether a decode forward can be captured into a hipGraph: the
        per-expert loop that serves expert sizes outside the grouped-GEMM
        kernel's tiling reads routing results on the host."""
        W = self.cfg.hidden_size
        return all(
            layer.mlp is None
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
        """hidden [T, width]: embeddings (first shard) or the previous shard's
        fp32 residual. Returns the final-normed activations on the last shard,
        the fp32 residual elsewhere. Each branch output waits in (y, scale)
        and is folded into the residual by the NEXT norm's kernel."""
        resid = hidden.float().contiguous()
        m = self.residual_mult
        y, scale = None, None
        for i, layer in enumerate(self.layers):
            h = layer.norm1(resid, y, scale, m)
            if self.tap is not None and i > 0:
                self.tap(self.start_layer + i - 1, resid)
            y, scale = layer.mixer(h, meta), layer.ls1
            if layer.mlp is not None:
                h = layer.norm2(resid, y, scale, m)
                y, scale = layer.mlp(h), layer.ls2
        if self.is_last:
            out = self.norm(resid, y, scale, m)
        else:
            ops.add_layernorm(resid, y, scale, m, None, None, 0.0, resid.dtype)
            out = resid
        if self.tap is not None and len(self.layers):
            self.tap(self.end_layer - 1, resid)
        return out

    def compute_logits(self, hidden: torch.Tensor) -> torch.Tensor:
        assert self.is_last, "only the last shard computes logits"
        return self.lm_head(
            hidden.to(self.lm_head.weight.dtype).contiguous()
        ).float()

    def finalize_weights(self) -> None:
        for layer in self.layers:
            if isinstance(layer.mixer, LatentWindowAttention):
                layer.mixer.invalidate_constants()

    # -- weight loading ---------------------------------------------------------

    def map_global_layer(self, name: str) -> Optional[str]:
        """Checkpoint name -> 'layers.<local>.<rest>' / 'embed' / 'final...' /
        'head' when this shard holds the tensor, else None."""
        if name == "embed":
            return name if self.is_first else None
        if name in ("final.norm", "final.norm.b", "head"):
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
        if local == "head":
            self.lm_head.load_full_weight(t)
            return True
        if local == "final.norm":
            self.norm.weight.data.copy_(t)
            return True
        if local == "final.norm.b":
            self.norm.bias.data.copy_(t)
            return True
        parts = local.split(".")
        layer: VurizenLayer = self.layers[int(parts[1])]
        key = ".".join(parts[2:])
        if layer.mlp is None and key in ("norm2", "norm2.b", "ls2"):
            return False  # a layer without feed-forward has no use for them
        if key in ("norm1", "norm2"):
            getattr(layer, key).weight.data.copy_(t)
        elif key in ("norm1.b", "norm2.b"):
            getattr(layer, key[:-2]).bias.data.copy_(t)
        elif key in ("ls1", "ls2"):
            getattr(layer, key).data.copy_(t)
        elif parts[2] == "mix":
            return self._load_mixer(layer.mixer, ".".join(parts[3:]), t)
        elif parts[2] == "mlp" and layer.mlp is not None:
            return self._load_mlp(layer.mlp, parts[3:], t)
        else:
            return False
        return True

    @staticmethod
    def _load_mixer(mixer: nn.Module, key: str, t: torch.Tensor) -> bool:
        if isinstance(mixer, GatedLinearAttention):
            slot = {"q": 0, "k": 1, "v": 2, "g": 3}.get(key)
            if slot is not None:
                mixer.in_proj.load_full_weight_part(slot, t)
            elif key == "o":
                mixer.o_proj.load_full_weight(t)
            elif key == "norm":
                mixer.norm_weight.data.copy_(t)
            elif key in ("a1", "a2"):
                mixer.load_decay(key, t)
            elif key == "a2.b":
                mixer.decay_bias.data.copy_(t)
            else:
                return False
            return True
        if key == "q":
            mixer.in_proj.load_full_weight_part(0, t)
        elif key == "dkv" and mixer.owns_cache:
            mixer.in_proj.load_full_weight_part(1, t)
        elif key == "dkv.norm" and mixer.owns_cache:
            mixer.latent_norm.data.copy_(t)
        elif key == "uk":
            mixer.w_uk.data.copy_(t.view(mixer.heads, mixer.dn, mixer.rank))
        elif key == "uv":
            mixer.w_uv.data.copy_(t.view(mixer.heads, mixer.dv, mixer.rank))
        elif key == "o":
            mixer.o_proj.load_full_weight(t)
        else:
            return False
        return True

    @staticmethod
    def _load_mlp(moe: FusedMoE, parts: List[str], t: torch.Tensor) -> bool:
        if parts == ["router"]:
            moe.router.weight.data.copy_(t)
        elif parts == ["correction"]:
            moe.router.e_score_correction_bias.data.copy_(t.float())
        elif len(parts) == 2 and parts[0][:1] == "e" and parts[0][1:].isdigit():
            e = int(parts[0][1:])
            if parts[1] == "gate":
                moe.load_expert_gate(e, t)
            elif parts[1] == "up":
                moe.load_expert_up(e, t)
            elif parts[1] == "down":
                moe.load_expert_down(e, t)
            else:
                return False
        else:
            return False
        return True

    @torch.no_grad()
    def init_random(self, seed: int = 1234) -> None:
        """Synthetic weights for benchmarking: projections ~ N(0, 1/fan_in),
        norms and layer scales 1, biases 0, decay bias 2 (slow decay)."""
        g = torch.Generator().manual_seed(seed)
        for name, p in self.named_parameters():
            if name.endswith(("norm.weight", "norm1.weight", "norm2.weight",
                              "norm_weight", "latent_norm", "ls1", "ls2")):
                p.data.fill_(1.0)
            elif name.endswith("decay_bias"):
                p.data.fill_(2.0)
            elif name.endswith(("bias", "e_score_correction_bias")):
                p.data.zero_()
            else:
                fan_in = p.shape[-1]
                p.data.copy_(
                    torch.randn(p.shape, generator=g, dtype=torch.float32)
                    .mul_(1.0 / math.sqrt(fan_in)).to(p.dtype)
                )
        self.finalize_weights()
