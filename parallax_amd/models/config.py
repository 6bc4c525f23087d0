"""Model configuration parsed from a HF config.json dict.

Covers the fields used by the supported families (Llama/Qwen2/Qwen3/Qwen3-MoE/
DeepSeek-V3/GPT-OSS/GLM4-MoE) plus layer-type derivation for hybrid stacks —
parity with the reference's utils/layer_types.py:5-20 and config normalization
(utils/utils.py:343)."""

from __future__ import annotations

import json
import os
from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional


# layer-list designs whose every layer keeps one plain cache row per token
# (no pooled rows, no recurrent state slots, no layer reading another's rows)
_PLAIN_ROW_DESIGNS = ("Pudizen",)


@dataclass
class ModelConfig:
    architecture: str = "LlamaForCausalLM"
    model_type: str = "llama"
    vocab_size: int = 32000
    hidden_size: int = 4096
    num_layers: int = 32
    num_heads: int = 32
    num_kv_heads: int = 8
    head_dim: int = 128
    intermediate_size: int = 14336
    rms_norm_eps: float = 1e-5
    rope_theta: float = 500000.0
    rope_scaling: Optional[Dict[str, Any]] = None
    max_position_embeddings: int = 131072
    tie_word_embeddings: bool = False
    attention_bias: bool = False
    o_proj_bias: bool = False
    mlp_bias: bool = False
    qk_norm: bool = False            # qwen3-style per-head q/k RMSNorm
    qk_norm_full: bool = False       # minimax-m2: RMSNorm over the FULL q/k width
    partial_rotary_factor: float = 1.0
    sliding_window: int = -1         # -1 = full attention
    # which layers use the sliding window ("full" layers interleave, gpt-oss)
    layer_types: Optional[List[str]] = None
    eos_token_ids: List[int] = field(default_factory=lambda: [2])
    bos_token_id: Optional[int] = 1
    torch_dtype: str = "bfloat16"

    # -- MoE ------------------------------------------------------------------
    num_experts: int = 0
    num_experts_per_tok: int = 0
    moe_intermediate_size: int = 0
    num_shared_experts: int = 0
    shared_expert_intermediate_size: int = 0
    first_k_dense_layers: int = 0     # deepseek: dense layers before MoE starts
    moe_layer_freq: int = 1
    norm_topk_prob: bool = True
    routed_scaling_factor: float = 1.0
    scoring_func: str = "softmax"     # or "sigmoid" (deepseek v3)
    topk_group: int = 0
    n_group: int = 0
    moe_router_bias: bool = False     # deepseek v3 e_score_correction_bias

    # -- MLA (deepseek) ----------------------------------------------------------
    rope_interleave: bool = False    # GPT-J pairwise rope (deepseek default)
    q_lora_rank: int = 0
    kv_lora_rank: int = 0
    qk_nope_head_dim: int = 0
    qk_rope_head_dim: int = 0
    v_head_dim: int = 0

    # -- DSA indexer (deepseek v3.2 sparse attention) ---------------------------
    index_n_heads: int = 0
    index_head_dim: int = 0
    index_topk: int = 0

    # -- MSA indexer (minimax-m3 block-sparse attention) ------------------------
    index_block_size: int = 0
    index_topk_blocks: int = 0
    index_local_blocks: int = 0

    # -- attention sinks (gpt-oss) --------------------------------------------------
    attention_sinks: bool = False
    use_attn_gate: bool = False    # step3p5 head-wise sigmoid output gate

    # -- hybrid linear attention (qwen3-next gated deltanet) --------------------------
    linear_num_key_heads: int = 0
    linear_num_value_heads: int = 0
    linear_key_head_dim: int = 0
    linear_value_head_dim: int = 0
    linear_conv_kernel_dim: int = 4

    # -- per-layer stacks (vurizen, sogidra, zabusun, pudizen): every layer carries its own mixer and
    # feed-forward description; the flat fields above hold the first layer's
    # values only so that sizing helpers have something to read ----------------
    layer_specs: Optional[List[Dict[str, Any]]] = None
    residual_mult: float = 1.0
    logit_scale: float = 1.0         # the logits are multiplied by this
    norm_groups: int = 1             # RMS norms split the width into this many parts
    embed_scale: float = 1.0         # the token embedding is multiplied by this
    # hashed (previous token, token) embedding: {"buckets", "mul_prev", "mul_cur"}
    pair_hash: Optional[Dict[str, int]] = None

    raw: Dict[str, Any] = field(default_factory=dict, repr=False)

    @property
    def rot_dim(self) -> int:
        return int(self.head_dim * self.partial_rotary_factor)

    @property
    def is_moe(self) -> bool:
        return self.num_experts > 0

    @property
    def is_mla(self) -> bool:
        return self.kv_lora_rank > 0

    # -- cache geometry per local layer (the engine sizes its pools from these) --

    def latent_cache_dims(self, start: int, end: int) -> List[tuple]:
        """Row geometry of every layer in [start, end) that OWNS a row-per-
        token cache entry, as (first part, second part) widths: (latent rank,
        rotated-key width) for compressed-latent layers, (key width, value
        width) over all key/value heads for the row-attention mixers. Layers
        that read another layer's entry (`kv_from`) and layers without a
        paged cache are left out."""
        if self.layer_specs is not None and self.architecture in _PLAIN_ROW_DESIGNS:
            # one row [keys | values] per token for the grouped-head mixers,
            # the latent alone (no rotated key part) for the latent ones
            dims = []
            for sp in self.layer_specs[start:end]:
                mx = sp["mixer"]
                if sp["type"] == "latent_attention":
                    dims.append((int(mx["kv_rank"]), 0))
                else:
                    g = int(mx.get("kv_heads", mx["heads"]))
                    dims.append((g * int(mx["dim"]),
                                 g * int(mx.get("vdim", mx["dim"]))))
            return dims
        if self.layer_specs is not None:
            dims = []
            for sp in self.layer_specs[start:end]:
                mx = sp["mixer"]
                if mx.get("kv_from") is not None:
                    continue
                if sp["type"] == "latent_attention":
                    dims.append((int(mx["kv_rank"]), int(mx["rot_dim"])))
                elif sp["type"] == "attention":      # two score maps per head
                    g = int(mx.get("kv_heads", mx["heads"]))
                    dims.append((g * 2 * int(mx["dim"]), g * int(mx["vdim"])))
                elif sp["type"] == "attention_2":    # values = unnormed keys
                    g = int(mx.get("kv_heads", mx["heads"]))
                    dims.append((g * int(mx["dim"]), g * int(mx["dim"])))
                elif sp["type"] == "parallel":       # the attention half's rows
                    left = mx["left"]
                    g = int(left.get("kv_heads", left["heads"]))
                    dims.append((g * int(left["dim"]),
                                 g * int(left.get("vdim", left["dim"]))))
            return dims
        if not self.is_mla:
            return []
        return [(self.kv_lora_rank, self.qk_rope_head_dim)] * (end - start)

    def pooled_cache_blocks(self, start: int, end: int) -> List[int]:
        """For every cache-owning layer of latent_cache_dims(start, end): the
        number of tokens whose mean row the layer also keeps (pooled blocks
        seen beyond a sliding window), 0 for layers that keep none."""
        if self.layer_specs is None or self.architecture in _PLAIN_ROW_DESIGNS:
            return [0] * len(self.latent_cache_dims(start, end))
        out = []
        for sp in self.layer_specs[start:end]:
            mx = sp["mixer"]
            if mx.get("kv_from") is not None:
                continue
            if sp["type"] in ("latent_attention", "attention", "parallel"):
                out.append(0)
            elif sp["type"] == "attention_2":
                out.append(int((mx.get("mask") or {}).get("pool", 0)))
        return out

    def linear_state_shapes(self, start: int, end: int) -> List[tuple]:
        """(conv-state shape, recurrent-state shape) of every linear-attention
        layer in [start, end)."""
        if self.layer_specs is not None and self.architecture in _PLAIN_ROW_DESIGNS:
            return []
        if self.layer_specs is not None:
            shapes = []
            for sp in self.layer_specs[start:end]:
                mx = sp["mixer"]
                if sp["type"] == "gla":
                    shapes.append(((0,), (int(mx["heads"]), int(mx["dim"]),
                                          int(mx["vdim"]))))
                elif sp["type"] == "parallel":   # the recurrent half: a vector
                    shapes.append(((0,), (int(mx["right"]["width"]),)))
            return shapes
        if not self.has_linear_layers:
            return []
        conv_dim = (2 * self.linear_num_key_heads * self.linear_key_head_dim
                    + self.linear_num_value_heads * self.linear_value_head_dim)
        n = sum(1 for g in range(start, end)
                if self.layer_type(g) == "linear_attention")
        return [((conv_dim, self.linear_conv_kernel_dim - 1),
                 (self.linear_num_value_heads, self.linear_key_head_dim,
                  self.linear_value_head_dim))] * n

    @property
    def is_dsa(self) -> bool:
        return self.index_topk > 0 and self.index_head_dim > 0

    @property
    def is_msa(self) -> bool:
        return self.index_topk_blocks > 0 and self.index_block_size > 0

    @property
    def has_linear_layers(self) -> bool:
        """Whether any layer keeps recurrent state in a per-request slot."""
        if self.layer_specs is not None:
            return self.architecture not in _PLAIN_ROW_DESIGNS and any(
                sp["type"] in ("gla", "parallel") for sp in self.layer_specs)
        return bool(self.layer_types) and "linear_attention" in self.layer_types

    def layer_type(self, layer_idx: int) -> str:
        """'attention' | 'sliding_attention' | 'linear_attention' | 'mla_attention'."""
        if self.layer_specs is not None:
            return self.layer_types[layer_idx]
        if self.is_mla:
            return "mla_attention"
        if self.layer_types is not None:
            return self.layer_types[layer_idx]
        if self.sliding_window > 0:
            return "sliding_attention"
        return "attention"

    def is_moe_layer(self, layer_idx: int) -> bool:
        if not self.is_moe:
            return False
        if layer_idx < self.first_k_dense_layers:
            return False
        return (layer_idx % max(1, self.moe_layer_freq)) == 0

    @classmethod
    def from_layer_list_config(cls, cfg: Dict[str, Any]) -> "ModelConfig":
        """Configs that describe the stack as a list of layers
        ({"architecture": ..., "layers": [{"type", "mixer", "mlp"}, ...],
        "norm": {"eps"}, "vocab", "width", ...}). Mixer types: 'gla',
        'latent_attention' (vurizen); 'attention' (differential softmax
        attention), 'attention_2' (sliding window with pooled blocks)
        (sogidra); 'parallel' (sigmoid attention beside a minGRU, both reading
        the layer's input) (zabusun). Feed-forward kinds: 'moe' (default),
        'dense'. Pudizen reuses three of the names for mixers of its own:
        'attention' (softmax, q/k norm over the whole projection, rotated
        values), 'attention_2' (sliding window, sigmoid key weights),
        'latent_attention' (no positions, gated); its top level also carries
        'embedding' {"scale", "bigram": {"buckets", "mul_prev", "mul_cur"}}
        and 'norm' {"eps", "groups"}."""
        if cfg["architecture"] in _PLAIN_ROW_DESIGNS:
            return cls._from_plain_row_config(cfg)
        layers = cfg["layers"]
        kinds = {"gla": "linear_attention", "latent_attention": "latent_attention",
                 "attention": "diff_attention",
                 "attention_2": "pooled_window_attention",
                 "parallel": "parallel_attention_recurrent"}
        for sp in layers:
            if sp["type"] not in kinds:
                raise ValueError(f"unknown layer type {sp['type']!r}")
            mlp = sp.get("mlp")
            if mlp is not None and mlp.get("kind", "moe") not in ("moe", "dense"):
                raise ValueError(f"unknown feed-forward kind {mlp.get('kind')!r}")
        latent = [sp["mixer"] for sp in layers if sp["type"] == "latent_attention"]
        linear = [sp["mixer"] for sp in layers if sp["type"] == "gla"]
        windowed = [sp["mixer"] for sp in layers if sp["type"] == "attention_2"]
        mlps = [sp["mlp"] for sp in layers if sp.get("mlp") is not None]

        def kind_of(m):   # a feed-forward without a router is a dense one
            return m.get("kind", "moe" if "router" in m else "dense")

        moes = [m for m in mlps if kind_of(m) == "moe"]
        dense = [m for m in mlps if kind_of(m) == "dense"]
        first = layers[0]["mixer"]
        if layers[0]["type"] == "parallel":
            first = first["left"]
        mc = cls(
            architecture=cfg["architecture"],
            model_type=str(cfg["architecture"]).lower(),
            vocab_size=int(cfg["vocab"]),
            hidden_size=int(cfg["width"]),
            num_layers=len(layers),
            num_heads=int(first["heads"]),
            num_kv_heads=int(first.get("kv_heads", first["heads"])),
            head_dim=int(first["dim"]),
            rms_norm_eps=float(cfg["norm"]["eps"]),
            max_position_embeddings=int(cfg.get("max_positions", 1 << 20)),
            layer_types=[kinds[sp["type"]] for sp in layers],
            eos_token_ids=[],
            bos_token_id=None,
            torch_dtype=cfg.get("torch_dtype", "bfloat16"),
            layer_specs=layers,
            residual_mult=float(cfg.get("residual_mult", 1.0)),
            logit_scale=float(cfg.get("logit_scale", 1.0)),
            raw=cfg,
        )
        if latent:
            mc.kv_lora_rank = int(latent[0]["kv_rank"])
            mc.qk_nope_head_dim = int(latent[0]["dim"])
            mc.qk_rope_head_dim = int(latent[0]["rot_dim"])
            mc.v_head_dim = int(latent[0]["vdim"])
            mc.sliding_window = int(latent[0]["mask"]["size"])
        if windowed:
            mc.sliding_window = int(windowed[0]["mask"]["size"])
        if linear:
            mc.linear_num_key_heads = mc.linear_num_value_heads = int(linear[0]["heads"])
            mc.linear_key_head_dim = int(linear[0]["dim"])
            mc.linear_value_head_dim = int(linear[0]["vdim"])
            mc.linear_conv_kernel_dim = 1
        if dense:
            mc.intermediate_size = int(dense[0]["ff"])
        if moes:
            r = moes[0]["router"]
            mc.num_experts = int(r["experts"])
            mc.num_experts_per_tok = int(r["top"])
            mc.moe_intermediate_size = int(moes[0]["expert"]["ff"])
            mc.intermediate_size = mc.moe_intermediate_size
            mc.scoring_func = "sigmoid"
            mc.routed_scaling_factor = float(r.get("scale", 1.0))
            g = r.get("groups") or {}
            mc.n_group = int(g.get("count", 0))
            mc.topk_group = int(g.get("keep", 0))
        return mc

    @classmethod
    def _from_plain_row_config(cls, cfg: Dict[str, Any]) -> "ModelConfig":
        layers = cfg["layers"]
        kinds = {"attention": "attention", "attention_2": "sliding_attention",
                 "latent_attention": "latent_attention"}
        for sp in layers:
            if sp["type"] not in kinds:
                raise ValueError(f"unknown layer type {sp['type']!r}")
            mlp = sp.get("mlp")
            if mlp is not None and mlp.get("kind", "dense") != "dense":
                raise ValueError(f"unknown feed-forward kind {mlp.get('kind')!r}")
        first = layers[0]["mixer"]
        emb = cfg.get("embedding") or {}
        pair = emb.get("bigram")
        norm = cfg.get("norm") or {}
        mc = cls(
            architecture=cfg["architecture"],
            model_type=str(cfg["architecture"]).lower(),
            vocab_size=int(cfg["vocab"]),
            hidden_size=int(cfg["width"]),
            num_layers=len(layers),
            num_heads=int(first["heads"]),
            num_kv_heads=int(first.get("kv_heads", first["heads"])),
            head_dim=int(first["dim"]),
            rms_norm_eps=float(norm.get("eps", 1e-5)),
            max_position_embeddings=int(cfg.get("max_positions", 1 << 20)),
            layer_types=[kinds[sp["type"]] for sp in layers],
            eos_token_ids=[],
            bos_token_id=None,
            torch_dtype=cfg.get("torch_dtype", "bfloat16"),
            layer_specs=layers,
            norm_groups=int(norm.get("groups", 1)),
            embed_scale=float(emb.get("scale", 1.0)),
            pair_hash={k: int(pair[k]) for k in ("buckets", "mul_prev", "mul_cur")}
            if pair else None,
            raw=cfg,
        )
        if mc.hidden_size % mc.norm_groups:
            raise ValueError(f"width {mc.hidden_size} does not split into "
                             f"{mc.norm_groups} norm groups")
        windows = [int(sp["mixer"]["mask"]["size"]) for sp in layers
                   if (sp["mixer"].get("mask") or {}).get("size")]
        if windows:
            mc.sliding_window = windows[0]
        ffs = [int(sp["mlp"]["ff"]) for sp in layers if sp.get("mlp") is not None]
        if ffs:
            mc.intermediate_size = ffs[0]
        return mc

    @classmethod
    def from_hf_config(cls, cfg: Dict[str, Any]) -> "ModelConfig":
        if "architecture" in cfg and isinstance(cfg.get("layers"), list):
            return cls.from_layer_list_config(cfg)
        arch = (cfg.get("architectures") or ["LlamaForCausalLM"])[0]
        num_heads = cfg.get("num_attention_heads", 32)
        hidden = cfg.get("hidden_size", 4096)
        head_dim = cfg.get("head_dim") or hidden // num_heads
        rope_params = cfg.get("rope_parameters") or {}
        eos = cfg.get("eos_token_id", 2)
        eos_ids = eos if isinstance(eos, list) else [eos]
        sliding = cfg.get("sliding_window") or -1
        if cfg.get("use_sliding_window") is False:
            sliding = -1
        layer_types = cfg.get("layer_types")
        mc = cls(
            architecture=arch,
            model_type=cfg.get("model_type", "llama"),
            vocab_size=cfg.get("vocab_size", 32000),
            hidden_size=hidden,
            num_layers=cfg.get("num_hidden_layers", 32),
            num_heads=num_heads,
            num_kv_heads=cfg.get("num_key_value_heads", num_heads),
            head_dim=head_dim,
            intermediate_size=cfg.get("intermediate_size", 4 * hidden),
            rms_norm_eps=cfg.get("rms_norm_eps", 1e-5),
            rope_theta=cfg.get("rope_theta") or rope_params.get("rope_theta", 10000.0),
            rope_scaling=cfg.get("rope_scaling") or (rope_params or None),
            partial_rotary_factor=cfg.get("partial_rotary_factor")
            or rope_params.get("partial_rotary_factor", 1.0),
            max_position_embeddings=cfg.get("max_position_embeddings", 32768),
            tie_word_embeddings=cfg.get("tie_word_embeddings", False),
            attention_bias=cfg.get("attention_bias", cfg.get("qkv_bias", False)),
            o_proj_bias=cfg.get("attention_bias", False)
            and cfg.get("model_type") == "gpt_oss",
            attention_sinks=cfg.get("model_type") == "gpt_oss",
            use_attn_gate=cfg.get("use_head_wise_attn_gate",
                                  cfg.get("model_type") == "step3p5"),
            qk_norm=cfg.get("use_qk_norm", False)
            or cfg.get("model_type", "") in ("qwen3", "qwen3_moe", "qwen3_next",
                                             "minimax_m2", "qwen3_5_text",
                                             "qwen3_5_moe_text",
                                             "minimax_m3_vl_text", "minimax_m3",
                                             "step3p5"),
            qk_norm_full=cfg.get("model_type", "") == "minimax_m2",
            sliding_window=sliding,
            layer_types=layer_types,
            eos_token_ids=[e for e in eos_ids if e is not None],
            bos_token_id=cfg.get("bos_token_id"),
            torch_dtype=cfg.get("torch_dtype", "bfloat16"),
            # MoE
            num_experts=cfg.get("n_routed_experts") or cfg.get("num_experts")
            or cfg.get("num_local_experts") or 0,
            num_experts_per_tok=cfg.get("num_experts_per_tok")
            or cfg.get("experts_per_token") or 0,
            moe_intermediate_size=cfg.get("moe_intermediate_size", 0),
            num_shared_experts=cfg.get("n_shared_experts", 0),
            shared_expert_intermediate_size=cfg.get("shared_expert_intermediate_size", 0),
            first_k_dense_layers=cfg.get("first_k_dense_replace", 0),
            moe_layer_freq=cfg.get("moe_layer_freq", 1) if not isinstance(
                cfg.get("moe_layer_freq"), list) else 1,
            norm_topk_prob=cfg.get("norm_topk_prob", True),
            routed_scaling_factor=cfg.get("routed_scaling_factor", 1.0),
            scoring_func=cfg.get("scoring_func")
            or ("sigmoid" if cfg.get("model_type") in ("deepseek_v3", "deepseek_v32",
                                                       "kimi_k2", "glm4_moe",
                                                       "glm4v_moe", "minimax_m2",
                                                       "minimax_m3_vl_text",
                                                       "minimax_m3")
                else "softmax"),
            topk_group=cfg.get("topk_group", 0),
            n_group=cfg.get("n_group", 0),
            # MLA
            rope_interleave=cfg.get(
                "rope_interleave",
                cfg.get("model_type", "") in (
                    "deepseek_v2", "deepseek_v3", "deepseek_v32", "kimi_k2"),
            ),
            q_lora_rank=cfg.get("q_lora_rank") or 0,
            kv_lora_rank=cfg.get("kv_lora_rank") or 0,
            qk_nope_head_dim=cfg.get("qk_nope_head_dim") or 0,
            qk_rope_head_dim=cfg.get("qk_rope_head_dim") or 0,
            v_head_dim=cfg.get("v_head_dim") or 0,
            # DSA / MSA indexer
            index_n_heads=cfg.get("index_n_heads") or 0,
            index_head_dim=cfg.get("index_head_dim") or 0,
            index_topk=cfg.get("index_topk") or 0,
            index_block_size=cfg.get("index_block_size") or 0,
            index_topk_blocks=cfg.get("index_topk_blocks") or 0,
            index_local_blocks=cfg.get("index_local_blocks")
            if cfg.get("index_local_blocks") is not None else 0,
            # hybrid linear attention
            linear_num_key_heads=cfg.get("linear_num_key_heads") or (
                num_heads if cfg.get("model_type") in ("minimax", "minimax_m1")
                else 0),
            linear_num_value_heads=cfg.get("linear_num_value_heads") or (
                num_heads if cfg.get("model_type") in ("minimax", "minimax_m1")
                else 0),
            linear_key_head_dim=cfg.get("linear_key_head_dim") or (
                head_dim if cfg.get("model_type") in ("minimax", "minimax_m1")
                else 0),
            linear_value_head_dim=cfg.get("linear_value_head_dim") or (
                head_dim if cfg.get("model_type") in ("minimax", "minimax_m1")
                else 0),
            linear_conv_kernel_dim=cfg.get("linear_conv_kernel_dim") or (
                1 if cfg.get("model_type") in ("minimax", "minimax_m1") else 4),
            raw=cfg,
        )
        return mc

    @classmethod
    def from_pretrained(cls, model_path: str) -> "ModelConfig":
        with open(os.path.join(model_path, "config.json")) as f:
            return cls.from_hf_config(json.load(f))

    # -- sizing helpers used by the scheduling brain (scheduling/model_info.py) ---

    def dtype_bytes(self) -> int:
        return {"bfloat16": 2, "float16": 2, "float32": 4, "float8": 1}.get(
            self.torch_dtype, 2
        )

    def embedding_bytes(self) -> int:
        return self.vocab_size * self.hidden_size * self.dtype_bytes()

    def lm_head_bytes(self) -> int:
        return 0 if self.tie_word_embeddings else self.embedding_bytes()

    def per_layer_param_bytes(self, layer_idx: int = -1) -> int:
        h, d = self.hidden_size, self.dtype_bytes()
        if self.is_mla:
            attn = (
                (self.q_lora_rank or h) * h
                + self.num_heads * (self.qk_nope_head_dim + self.qk_rope_head_dim)
                * (self.q_lora_rank or h)
                + h * (self.kv_lora_rank + self.qk_rope_head_dim)
                + self.num_heads * (self.qk_nope_head_dim + self.v_head_dim)
                * self.kv_lora_rank
                + self.num_heads * self.v_head_dim * h
            )
        else:
            attn = (
                h * self.num_heads * self.head_dim
                + 2 * h * self.num_kv_heads * self.head_dim
                + self.num_heads * self.head_dim * h
            )
        if self.is_moe and (layer_idx < 0 or self.is_moe_layer(layer_idx)):
            inter = self.moe_intermediate_size or self.intermediate_size
            mlp = 3 * h * inter * self.num_experts
            if self.num_shared_experts:
                mlp += 3 * h * inter * self.num_shared_experts
            if self.shared_expert_intermediate_size:
                mlp += 3 * h * self.shared_expert_intermediate_size
        else:
            mlp = 3 * h * self.intermediate_size
        return int((attn + mlp) * d)
