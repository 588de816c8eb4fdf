"""Llama 4 text configuration.

Every option that a Llama 4 ``config.json`` carries for the text decoder is a
field here.  The reference reads the sizes from GGUF metadata
(reference: src/SharpInference.Core/ModelGraph.cs:330-340, 492-514) and hard-codes the
Llama 4 switches (NoPE every 4th layer, sigmoid gating, L2 QK norm;
ModelGraph.cs:292-301); here each switch is a key with that behaviour as default.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional

from .base import ConfigError, ModelConfig, special_tokens_from


@dataclass
class RopeScaling:
    """llama3-style frequency scaling of the rotary table."""

    rope_type: str = "llama3"
    factor: float = 1.0
    low_freq_factor: float = 1.0
    high_freq_factor: float = 4.0
    original_max_position_embeddings: int = 8192

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "RopeScaling":
        kind = d.get("rope_type", d.get("type"))
        if kind != "llama3":
            raise ConfigError(f"rope_scaling.rope_type {kind!r} is not supported (known: 'llama3')")
        try:
            return cls(
                rope_type="llama3",
                factor=float(d["factor"]),
                low_freq_factor=float(d.get("low_freq_factor", 1.0)),
                high_freq_factor=float(d.get("high_freq_factor", 4.0)),
                original_max_position_embeddings=int(d["original_max_position_embeddings"]),
            )
        except KeyError as e:
            raise ConfigError(f"rope_scaling lacks key {e.args[0]!r}") from None

    def to_dict(self) -> Dict[str, Any]:
        return {
            "rope_type": self.rope_type,
            "factor": self.factor,
            "low_freq_factor": self.low_freq_factor,
            "high_freq_factor": self.high_freq_factor,
            "original_max_position_embeddings": self.original_max_position_embeddings,
        }


_REQUIRED = (
    "hidden_size",
    "num_hidden_layers",
    "num_attention_heads",
    "vocab_size",
    "intermediate_size",
    "num_local_experts",
)


@dataclass
class Llama4TextConfig(ModelConfig):
    architecture: str = "Llama4ForCausalLM"
    hidden_size: int = 0
    num_hidden_layers: int = 0
    num_attention_heads: int = 0
    num_key_value_heads: int = 0
    head_dim: int = 0
    vocab_size: int = 0
    # feed-forward
    intermediate_size: int = 0            # width of each routed expert and of the shared expert
    intermediate_size_mlp: int = 0        # width of the dense feed-forward on non-MoE layers
    num_local_experts: int = 0
    num_experts_per_tok: int = 1
    interleave_moe_layer_step: int = 1    # layer L is MoE iff (L+1) % step == 0
    moe_layers: Optional[List[int]] = None  # explicit list overrides the step rule
    # attention
    no_rope_layers: List[int] = field(default_factory=list)  # per layer: non-zero = rotary, 0 = no position encoding
    attention_chunk_size: int = 8192
    use_qk_norm: bool = True
    attn_temperature_tuning: bool = True
    floor_scale: float = 8192.0
    attn_scale: float = 0.1
    # norms / rotary
    rms_norm_eps: float = 1e-5
    rope_theta: float = 500000.0
    rope_scaling: Optional[RopeScaling] = None
    # head
    tie_word_embeddings: bool = False
    max_position_embeddings: int = 0
    torch_dtype: str = "bfloat16"

    # ------------------------------------------------------------------
    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "Llama4TextConfig":
        # Multimodal checkpoints nest the decoder's keys under text_config.
        src = dict(d.get("text_config") or {})
        for k, v in d.items():
            if k != "text_config" and k not in src:
                src[k] = v
        missing = [k for k in _REQUIRED if k not in src]
        if missing:
            raise ConfigError("config.json lacks required key(s): " + ", ".join(missing))
        nh = int(src["num_attention_heads"])
        hidden = int(src["hidden_size"])
        layers = int(src["num_hidden_layers"])
        step = int(src.get("interleave_moe_layer_step", 1))
        moe_layers = src.get("moe_layers")
        scaling = src.get("rope_scaling")
        nrl = src.get("no_rope_layers") or []
        if not nrl:
            # the reference's fixed rule (ModelGraph.cs:292-295): every 4th layer has no rotary
            nrl = [0 if (l + 1) % 4 == 0 else 1 for l in range(layers)]
        archs = d.get("architectures") or ["Llama4ForCausalLM"]
        return cls(
            architecture=str(archs[0]),
            hidden_size=hidden,
            num_hidden_layers=layers,
            num_attention_heads=nh,
            num_key_value_heads=int(src.get("num_key_value_heads", nh)),
            head_dim=int(src.get("head_dim") or (hidden // max(nh, 1))),
            vocab_size=int(src["vocab_size"]),
            intermediate_size=int(src["intermediate_size"]),
            intermediate_size_mlp=int(src.get("intermediate_size_mlp", 0)),
            num_local_experts=int(src["num_local_experts"]),
            num_experts_per_tok=int(src.get("num_experts_per_tok", 1)),
            interleave_moe_layer_step=step,
            moe_layers=[int(x) for x in moe_layers] if moe_layers is not None else None,
            no_rope_layers=[int(x) for x in nrl],
            attention_chunk_size=int(src.get("attention_chunk_size", 8192)),
            use_qk_norm=bool(src.get("use_qk_norm", True)),
            attn_temperature_tuning=bool(src.get("attn_temperature_tuning", True)),
            floor_scale=float(src.get("floor_scale", 8192)),
            attn_scale=float(src.get("attn_scale", 0.1)),
            rms_norm_eps=float(src.get("rms_norm_eps", 1e-5)),
            rope_theta=float(src.get("rope_theta", 500000.0)),
            rope_scaling=RopeScaling.from_dict(scaling) if scaling else None,
            tie_word_embeddings=bool(src.get("tie_word_embeddings", False)),
            max_position_embeddings=int(src.get("max_position_embeddings", 0)),
            torch_dtype=str(src.get("torch_dtype", "bfloat16")),
            **special_tokens_from(src),
        )

    def to_dict(self) -> Dict[str, Any]:
        out: Dict[str, Any] = {
            "architectures": [self.architecture],
            "model_type": "llama4_text",
            "hidden_size": self.hidden_size,
            "num_hidden_layers": self.num_hidden_layers,
            "num_attention_heads": self.num_attention_heads,
            "num_key_value_heads": self.num_key_value_heads,
            "head_dim": self.head_dim,
            "vocab_size": self.vocab_size,
            "intermediate_size": self.intermediate_size,
            "intermediate_size_mlp": self.intermediate_size_mlp,
            "num_local_experts": self.num_local_experts,
            "num_experts_per_tok": self.num_experts_per_tok,
            "interleave_moe_layer_step": self.interleave_moe_layer_step,
            "no_rope_layers": list(self.no_rope_layers),
            "attention_chunk_size": self.attention_chunk_size,
            "use_qk_norm": self.use_qk_norm,
            "attn_temperature_tuning": self.attn_temperature_tuning,
            "floor_scale": self.floor_scale,
            "attn_scale": self.attn_scale,
            "rms_norm_eps": self.rms_norm_eps,
            "rope_theta": self.rope_theta,
            "rope_scaling": self.rope_scaling.to_dict() if self.rope_scaling else None,
            "tie_word_embeddings": self.tie_word_embeddings,
            "max_position_embeddings": self.max_position_embeddings,
            "torch_dtype": self.torch_dtype,
        }
        if self.moe_layers is not None:
            out["moe_layers"] = list(self.moe_layers)
        out.update(self.special_tokens_dict())
        return out

    # ------------------------------------------------------------------
    def validate(self) -> None:
        def need(cond: bool, msg: str) -> None:
            if not cond:
                raise ConfigError(msg)

        for k in ("hidden_size", "num_hidden_layers", "num_attention_heads", "num_key_value_heads",
                  "head_dim", "vocab_size"):
            need(getattr(self, k) > 0, f"{k} must be positive (got {getattr(self, k)})")
        need(self.num_attention_heads % self.num_key_value_heads == 0,
             f"num_attention_heads {self.num_attention_heads} is not a multiple of "
             f"num_key_value_heads {self.num_key_value_heads}")
        need(self.head_dim % 2 == 0, f"head_dim {self.head_dim} must be even (rotary pairs)")
        need(len(self.no_rope_layers) == self.num_hidden_layers,
             f"no_rope_layers has {len(self.no_rope_layers)} entries for {self.num_hidden_layers} layers")
        need(self.attention_chunk_size > 0, f"attention_chunk_size must be positive (got {self.attention_chunk_size})")
        need(self.interleave_moe_layer_step >= 0, "interleave_moe_layer_step must not be negative")
        need(self.rms_norm_eps > 0, "rms_norm_eps must be positive")
        need(self.rope_theta > 0, "rope_theta must be positive")
        need(self.floor_scale > 0, "floor_scale must be positive")
        if self.moe_layers is not None:
            bad = [l for l in self.moe_layers if not 0 <= l < self.num_hidden_layers]
            need(not bad, f"moe_layers names layers out of range: {bad}")
        any_moe = any(self.is_moe_layer(l) for l in range(self.num_hidden_layers))
        any_dense = any(not self.is_moe_layer(l) for l in range(self.num_hidden_layers))
        if any_moe:
            need(self.num_local_experts > 0, "num_local_experts must be positive on a model with MoE layers")
            need(self.intermediate_size > 0, "intermediate_size must be positive on a model with MoE layers")
            need(1 <= self.num_experts_per_tok <= self.num_local_experts,
                 f"num_experts_per_tok {self.num_experts_per_tok} must lie in 1..num_local_experts "
                 f"{self.num_local_experts}")
        if any_dense:
            need(self.intermediate_size_mlp > 0,
                 "intermediate_size_mlp must be positive: the model has dense feed-forward layers")
        if self.rope_scaling is not None:
            rs = self.rope_scaling
            need(rs.factor >= 1.0, "rope_scaling.factor must be >= 1")
            need(rs.high_freq_factor > rs.low_freq_factor,
                 "rope_scaling.high_freq_factor must exceed low_freq_factor")
            need(rs.original_max_position_embeddings > 0,
                 "rope_scaling.original_max_position_embeddings must be positive")

    # ------------------------------------------------------------------
    def is_moe_layer(self, layer: int) -> bool:
        if self.moe_layers is not None:
            return layer in self.moe_layers
        step = self.interleave_moe_layer_step
        return step > 0 and (layer + 1) % step == 0

    def uses_rope(self, layer: int) -> bool:
        return self.no_rope_layers[layer] != 0
