"""Llama 4 text configuration.

Every option that a Llama 4 ``config.json`` carries for the text decoder is a
field here.  The reference reads the sizes from GGUF metadata
(reference: src/SharpInference.Core/ModelGraph.cs:330-340, 492-514) and hard-codes the
Llama 4 switches (NoPE every 4th layer, sigmoid gating, L2 QK norm;
ModelGraph.cs:292-301); here each switch is a key with that behaviour as default.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional, Tuple

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

# Every key of the text decoder's config.json falls in one of three classes: read into a field
# (_READ), known to leave the forward pass of an inference engine as it is (_INERT: training
# options, bookkeeping of the tool that wrote the file, hints for other runtimes), or checked
# against what the fields read elsewhere imply (layer_types).
# A key outside the three whose value is a number, a list or an object may change the
# computation: it is refused.  Text and null values of unknown keys are kept in ``unread_keys``.
_READ = frozenset({
    "hidden_size", "num_hidden_layers", "num_attention_heads", "num_key_value_heads", "head_dim", "vocab_size",
    "intermediate_size", "intermediate_size_mlp", "num_local_experts", "num_experts_per_tok",
    "interleave_moe_layer_step", "moe_layers", "no_rope_layers", "no_rope_layer_interval", "attention_chunk_size",
    "use_qk_norm", "attn_temperature_tuning", "floor_scale", "attn_scale", "rms_norm_eps", "rope_theta",
    "rope_scaling", "rope_parameters", "tie_word_embeddings", "max_position_embeddings", "torch_dtype", "dtype",
    "eos_token_id", "bos_token_id", "architectures", "hidden_act", "attention_bias", "layer_types",
})
_INERT = frozenset({
    "model_type", "attention_dropout", "initializer_range", "output_router_logits", "router_aux_loss_coef",
    "router_jitter_noise", "use_cache", "pad_token_id", "transformers_version", "for_llm_compressor",
    "cache_implementation", "output_attentions", "output_hidden_states", "return_dict", "is_decoder",
    "is_encoder_decoder", "add_cross_attention", "tie_encoder_decoder", "chunk_size_feed_forward",
    "id2label", "label2id", "problem_type", "finetuning_task", "tokenizer_class", "prefix", "sep_token_id",
    "decoder_start_token_id", "task_specific_params", "pruned_heads", "torchscript", "_name_or_path",
    "_attn_implementation", "attn_implementation", "_attn_implementation_autoset", "quantization_config",
})
_LAYER_KIND_OF_ROPE = {True: "chunked_attention", False: "full_attention"}
# config.json's names of the gated unit's activation -> the names the feed-forward parts take
_ACTIVATIONS = {"silu": "silu", "swish": "silu", "gelu_pytorch_tanh": "gelu_tanh", "gelu_tanh": "gelu_tanh"}


def _number(src: Dict[str, Any], key: str, kind, default=None):
    """src[key] as int or float; ConfigError (naming the key) for null, text, lists."""
    v = src.get(key, default) if default is not None else src.get(key)
    if v is None and key not in src and default is None:
        return None
    if isinstance(v, bool) or not isinstance(v, (int, float)):
        raise ConfigError(f"{key} must be a number (got {v!r})")
    if kind is int and int(v) != v:
        raise ConfigError(f"{key} must be a whole number (got {v!r})")
    return kind(v)


def _rope_from(src: Dict[str, Any]):
    """(theta, scaling) from the two forms a file may carry: ``rope_theta`` + ``rope_scaling``,
    or one ``rope_parameters`` object holding the base and the scaling fields together.  Both
    present must agree."""
    theta = _number(src, "rope_theta", float)
    scaling = src.get("rope_scaling")
    if scaling is not None and not isinstance(scaling, dict):
        raise ConfigError(f"rope_scaling must be an object or null (got {scaling!r})")
    rp = src.get("rope_parameters")
    if rp is not None:
        if not isinstance(rp, dict):
            raise ConfigError(f"rope_parameters must be an object (got {rp!r})")
        known = {"rope_theta", "rope_type", "type", "factor", "low_freq_factor", "high_freq_factor",
                 "original_max_position_embeddings"}
        extra = sorted(set(rp) - known)
        if extra:
            raise ConfigError("rope_parameters holds key(s) that are not understood: " + ", ".join(extra))
        p_theta = _number(rp, "rope_theta", float)
        if p_theta is not None:
            if theta is not None and theta != p_theta:
                raise ConfigError(f"rope_theta {theta} contradicts rope_parameters.rope_theta {p_theta}")
            theta = p_theta
        p_scaling = {k: v for k, v in rp.items() if k != "rope_theta"}
        kind = p_scaling.get("rope_type", p_scaling.get("type", "default"))
        if kind in (None, "default"):
            leftover = sorted(k for k in p_scaling if k not in ("rope_type", "type"))
            if leftover:
                raise ConfigError("rope_parameters has rope_type 'default' but carries scaling key(s): " + ", ".join(leftover))
            p_scaling = None
        if p_scaling is not None:
            if scaling and RopeScaling.from_dict(scaling) != RopeScaling.from_dict(p_scaling):
                raise ConfigError("rope_scaling contradicts rope_parameters")
            scaling = p_scaling
    if scaling and scaling.get("rope_type", scaling.get("type")) in (None, "default") and \
            not (set(scaling) - {"rope_type", "type"}):
        scaling = None
    return (500000.0 if theta is None else theta), (RopeScaling.from_dict(scaling) if scaling else None)


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
    hidden_act: str = "silu"              # the gated unit's activation, as config.json names it
    attention_bias: bool = False          # q, k, v and o projections carry biases
    # head
    tie_word_embeddings: bool = False
    max_position_embeddings: int = 0
    torch_dtype: str = "bfloat16"
    # keys of the file that were neither read nor known to be without effect (text or null values)
    unread_keys: Tuple[str, ...] = field(default=(), compare=False)

    # ------------------------------------------------------------------
    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "Llama4TextConfig":
        # Multimodal checkpoints nest the decoder's keys under text_config; beside it, only the
        # keys that name the model, its tokens and the tied head count at the top level.
        nested = d.get("text_config")
        if nested is not None and not isinstance(nested, dict):
            raise ConfigError("text_config must be an object")
        if nested is not None:
            src = dict(nested)
            for k in ("architectures", "tie_word_embeddings", "eos_token_id", "bos_token_id", "torch_dtype", "dtype"):
                if k in d and k not in src:
                    src[k] = d[k]
        else:
            src = dict(d)
        missing = [k for k in _REQUIRED if k not in src]
        if missing:
            raise ConfigError("config.json lacks required key(s): " + ", ".join(missing))
        unknown = sorted(k for k in src if k not in _READ and k not in _INERT)
        refused = [k for k in unknown if isinstance(src[k], (bool, int, float, list, dict))]
        if refused:
            raise ConfigError("config.json holds key(s) that this reader does not understand and that may change "
                              "the computation: " + ", ".join(f"{k}={src[k]!r}" for k in refused))
        act = src.get("hidden_act", "silu")
        if act not in _ACTIVATIONS:
            raise ConfigError(f"hidden_act {act!r} is not supported: the feed-forward kernels apply "
                              + ", ".join(sorted(_ACTIVATIONS)))
        bias = src.get("attention_bias", False)
        if not isinstance(bias, bool):
            raise ConfigError(f"attention_bias must be true or false (got {bias!r})")
        nh = _number(src, "num_attention_heads", int)
        hidden = _number(src, "hidden_size", int)
        layers = _number(src, "num_hidden_layers", int)
        if layers <= 0:
            raise ConfigError(f"num_hidden_layers must be positive (got {layers})")
        moe_layers = src.get("moe_layers")
        if moe_layers is not None and not isinstance(moe_layers, list):
            raise ConfigError(f"moe_layers must be a list of layer numbers (got {moe_layers!r})")
        nrl = src.get("no_rope_layers") or []
        if not isinstance(nrl, list):
            raise ConfigError(f"no_rope_layers must be a list with one entry per layer (got {nrl!r})")
        if not nrl:
            # the reference's fixed rule (ModelGraph.cs:292-295): every 4th layer has no rotary;
            # the interval is a key of its own in files that give no list
            interval = _number(src, "no_rope_layer_interval", int, 4)
            if interval <= 0:
                raise ConfigError(f"no_rope_layer_interval must be positive (got {interval})")
            nrl = [0 if (l + 1) % interval == 0 else 1 for l in range(layers)]
        kinds = src.get("layer_types")
        if kinds is not None:
            # the window of a layer goes with its position encoding here (rotary layers see their
            # chunk, the others every key): a file that says otherwise is not this architecture
            want = [_LAYER_KIND_OF_ROPE[bool(x)] for x in nrl]
            if list(kinds) != want:
                raise ConfigError(f"layer_types {kinds!r} contradicts no_rope_layers {nrl!r}: rotary layers are "
                                  "'chunked_attention', the others 'full_attention'")
        chunk = src.get("attention_chunk_size", 8192)
        if isinstance(chunk, bool) or not isinstance(chunk, int):
            raise ConfigError(f"attention_chunk_size must be a positive whole number (got {chunk!r})")
        theta, scaling = _rope_from(src)
        archs = d.get("architectures") or ["Llama4ForCausalLM"]
        return cls(
            architecture=str(archs[0]),
            hidden_size=hidden,
            num_hidden_layers=layers,
            num_attention_heads=nh,
            num_key_value_heads=_number(src, "num_key_value_heads", int, nh),
            head_dim=int(src.get("head_dim") or (hidden // max(nh, 1))),
            vocab_size=_number(src, "vocab_size", int),
            intermediate_size=_number(src, "intermediate_size", int),
            intermediate_size_mlp=_number(src, "intermediate_size_mlp", int) or 0,
            num_local_experts=_number(src, "num_local_experts", int),
            num_experts_per_tok=_number(src, "num_experts_per_tok", int, 1),
            interleave_moe_layer_step=_number(src, "interleave_moe_layer_step", int, 1),
            moe_layers=[int(x) for x in moe_layers] if moe_layers is not None else None,
            no_rope_layers=[int(x) for x in nrl],
            attention_chunk_size=chunk,
            use_qk_norm=bool(src.get("use_qk_norm", True)),
            attn_temperature_tuning=bool(src.get("attn_temperature_tuning", True)),
            floor_scale=_number(src, "floor_scale", float, 8192.0),
            attn_scale=_number(src, "attn_scale", float, 0.1),
            rms_norm_eps=_number(src, "rms_norm_eps", float, 1e-5),
            rope_theta=theta,
            rope_scaling=scaling,
            hidden_act=str(act),
            attention_bias=bias,
            tie_word_embeddings=bool(src.get("tie_word_embeddings", False)),
            max_position_embeddings=_number(src, "max_position_embeddings", int) or 0,
            torch_dtype=str(src.get("torch_dtype") or src.get("dtype") or "bfloat16"),
            unread_keys=tuple(k for k in unknown if k not in refused),
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
            "hidden_act": self.hidden_act,
            "attention_bias": self.attention_bias,
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
        need(self.hidden_act in _ACTIVATIONS, f"hidden_act {self.hidden_act!r} is not known ({', '.join(sorted(_ACTIVATIONS))})")
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

    @property
    def activation(self) -> str:
        """The gated unit's activation under the name the feed-forward parts take."""
        return _ACTIVATIONS[self.hidden_act]

    def uses_rope(self, layer: int) -> bool:
        return self.no_rope_layers[layer] != 0
