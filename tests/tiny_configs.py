"""Two tiny Llama 4 configurations that differ in every size and option, as raw config.json dicts."""

TINY_A = {
    "architectures": ["Llama4ForCausalLM"],
    "hidden_size": 64, "num_hidden_layers": 2, "num_attention_heads": 4, "num_key_value_heads": 2,
    "head_dim": 16, "vocab_size": 256,
    "intermediate_size": 128, "intermediate_size_mlp": 256,
    "num_local_experts": 4, "num_experts_per_tok": 1, "interleave_moe_layer_step": 1,
    "no_rope_layers": [1, 0], "attention_chunk_size": 16,
    "use_qk_norm": True, "attn_temperature_tuning": True, "floor_scale": 8, "attn_scale": 0.1,
    "rms_norm_eps": 1e-5, "rope_theta": 10000.0, "rope_scaling": None,
    "tie_word_embeddings": False, "max_position_embeddings": 512, "torch_dtype": "bfloat16",
}

TINY_B = {
    "architectures": ["Llama4ForCausalLM"],
    "hidden_size": 96, "num_hidden_layers": 5, "num_attention_heads": 6, "num_key_value_heads": 3,
    "head_dim": 32, "vocab_size": 384,
    "intermediate_size": 64, "intermediate_size_mlp": 160,
    "num_local_experts": 8, "num_experts_per_tok": 2, "interleave_moe_layer_step": 2,
    "no_rope_layers": [1, 1, 1, 0, 1], "attention_chunk_size": 24,
    "use_qk_norm": False, "attn_temperature_tuning": True, "floor_scale": 32, "attn_scale": 0.2,
    "rms_norm_eps": 1e-6, "rope_theta": 500000.0,
    "rope_scaling": {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                     "original_max_position_embeddings": 32},
    "tie_word_embeddings": False, "max_position_embeddings": 1024, "torch_dtype": "bfloat16",
}

# a third one: tied head, one kv head per head, odd-ish sizes, every layer dense but one
TINY_C = {
    "architectures": ["Llama4ForCausalLM"],
    "hidden_size": 80, "num_hidden_layers": 3, "num_attention_heads": 5, "num_key_value_heads": 5,
    "head_dim": 48, "vocab_size": 203,
    "intermediate_size": 48, "intermediate_size_mlp": 112,
    "num_local_experts": 3, "num_experts_per_tok": 3, "interleave_moe_layer_step": 3,
    "no_rope_layers": [0, 1, 1], "attention_chunk_size": 40,
    "use_qk_norm": True, "attn_temperature_tuning": False, "floor_scale": 4, "attn_scale": 0.5,
    "rms_norm_eps": 1e-4, "rope_theta": 1000.0, "rope_scaling": None,
    "tie_word_embeddings": True, "max_position_embeddings": 512, "torch_dtype": "bfloat16",
}

# a fourth one whose widths are multiples of 128 and whose head size is 64: the sizes at which the
# matrix-core kernels (few-row and grouped products, flash attention) take over from the generic ones
TINY_D = {
    "architectures": ["Llama4ForCausalLM"],
    "hidden_size": 256, "num_hidden_layers": 3, "num_attention_heads": 6, "num_key_value_heads": 2,
    "head_dim": 64, "vocab_size": 500,
    "intermediate_size": 128, "intermediate_size_mlp": 384,
    "num_local_experts": 6, "num_experts_per_tok": 1, "interleave_moe_layer_step": 1,
    "no_rope_layers": [1, 0, 1], "attention_chunk_size": 48,
    "use_qk_norm": True, "attn_temperature_tuning": True, "floor_scale": 16, "attn_scale": 0.15,
    "rms_norm_eps": 1e-5, "rope_theta": 500000.0,
    "rope_scaling": {"rope_type": "llama3", "factor": 4.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                     "original_max_position_embeddings": 64},
    "tie_word_embeddings": False, "max_position_embeddings": 1024, "torch_dtype": "bfloat16",
}

SEEDS = {"A": 0, "B": 1, "C": 5, "D": 9}
CONFIGS = {"A": TINY_A, "B": TINY_B, "C": TINY_C, "D": TINY_D}
# tensors kept in float32 in B's file: shows that 32-bit tensors stay 32-bit in a bfloat16 run
FLOAT32_NAMES = {"A": (), "B": ("layernorm.weight", "model.norm.weight", "router.weight"), "C": (), "D": ()}


def as_other_tools_write_it(d):
    """The same model in the other form a Llama 4 config.json is found in: the text keys nested,
    the rotary base and scaling in one ``rope_parameters`` object, the window of every layer
    named in ``layer_types``, and the training / bookkeeping keys such files carry."""
    text = {k: v for k, v in d.items() if k not in ("architectures", "rope_theta", "rope_scaling", "tie_word_embeddings")}
    rp = {"rope_theta": d["rope_theta"], "rope_type": "default"}
    if d.get("rope_scaling"):
        rp = {"rope_theta": d["rope_theta"], **d["rope_scaling"]}
    text.update({
        "rope_parameters": rp, "model_type": "llama4_text", "hidden_act": "silu", "attention_bias": False,
        "attention_dropout": 0.0, "initializer_range": 0.02, "output_router_logits": False,
        "router_aux_loss_coef": 0.001, "router_jitter_noise": 0.0, "use_cache": True, "pad_token_id": 0,
        "layer_types": ["chunked_attention" if r else "full_attention" for r in d["no_rope_layers"]],
        "no_rope_layer_interval": 4, "for_llm_compressor": False, "cache_implementation": "hybrid",
    })
    return {"architectures": ["Llama4ForConditionalGeneration"], "model_type": "llama4", "text_config": text,
            "tie_word_embeddings": d["tie_word_embeddings"], "transformers_version": "5.0.0",
            "vision_config": {"hidden_size": 32}, "image_token_index": 7, "boi_token_index": 8, "eoi_token_index": 9}


def make_model_dir(tmp_path, which: str, std: float = 0.02, **overrides) -> str:
    from sharpinference_amd.config.base import load_config
    from sharpinference_amd.weights.loader import write_random_model

    d = dict(CONFIGS[which])
    d.update(overrides)
    cfg = load_config(d)
    out = str(tmp_path / f"tiny_{which}")
    write_random_model(cfg, out, SEEDS[which], std=std, float32_names=FLOAT32_NAMES[which])
    return out


def write_other_layout(src_dir, out_dir, prefix, extra=()):
    """The tensors of a model folder under a container prefix, the experts' gate and up fused as
    [E, in, 2 * out] and their down stored [E, in, out]; `extra` tensors are added as they are."""
    import os

    import torch

    from sharpinference_amd.weights import safetensors_io as st

    entries = st.index_folder(src_dir)
    tensors = {n: st.read_tensor(e) for n, e in entries.items()}
    out = {}
    for n, t in tensors.items():
        if n.endswith("experts.gate_proj"):
            up = tensors[n[:-len("gate_proj")] + "up_proj"]
            out[prefix + n[:-len("gate_proj")] + "gate_up_proj"] = torch.cat([t, up], 1).transpose(1, 2).contiguous()
        elif n.endswith("experts.up_proj"):
            continue
        elif n.endswith("experts.down_proj"):
            out[prefix + n] = t.transpose(1, 2).contiguous()
        else:
            out[prefix + n] = t
    out.update(extra)
    os.makedirs(out_dir, exist_ok=True)
    with open(os.path.join(src_dir, "config.json")) as f, open(os.path.join(out_dir, "config.json"), "w") as g:
        g.write(f.read())
    st.write_file(os.path.join(out_dir, "model.safetensors"), sorted(out.items()))
    return out_dir
