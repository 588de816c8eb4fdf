"""Configuration, registry and weight loading (no GPU)."""
import json
import os

import pytest
import torch

from sharpinference_amd import ConfigError, build_model, load_config, registered_architectures
from sharpinference_amd.config.llama4 import Llama4TextConfig
from sharpinference_amd.weights import safetensors_io as st
from sharpinference_amd.weights.loader import (RandomSource, SafetensorsSource, WeightError, check_specs,
                                               load_model_weights, storage_dtype, write_random_model)
from tiny_configs import CONFIGS, TINY_A, TINY_B, as_other_tools_write_it, make_model_dir, write_other_layout


def test_every_key_is_read_and_round_trips():
    for d in CONFIGS.values():
        cfg = load_config(d)
        again = load_config(cfg.to_dict())
        assert again == cfg
    b = load_config(TINY_B)
    assert (b.hidden_size, b.num_hidden_layers, b.num_attention_heads, b.num_key_value_heads, b.head_dim) == (96, 5, 6, 3, 32)
    assert b.rope_scaling.factor == 8.0 and b.rope_scaling.original_max_position_embeddings == 32
    assert [b.is_moe_layer(l) for l in range(5)] == [False, True, False, True, False]
    assert [b.uses_rope(l) for l in range(5)] == [True, True, True, False, True]
    assert not b.use_qk_norm and b.floor_scale == 32 and b.attn_scale == 0.2 and b.rms_norm_eps == 1e-6


def test_defaults_follow_the_reference_rule():
    d = {k: v for k, v in TINY_A.items() if k not in ("no_rope_layers", "head_dim", "num_key_value_heads")}
    d["num_hidden_layers"] = 8
    cfg = load_config(d)
    assert cfg.no_rope_layers == [1, 1, 1, 0, 1, 1, 1, 0]          # every 4th layer has no rotary
    assert cfg.head_dim == 16 and cfg.num_key_value_heads == 4


def test_nested_text_config():
    d = {"architectures": ["Llama4ForCausalLM"], "text_config": {k: v for k, v in TINY_A.items() if k != "architectures"}}
    assert load_config(d).hidden_size == 64


@pytest.mark.parametrize("change,word", [
    ({"num_key_value_heads": 3}, "multiple"), ({"head_dim": 15}, "even"), ({"num_experts_per_tok": 9}, "num_experts_per_tok"),
    ({"no_rope_layers": [1]}, "no_rope_layers"), ({"attention_chunk_size": 0}, "attention_chunk_size"),
    ({"rope_scaling": {"rope_type": "yarn", "factor": 2}}, "rope_type"), ({"rms_norm_eps": 0}, "rms_norm_eps"),
    ({"interleave_moe_layer_step": 2, "intermediate_size_mlp": 0}, "intermediate_size_mlp"),
])
def test_contradictions_are_refused(change, word):
    with pytest.raises(ConfigError, match=word):
        load_config({**TINY_A, **change})


def test_the_other_form_of_the_same_config_reads_the_same():
    """rope_parameters instead of rope_theta + rope_scaling: the base and the llama3 fields must
    arrive (a reader that only knows the old names would fall back to 500000 and no scaling)."""
    for d in CONFIGS.values():
        a, b = load_config(d), load_config(as_other_tools_write_it(d))
        assert (a.rope_theta, a.rope_scaling) == (b.rope_theta, b.rope_scaling)
        for f in ("hidden_size", "no_rope_layers", "attention_chunk_size", "floor_scale", "attn_scale", "rms_norm_eps",
                  "intermediate_size_mlp", "num_experts_per_tok", "tie_word_embeddings", "use_qk_norm"):
            assert getattr(a, f) == getattr(b, f), f
        assert [a.is_moe_layer(l) for l in range(a.num_hidden_layers)] == [b.is_moe_layer(l) for l in range(b.num_hidden_layers)]
        assert b.unread_keys == ()
    a = load_config(TINY_A)
    assert a.rope_theta == 10000.0 and a.rope_scaling is None
    b = load_config(as_other_tools_write_it(TINY_B))
    assert b.rope_theta == 500000.0 and b.rope_scaling.factor == 8.0 and b.rope_scaling.original_max_position_embeddings == 32
    assert build_model(b).blocks[0].mixer.rotary.scaling == b.rope_scaling


def test_no_rope_layer_interval_fills_the_list():
    d = {k: v for k, v in TINY_A.items() if k != "no_rope_layers"}
    d.update(num_hidden_layers=6, no_rope_layer_interval=3)
    assert load_config(d).no_rope_layers == [1, 1, 0, 1, 1, 0]
    d["no_rope_layers"] = []                 # an empty list is "not given"
    assert load_config(d).no_rope_layers == [1, 1, 0, 1, 1, 0]


@pytest.mark.parametrize("change,word", [
    ({"hidden_act": "gelu"}, "hidden_act"), ({"hidden_act": "relu"}, "hidden_act"), ({"attention_bias": "yes"}, "attention_bias"),
    ({"layer_types": ["full_attention", "full_attention"]}, "layer_types"),
    ({"attention_chunk_size": None}, "attention_chunk_size"), ({"attention_chunk_size": "8192"}, "attention_chunk_size"),
    ({"rope_parameters": {"rope_theta": 5.0}}, "contradicts"),
    ({"rope_parameters": {"rope_theta": 10000.0, "rope_type": "llama3", "factor": 2.0,
                          "original_max_position_embeddings": 8}, "rope_scaling": {"rope_type": "llama3", "factor": 4.0,
                                                                                   "original_max_position_embeddings": 8}}, "contradicts"),
    ({"rope_parameters": {"rope_theta": 10000.0, "rope_type": "yarn", "factor": 2.0}}, "rope_type"),
    ({"rope_parameters": {"rope_theta": 10000.0, "beta_fast": 32}}, "beta_fast"),
    ({"rope_parameters": {"rope_theta": 10000.0, "rope_type": "default", "factor": 2.0}}, "factor"),
    ({"sliding_window": 128}, "sliding_window"), ({"partial_rotary_factor": 0.5, "logit_cap": 30.0}, "logit_cap.*partial_rotary_factor"),
    ({"rms_norm_eps": None}, "rms_norm_eps"), ({"num_hidden_layers": "3"}, "num_hidden_layers"),
    ({"text_config": 3}, "text_config"),
])
def test_keys_that_would_change_the_computation_are_not_passed_over(change, word):
    with pytest.raises(ConfigError, match=word):
        load_config({**TINY_A, **change})


def test_activation_and_attention_biases_come_from_the_file():
    """hidden_act names the gated unit's activation of every feed-forward (the names config.json uses
    for the two the kernels apply); attention_bias gives the four projections biases, which the
    model then asks the weight file for."""
    from sharpinference_amd import ops

    plain = build_model(load_config(TINY_B))
    assert all(b.ffn.act == ops.ACT_SILU for b in plain.blocks)
    assert not any(n.endswith(".bias") for n in plain.param_specs())
    for name in ("gelu_pytorch_tanh", "gelu_tanh"):
        cfg = load_config({**TINY_B, "hidden_act": name})
        assert cfg.activation == "gelu_tanh" and cfg.to_dict()["hidden_act"] == name
        m = build_model(cfg)
        assert all(b.ffn.act == ops.ACT_GELU_TANH for b in m.blocks)
        assert all(b.ffn.shared.act == ops.ACT_GELU_TANH for b in m.blocks if hasattr(b.ffn, "shared") and b.ffn.shared)
    cfg = load_config({**TINY_B, "attention_bias": True})
    assert load_config(cfg.to_dict()).attention_bias is True
    specs = build_model(cfg).param_specs()
    q, kv = TINY_B["num_attention_heads"] * TINY_B["head_dim"], TINY_B["num_key_value_heads"] * TINY_B["head_dim"]
    for l in range(TINY_B["num_hidden_layers"]):
        p = f"model.layers.{l}.self_attn."
        assert specs[p + "q_proj.bias"].shape == (q,) and specs[p + "k_proj.bias"].shape == (kv,)
        assert specs[p + "v_proj.bias"].shape == (kv,) and specs[p + "o_proj.bias"].shape == (TINY_B["hidden_size"],)


def test_unknown_text_keys_are_listed_not_refused():
    cfg = load_config({**TINY_A, "some_note": "hello", "another": None})
    assert cfg.unread_keys == ("another", "some_note")
    assert load_config({**TINY_A, "rope_scaling": {"rope_type": "default"}}).rope_scaling is None


def test_missing_keys_and_unknown_architecture():
    with pytest.raises(ConfigError, match="hidden_size"):
        load_config({"architectures": ["Llama4ForCausalLM"], "vocab_size": 10})
    with pytest.raises(ConfigError, match="not registered.*Llama4ForCausalLM"):
        load_config({**TINY_A, "architectures": ["NoSuchModel"]})
    assert "Llama4ForCausalLM" in registered_architectures()


def test_model_is_assembled_layer_by_layer():
    m = build_model(load_config(TINY_B))
    kinds = [(type(b.mixer).__name__, b.mixer.rotary is not None, b.mixer.window_kind, type(b.ffn).__name__) for b in m.blocks]
    assert kinds[3] == ("Attention", False, 0, "MoESwiGLU") and kinds[0] == ("Attention", True, 1, "DenseSwiGLU")
    assert m.blocks[0].mixer.window == 24 and m.blocks[3].mixer.q_temperature == (32.0, 0.2)
    assert m.blocks[1].ffn.k == 2 and m.blocks[1].ffn.E == 8 and m.blocks[0].ffn.inter == 160
    specs = m.param_specs()
    assert specs["model.layers.1.feed_forward.experts.down_proj"].shape == (8, 96, 64)
    assert specs["model.layers.0.self_attn.q_proj.weight"].shape == (192, 96)


def test_safetensors_round_trip(tmp_path):
    t = {"a": torch.randn(3, 5).to(torch.bfloat16), "b": torch.arange(7, dtype=torch.int64), "c": torch.randn(2, 2)}
    path = str(tmp_path / "x.safetensors")
    st.write_file(path, t.items(), {"k": "v"})
    from safetensors.torch import load_file

    other = load_file(path)                      # the library reads what we write
    for k in t:
        assert torch.equal(other[k], t[k])
    hdr = st.read_header(path)
    for k in t:
        assert torch.equal(st.read_tensor(hdr[k]), t[k]) and hdr[k].shape == tuple(t[k].shape)
    with open(path, "r+b") as f:                 # a truncated file is noticed
        f.truncate(os.path.getsize(path) - 4)
    with pytest.raises(st.SafetensorsError, match="beyond the end"):
        st.read_header(path)


def test_random_model_folder_and_dtype_policy(tmp_path):
    d = make_model_dir(tmp_path, "B")
    assert sorted(os.listdir(d)) == ["config.json", "model.safetensors"]
    assert json.load(open(os.path.join(d, "config.json")))["hidden_size"] == 96
    src = SafetensorsSource(d, torch.bfloat16, "cpu")
    assert src.get("model.layers.0.self_attn.q_proj.weight").dtype == torch.bfloat16
    assert src.get("model.norm.weight").dtype == torch.float32          # stored in 32-bit: stays so
    assert src.get("model.layers.1.feed_forward.router.weight").dtype == torch.float32
    assert SafetensorsSource(d, torch.float32, "cpu").get("model.layers.0.self_attn.q_proj.weight").dtype == torch.float32
    assert storage_dtype(torch.float16, torch.bfloat16) == torch.bfloat16
    assert storage_dtype(torch.int64, torch.bfloat16) == torch.int32
    again = make_model_dir(tmp_path / "again", "B")                       # same seed, same bytes
    assert open(os.path.join(d, "model.safetensors"), "rb").read() == open(os.path.join(again, "model.safetensors"), "rb").read()
    w = SafetensorsSource(d, torch.float32, "cpu").get("model.layers.0.input_layernorm.weight")
    assert 0.9 <= float(w.min()) and float(w.max()) <= 1.1


def test_one_error_lists_everything(tmp_path):
    d = make_model_dir(tmp_path, "A")
    path = os.path.join(d, "model.safetensors")
    hdr = st.read_header(path)
    tensors = {n: st.read_tensor(e) for n, e in hdr.items()}
    del tensors["model.norm.weight"]
    del tensors["model.layers.1.self_attn.o_proj.weight"]
    tensors["model.layers.0.self_attn.k_proj.weight"] = torch.zeros(7, 64, dtype=torch.bfloat16)
    tensors["extra.tensor"] = torch.zeros(2)
    tensors["model.layers.0.feed_forward.router.weight"] = torch.zeros(4, 64, dtype=torch.int32)
    st.write_file(path, tensors.items())
    model = build_model(load_config(d))
    with pytest.raises(WeightError) as ei:
        load_model_weights(model, SafetensorsSource(d, torch.float32, "cpu"))
    e = ei.value
    assert e.missing == ["model.layers.1.self_attn.o_proj.weight", "model.norm.weight"]
    assert e.unexpected == ["extra.tensor"]
    assert len(e.wrong_shape) == 1 and "expected [32, 64], found [7, 64]" in e.wrong_shape[0]
    assert len(e.wrong_kind) == 1 and "router" in e.wrong_kind[0]
    msg = str(e)
    for word in ("missing (2)", "unexpected (1)", "wrong shape (1)", "wrong kind (1)"):
        assert word in msg


def test_random_source_is_order_independent():
    m = build_model(load_config(TINY_A))
    specs = m.param_specs()
    a = RandomSource(specs, 3, torch.float32, "cpu")
    b = RandomSource(specs, 3, torch.float32, "cpu")
    names = sorted(specs)
    for n in names:
        a.get(n)
    assert torch.equal(a.get(names[-1]), b.get(names[-1]))
    assert not torch.equal(RandomSource(specs, 4, torch.float32, "cpu").get(names[0]), b.get(names[0]))
    check_specs(specs, a.available())


def test_random_values_are_a_function_of_seed_name_and_element():
    """Any part of a seeded tensor can be made on its own, and the numbers are pinned (the device
    kernel must give the same ones: tests/test_gpu_kernels.py compares them)."""
    from sharpinference_amd.weights import random_fill as rf

    key = rf.name_key(2, "model.layers.0.self_attn.q_proj.weight")
    whole = rf.host_fill(5000, key, rf.FILL_NORMAL, 0.02)
    assert (rf.host_fill(17, key, rf.FILL_NORMAL, 0.02, start=4000) == whole[4000:4017]).all()
    assert (whole != rf.host_fill(5000, rf.name_key(3, "model.layers.0.self_attn.q_proj.weight"), rf.FILL_NORMAL, 0.02)).mean() > 0.99
    assert (whole != rf.host_fill(5000, rf.name_key(2, "model.layers.1.self_attn.q_proj.weight"), rf.FILL_NORMAL, 0.02)).mean() > 0.99
    # written out from the formula for one element: word(c) = mix(key + (c + 1) * golden), twelve 16-bit fields
    M = (1 << 64) - 1

    def mix(z):
        z ^= z >> 30
        z = (z * 0xBF58476D1CE4E5B9) & M
        z ^= z >> 27
        z = (z * 0x94D049BB133111EB) & M
        return z ^ (z >> 31)

    i = 1234
    s = 0
    for j in range(3):
        w = mix((key + (3 * i + j + 1) * 0x9E3779B97F4A7C15) & M)
        s += sum((w >> sh) & 0xFFFF for sh in (0, 16, 32, 48))
    import numpy as np
    assert whole[i] == np.float32(s - 393210) * np.float32(0.02 / 65536.0)
    u = rf.host_fill(3, key, rf.FILL_UNIFORM)
    w0 = mix((key + 0x9E3779B97F4A7C15) & M) >> 40
    assert u[0] == np.float32(15099494 + ((w0 * 3355443) >> 24)) * np.float32(2.0 ** -24)


def test_bench_refuses_more_than_one_gpu():
    """The benchmark measures one GPU: for N > 1 it says so in one line and exits with 2, before
    anything touches a device."""
    import os
    import subprocess
    import sys

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    p = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2", "--steps", "1", "--warmup", "0"],
                       capture_output=True, text=True, timeout=60)
    assert p.returncode == 2 and len(p.stdout.strip().splitlines()) == 1 and "one GPU" in p.stdout


def test_bench_counts_what_a_chunked_layer_sees():
    """The roofline's bytes and the prefill's flops follow the layer kinds: a chunked layer sees
    the keys of its chunk only."""
    import os
    import sys

    sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
    import bench
    from sharpinference_amd.config.base import load_config

    d = dict(bench.SCOUT)
    d["num_hidden_layers"] = 4
    d["no_rope_layers"] = [1, 1, 1, 0]
    cfg = load_config(d)
    C = cfg.attention_chunk_size
    assert bench.visible_keys(cfg, 0, C - 1) == C and bench.visible_keys(cfg, 0, C) == 1
    assert bench.visible_keys(cfg, 3, C) == C + 1
    # twice the chunk: chunked layers do the work of two chunks, the global layer of one long prompt
    lin = bench.prefill_flops(cfg, 2 * C, 4) - bench.prefill_flops(cfg, 2 * C, 0)
    per_pair = 4 * cfg.num_attention_heads * cfg.head_dim
    pairs = 3 * 2 * (C * (C + 1) // 2) + (2 * C) * (2 * C + 1) // 2
    dense = bench.prefill_flops(cfg, 1, 4) - bench.prefill_flops(cfg, 1, 0) - 4 * per_pair   # the linear part of one token
    assert abs(lin - (2 * C * dense + per_pair * pairs)) <= 1e-6 * lin


def test_random_model_command_writes_a_folder_that_loads(tmp_path):
    """bin/sharpi-random-model: a configuration and a seed give a model folder, the same bytes
    each time, whose tensors are those the model asks for (32-bit where asked)."""
    import json
    import os
    import subprocess
    import sys

    from tiny_configs import TINY_C

    from sharpinference_amd.config.base import load_config
    from sharpinference_amd.registry import build_model
    from sharpinference_amd.weights import safetensors_io as st

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    cfg_path = tmp_path / "config.json"
    cfg_path.write_text(json.dumps(TINY_C))
    outs = []
    for name in ("m1", "m2"):
        p = subprocess.run([sys.executable, os.path.join(root, "bin", "sharpi-random-model"), "--config", str(cfg_path),
                            "--seed", "4", "--out", str(tmp_path / name), "--float32", "norm.weight"],
                           capture_output=True, text=True, timeout=120)
        assert p.returncode == 0, p.stderr
        outs.append(tmp_path / name)
    a, b = [(o / "model.safetensors").read_bytes() for o in outs]
    assert a == b
    cfg = load_config(str(outs[0]))
    assert cfg.to_dict() == load_config(dict(TINY_C)).to_dict()
    index = st.index_folder(str(outs[0]))
    specs = build_model(cfg).param_specs()
    assert set(index) == set(specs)
    for n, info in index.items():
        assert tuple(info.shape) == tuple(specs[n].shape), n
        assert info.dtype == (torch.float32 if n.endswith("norm.weight") else torch.bfloat16), n


def test_command_line_takes_the_reference_s_option_names():
    """Names and defaults of the reference's options (src/SharpInference.Cli/RunCommand.cs:50-210)."""
    from sharpinference_amd.cli import build_parser, parse_device

    a = build_parser().parse_args(["-m", "X", "-p", "1 2"])
    assert (a.temp, a.top_k, a.top_p, a.min_p, a.n_predict, a.seed, a.ctx_size) == (0.7, 40, 0.95, 0.05, 512, -1, 0)
    assert (a.repeat_penalty, a.frequency_penalty, a.presence_penalty, a.backend, a.n_gpu_layers) == (1.1, 0.0, 0.0, "auto", -1)
    b = build_parser().parse_args(["--model", "X", "--prompt", "1", "--rep-penalty", "1.3", "--ngl", "99", "--device", "CUDA0",
                                   "--n-predict", "7", "--ctx-size", "256", "--no-display-prompt", "--verbose-prompt"])
    assert b.repeat_penalty == 1.3 and b.n_gpu_layers == 99 and b.n_predict == 7 and b.ctx_size == 256
    assert parse_device(b.device) == "cuda:0" and parse_device("1") == "cuda:1" and parse_device(None) == "cuda:0"
    for bad in ("none", "Vulkan1x"):
        try:
            parse_device(bad)
        except SystemExit:
            pass
        else:
            raise AssertionError(bad)


def test_end_and_begin_tokens_of_config_json():
    base = dict(TINY_A)
    assert load_config(base).eos_token_ids == () and load_config(base).bos_token_id is None
    one = load_config({**base, "eos_token_id": 7, "bos_token_id": 3})
    assert one.eos_token_ids == (7,) and one.bos_token_id == 3 and one.to_dict()["eos_token_id"] == 7
    many = load_config({**base, "eos_token_id": [7, 9, 11]})
    assert many.eos_token_ids == (7, 9, 11) and load_config(many.to_dict()) == many
    nested = load_config({"architectures": base["architectures"], "text_config": {k: v for k, v in base.items() if k != "architectures"},
                          "eos_token_id": [5]})
    assert nested.eos_token_ids == (5,)
    with pytest.raises(ConfigError, match="eos_token_id"):
        load_config({**base, "eos_token_id": "</s>"})


def _word_tokenizer(folder):
    """A tokenizer.json of whole words, made with the tokenizers package."""
    from tokenizers import Tokenizer, models, pre_tokenizers

    vocab = {"<unk>": 0, "<s>": 1, "the": 2, "cat": 3, "sat": 4, "on": 5, "mat": 6}
    tok = Tokenizer(models.WordLevel(vocab, unk_token="<unk>"))
    tok.pre_tokenizer = pre_tokenizers.Whitespace()
    tok.save(os.path.join(folder, "tokenizer.json"))


def test_prompts_as_text_or_ids(tmp_path):
    from sharpinference_amd.cli import prompt_ids
    from sharpinference_amd.text import TextCodec

    assert TextCodec.from_folder(str(tmp_path)) is None
    assert prompt_ids("1, 2 3", None) == [1, 2, 3]
    with pytest.raises(SystemExit, match="tokenizer.json"):
        prompt_ids("the cat", None)
    _word_tokenizer(str(tmp_path))
    codec = TextCodec.from_folder(str(tmp_path), bos_token_id=1)
    assert prompt_ids("the cat sat", codec) == [1, 2, 3, 4]            # the begin token leads, once
    assert prompt_ids("4 5 6", codec) == [4, 5, 6]                     # numbers stay token ids
    assert TextCodec.from_folder(str(tmp_path)).encode("on the mat") == [5, 2, 6]
    s = codec.streamer()
    assert [s.push(t) for t in (2, 3, 6)] == ["the", " cat", " mat"] and s.flush() == ""


def test_a_head_size_no_kernel_takes_is_refused_when_the_model_is_built():
    for hd in (272, 24):
        cfg = load_config({**TINY_A, "head_dim": hd})
        with pytest.raises(ValueError, match=f"head_dim {hd}"):
            build_model(cfg)
    with pytest.raises(ValueError, match="1025 experts"):
        build_model(load_config({**TINY_A, "num_local_experts": 1025}))


def test_other_layouts_of_the_same_tensors_are_read(tmp_path):
    """A container prefix, fused gate|up and [E, in, out] experts are found from names and shapes."""
    from sharpinference_amd.weights.loader import LayoutAdapter

    d = make_model_dir(tmp_path, "B")
    cfg = load_config(d)
    specs = build_model(cfg).param_specs()
    other = write_other_layout(d, str(tmp_path / "other"), "language_model.",
                                extra={"vision_model.patch.weight": torch.zeros(3, 5, dtype=torch.bfloat16)})
    plain = SafetensorsSource(d, torch.bfloat16, "cpu")
    adapted = LayoutAdapter(SafetensorsSource(other, torch.bfloat16, "cpu"), specs)
    assert adapted.prefix == "language_model."
    check_specs(specs, adapted.available(), other)                    # the other tower's tensor is not the decoder's business
    for n in specs:
        assert torch.equal(adapted.get(n), plain.get(n)), n
    # a canonical folder passes through untouched, and faults are still told in one error
    same = LayoutAdapter(SafetensorsSource(d, torch.bfloat16, "cpu"), specs)
    assert same.prefix == "" and all(torch.equal(same.get(n), plain.get(n)) for n in list(specs)[:5])
    broken = write_other_layout(d, str(tmp_path / "broken"), "language_model.",
                                 extra={"language_model.model.layers.9.extra.weight": torch.zeros(2, dtype=torch.bfloat16)})
    with pytest.raises(WeightError) as e:
        check_specs(specs, LayoutAdapter(SafetensorsSource(broken, torch.bfloat16, "cpu"), specs).available(), broken)
    assert "model.layers.9.extra.weight" in str(e.value)


@pytest.mark.parametrize("hidden,inter", [(64, 64), (64, 32), (64, 128)])
def test_axis_order_is_decided_by_name_where_the_shape_cannot_tell(tmp_path, hidden, inter):
    """A stacked expert tensor whose two sizes are equal (down: hidden == width; fused gate|up:
    hidden == 2 * width) reads the same transposed or not; the name decides: without a
    ``.weight`` suffix a fused tensor is [E, in, 2 * out] and the down beside it [E, in, out].
    The tensors are made unsymmetric so that a wrong reading cannot equal the right one."""
    from sharpinference_amd.weights.loader import LayoutAdapter

    d = make_model_dir(tmp_path, "A", hidden_size=hidden, intermediate_size=inter, head_dim=16)
    specs = build_model(load_config(d)).param_specs()
    other = write_other_layout(d, str(tmp_path / "other"), "")
    plain = SafetensorsSource(d, torch.bfloat16, "cpu")
    adapted = LayoutAdapter(SafetensorsSource(other, torch.bfloat16, "cpu"), specs)
    check_specs(specs, adapted.available(), other)
    for n in specs:
        got, want = adapted.get(n), plain.get(n)
        assert torch.equal(got, want), n
        if want.dim() == 3 and want.shape[1] == want.shape[2]:
            assert not torch.equal(want, want.transpose(1, 2)), "the test's tensor must tell the two readings apart"
    # the canonical folder (separate gate and up, down [E, out, in]) with the same sizes is left as it is
    same = LayoutAdapter(SafetensorsSource(d, torch.bfloat16, "cpu"), specs)
    assert all(torch.equal(same.get(n), plain.get(n)) for n in specs)


def test_chat_form_system_prompt_and_raw_text(tmp_path):
    """Text prompts take the Llama 4 chat form of the reference's fallback template
    (src/SharpInference.Cli/RunCommand.cs:2588-2596) when the tokenizer knows its marks;
    --system-prompt adds the system message; --raw-prompt leaves the text alone."""
    from tokenizers import Tokenizer, models, pre_tokenizers
    from tokenizers import AddedToken

    from sharpinference_amd.cli import build_parser, prompt_ids
    from sharpinference_amd.text import TextCodec, format_llama4_chat

    assert format_llama4_chat("hi", None) == \
        "<|begin_of_text|><|header_start|>user<|header_end|>\n\nhi<|eot|><|header_start|>assistant<|header_end|>\n\n"
    assert format_llama4_chat("hi", "be brief").startswith(
        "<|begin_of_text|><|header_start|>system<|header_end|>\n\nbe brief<|eot|><|header_start|>user<|header_end|>")
    words = ["<unk>", "hi", "there", "be", "brief", "user", "system", "assistant"]
    tok = Tokenizer(models.WordLevel({w: i for i, w in enumerate(words)}, unk_token="<unk>"))
    tok.pre_tokenizer = pre_tokenizers.Whitespace()
    plain_dir = tmp_path / "plain"
    plain_dir.mkdir()
    tok.save(str(plain_dir / "tokenizer.json"))
    plain = TextCodec.from_folder(str(plain_dir), None)
    assert not plain.knows_chat_marks() and prompt_ids("hi there", plain) == [1, 2]
    with pytest.raises(SystemExit, match="chat form"):
        prompt_ids("hi", plain, system="be brief")
    marks = ["<|begin_of_text|>", "<|header_start|>", "<|header_end|>", "<|eot|>"]
    tok.add_special_tokens([AddedToken(m, special=True) for m in marks])
    chat_dir = tmp_path / "chat"
    chat_dir.mkdir()
    tok.save(str(chat_dir / "tokenizer.json"))
    chat = TextCodec.from_folder(str(chat_dir), None)
    b, hs, he, eot = (tok.token_to_id(m) for m in marks)
    assert chat.knows_chat_marks()
    assert prompt_ids("hi there", chat) == [b, hs, 5, he, 1, 2, eot, hs, 7, he]
    assert prompt_ids("hi", chat, system="be brief") == [b, hs, 6, he, 3, 4, eot, hs, 5, he, 1, eot, hs, 7, he]
    assert prompt_ids("hi there", chat, raw=True) == [1, 2]
    assert prompt_ids("5, 6 7", chat) == [5, 6, 7]                      # numbers are token ids, whatever the tokenizer
    a = build_parser().parse_args(["-m", "X", "--single-turn", "--system-prompt", "be brief", "--profile"])
    assert a.single_turn and a.system_prompt == "be brief" and a.profile and a.prompt is None
