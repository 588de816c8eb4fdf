"""The engine at the layer sizes of the model that is served (Llama 4 Scout: width 5,120, 40 heads
of 128 in 8 groups, 16 experts of width 8,192 and a shared one), two layers (one rotary with a
chunk window, one without), against the plain implementation.  The tiny configurations cannot
show a fault that appears only at these sizes: kernels chosen by size, weights stored tile by
tile, 16 experts on 16 waves, sums over 5,120 and 8,192 terms."""
import shutil

import pytest
import torch

import helpers as H

pytestmark = pytest.mark.gpu

SCOUT_SHAPED = {
    "architectures": ["Llama4ForCausalLM"],
    "hidden_size": 5120, "num_hidden_layers": 2, "num_attention_heads": 40, "num_key_value_heads": 8,
    "head_dim": 128, "vocab_size": 8192, "intermediate_size": 8192, "intermediate_size_mlp": 16384,
    "num_local_experts": 16, "num_experts_per_tok": 1, "interleave_moe_layer_step": 1,
    "no_rope_layers": [1, 0], "attention_chunk_size": 32, "use_qk_norm": True, "attn_temperature_tuning": True,
    "floor_scale": 16, "attn_scale": 0.1, "rms_norm_eps": 1e-5, "rope_theta": 500000.0,
    "rope_scaling": {"rope_type": "llama3", "factor": 16.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                     "original_max_position_embeddings": 8192},
    "tie_word_embeddings": False, "max_position_embeddings": 4096, "torch_dtype": "bfloat16",
}
N_TOKENS = 80


@pytest.fixture(scope="module")
def scout_dir(tmp_path_factory):
    from sharpinference_amd import load_config
    from sharpinference_amd.weights.loader import write_random_model

    root = tmp_path_factory.mktemp("scout_shaped")
    if shutil.disk_usage(root).free < 14 * 2 ** 30:
        pytest.skip("the two-layer model file takes 9 GB of temporary disk")
    d = str(root / "model")
    write_random_model(load_config(SCOUT_SHAPED), d, 2, std=0.02)
    yield d
    shutil.rmtree(d, ignore_errors=True)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_scout_shaped_every_cut(scout_dir, dtype):
    toks = H.random_tokens(N_TOKENS, SCOUT_SHAPED["vocab_size"], 1)
    eng = H.make_engine(scout_dir, dtype, kv_tokens=256, max_num_seqs=2)
    for name, cut in (("whole", H.whole(N_TOKENS)), ("last 32 decoded", H.last_decoded(N_TOKENS)),
                      ("portions", H.changing_portions(N_TOKENS, 1))):
        H.check_against_plain(eng, scout_dir, dtype, "x", toks, cut, f"scout-shaped {dtype} {name}")
    if dtype == "float32":   # the cut must not show beyond rounding
        a = H.run_cut(eng, "a", toks, H.whole(N_TOKENS))
        b = H.run_cut(eng, "b", toks, H.changing_portions(N_TOKENS, 2))
        assert float((a - b).abs().max()) <= 1e-5 * max(1.0, float(a.abs().max()))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_scout_shaped_mixed_batches(scout_dir, dtype):
    lens = [37, 70, 5, 64, 49]
    reqs = {f"r{i}": H.random_tokens(n, SCOUT_SHAPED["vocab_size"], 400 + i) for i, n in enumerate(lens)}
    steps = H.mixed_trace(reqs, 0)
    eng = H.make_engine(scout_dir, dtype, kv_tokens=H.tokens_held(steps), max_num_seqs=4)
    H.check_trace_against_plain(eng, scout_dir, dtype, reqs, steps, f"scout-shaped {dtype} mixed")
    for g in eng.cache.groups:
        assert g.pool.num_free == g.pool.num_pages


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("width", [8, 17, 33, 65])
def test_scout_shaped_wide_decode_batches(scout_dir, width, dtype):
    """The served model's layer sizes with as many live requests as a serving step has, on both
    sides of the batch sizes at which a step changes kernels."""
    import random

    rng = random.Random(width)
    reqs = {f"w{i}": H.random_tokens(rng.randint(4, 12), SCOUT_SHAPED["vocab_size"], 8000 + 100 * width + i)
            for i in range(width)}
    steps = H.wide_trace(reqs, tail=2, per_prefill_step=16)
    eng = H.make_engine(scout_dir, dtype, kv_tokens=H.tokens_held(steps), max_num_seqs=width)
    H.check_trace_against_plain(eng, scout_dir, dtype, reqs, steps, f"scout-shaped {dtype} {width} live requests")
