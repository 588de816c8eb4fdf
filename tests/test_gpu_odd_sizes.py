"""Sizes at the edges of what the kernels take: head sizes in steps of 16 that no matrix-core
kernel serves, widths that are no multiple of 8, prime vocabularies, one kv head, as many kv
heads as heads, one expert, every expert picked, 130 experts, no routed layer.  Each configuration runs whole, with its last
tokens decoded one by one and in portions, in 32-bit and in bfloat16, against the plain
implementation: a size a kernel cannot take must go to another kernel, never to a wrong result."""
import pytest

import helpers as H
from tiny_configs import make_model_dir

pytestmark = pytest.mark.gpu

CASES = {
    # head size 80 (generic attention, scalar rotary kernel), width 76 (no multiple of 8), prime vocabulary
    "hd80_w76": ("A", dict(hidden_size=76, num_attention_heads=3, num_key_value_heads=1, head_dim=80, vocab_size=251,
                           intermediate_size=52, num_local_experts=3, num_experts_per_tok=2, attention_chunk_size=24)),
    # head size 112, seven heads on seven kv heads, one expert (the router has nothing to choose)
    "hd112_e1": ("B", dict(hidden_size=104, num_attention_heads=7, num_key_value_heads=7, head_dim=112, vocab_size=307,
                           intermediate_size=40, intermediate_size_mlp=72, num_local_experts=1, num_experts_per_tok=1)),
    # head size 144 > 128, widths that are multiples of 128 (matrix-core products) beside an attention they refuse
    "hd144_w256": ("D", dict(hidden_size=256, num_attention_heads=4, num_key_value_heads=2, head_dim=144, vocab_size=509,
                             intermediate_size=128, num_local_experts=5, num_experts_per_tok=5)),
    # head size 96 and 192: matrix-core attention at sizes the other tests do not use, many heads per kv head
    "hd96_g8": ("D", dict(hidden_size=128, num_attention_heads=8, num_key_value_heads=1, head_dim=96, vocab_size=1000,
                          intermediate_size=256, num_local_experts=2, num_experts_per_tok=1)),
    # no layer routed at all (the step is larger than the model), and many experts, no power of two, four picked
    "dense_only": ("B", dict(interleave_moe_layer_step=7, vocab_size=384)),
    "e130_k4": ("A", dict(num_local_experts=130, num_experts_per_tok=4, vocab_size=256)),
    # head sizes 160 and 256: the decode attention's matrix-core kernel with one chunk in flight, prompts through
    # the generic kernel; 256 is the largest head size taken
    "hd160": ("B", dict(hidden_size=96, num_attention_heads=3, num_key_value_heads=1, head_dim=160, vocab_size=311,
                        attention_chunk_size=20)),
    "hd256": ("D", dict(hidden_size=128, num_attention_heads=2, num_key_value_heads=2, head_dim=256, vocab_size=499,
                        intermediate_size=128, num_local_experts=3, num_experts_per_tok=2, attention_chunk_size=56)),
    # the tanh form of GELU in every feed-forward, and biases on the four attention projections
    "gelu_bias": ("B", dict(hidden_act="gelu_pytorch_tanh", attention_bias=True, vocab_size=384)),
    "bias_mfma": ("D", dict(attention_bias=True, vocab_size=500)),
    "hd192": ("D", dict(hidden_size=384, num_attention_heads=2, num_key_value_heads=2, head_dim=192, vocab_size=333,
                        intermediate_size=128, num_local_experts=4, num_experts_per_tok=2, attention_chunk_size=40)),
}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("case", sorted(CASES))
def test_sizes_at_the_edges(tmp_path, case, dtype):
    base, overrides = CASES[case]
    # (weights of this scale keep bfloat16's rounding at half the tolerance on the widest of the cases:
    # every cut of a request shows the same level, so it is the model's, not a cut's)
    d = make_model_dir(tmp_path, base, std=0.05, **overrides)
    vocab = overrides["vocab_size"]
    eng = H.make_engine(d, dtype, kv_tokens=512, max_num_seqs=2)
    toks = H.random_tokens(75, vocab, 11)
    H.check_against_plain(eng, d, dtype, "w", toks, H.whole(len(toks)), f"{case} {dtype} whole")
    H.check_against_plain(eng, d, dtype, "d", toks, H.last_decoded(len(toks), 20), f"{case} {dtype} decoded")
    H.check_against_plain(eng, d, dtype, "p", toks, H.changing_portions(len(toks), 3), f"{case} {dtype} portions")
    eng.cache.check_invariants()
