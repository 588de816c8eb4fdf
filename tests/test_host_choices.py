"""Choices the host makes without a GPU: the shapes of the few-rows product's launches, the
benchmark's refusal of more than one GPU, the byte counts its roofline is priced with."""
import json
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_few_rows_launch_shapes_follow_the_rows_and_the_compute_units():
    from sharpinference_amd import ops

    # the waves that split K are the same whatever the rows: a row's sums do not change with the batch
    assert {ops.skinny_plan(N, K, rb, g)[1] for N in (5120, 7168, 16384, 202048) for K in (5120, 8192)
            for rb in (1, 2, 4) for g in (1, 2, 9, 17)} == {8}
    # one block of rows: two tiles a block (two K units in flight), wide or not
    assert ops.skinny_plan(7168, 5120, 1)[0] == 2 and ops.skinny_plan(202048, 5120, 1)[0] == 2
    assert ops.skinny_plan(16384, 5120, 1, 9, act=True)[0] == 2
    # ... unless that makes between one and two blocks per compute unit: the merged down projection of one token
    assert ops.skinny_plan(5120, 8192, 1, 2)[0] == 1 and ops.skinny_plan(5120, 8192, 1, 9)[0] == 2
    assert ops.skinny_plan(5120, 5120, 1, 1)[0] == 2            # 160 blocks: every unit has at most one
    assert ops.skinny_plan(16384, 5120, 1, 1, act=True)[0] == 2  # the gated form pairs tiles: never one
    # more rows: four tiles for wide matrices
    assert ops.skinny_plan(16384, 5120, 4, 17)[0] == 4 and ops.skinny_plan(5120, 8192, 4, 17)[0] == 2


def test_the_decode_attention_s_runs_cover_every_window():
    """The decode attention cuts a token's visible keys into runs of 256, counted from the 16-key
    block that holds the first visible key, and sizes its workspace for a bound on the contexts.
    The bound's runs cover every token below it: all keys, chunks, and sliding windows that start
    inside a 16-key block (a window of 257 keys that starts at key 15 spans two runs)."""
    from sharpinference_amd import ops
    from sharpinference_amd.cache.spec import KVSpec, WINDOW_CHUNK, WINDOW_NONE, WINDOW_SLIDING

    run = ops.DECODE_RUN_KEYS
    assert run % 16 == 0
    specs = [KVSpec(1, 16, WINDOW_NONE, 0)] + [KVSpec(1, 16, kind, w) for kind in (WINDOW_CHUNK, WINDOW_SLIDING)
                                                for w in (1, 17, 24, 250, 256, 300, 1000, 4099)]
    for context in (1, 15, 16, 17, 255, 256, 257, 511, 513, 4096, 4097, 9000):
        bound = ops.decode_max_splits(context)
        assert bound == (context - 1) // run + 1            # the runs a context spans from key 0
        for spec in specs:
            for p in {0, context // 3, context - 2, context - 1} - {-1}:
                if p < 0:
                    continue
                s = spec.first_visible(p)
                wanted = ((p >> 4) - (s >> 4)) // (run // 16) + 1     # what the kernels walk (attention_decode.hip)
                assert (s >> 4) * 16 + wanted * run > p               # ... reaches the token's own key
                assert (s >> 4) * 16 + (wanted - 1) * run <= p        # ... with no run to spare
                assert wanted <= bound, (context, spec, p)


def test_benchmark_refuses_more_than_one_gpu():
    out = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert out.returncode == 2
    assert len(out.stdout.strip().splitlines()) == 1 and "one GPU" in out.stdout


def test_roofline_bytes_count_every_weight_once_and_the_live_cache():
    sys.path.insert(0, ROOT)
    import bench
    from sharpinference_amd import load_config

    cfg = load_config(dict(bench.SCOUT, num_hidden_layers=48, no_rope_layers=[0 if (l + 1) % 4 == 0 else 1 for l in range(48)]))
    H, I, V = cfg.hidden_size, cfg.intermediate_size, cfg.vocab_size
    attn = H * (cfg.num_attention_heads + 2 * cfg.num_key_value_heads) * cfg.head_dim + cfg.num_attention_heads * cfg.head_dim * H
    expert = 3 * H * I
    router = cfg.num_local_experts * H
    ctx, batch, distinct = 2100, 8, 6.5
    kv = 2 * cfg.num_key_value_heads * cfg.head_dim * ctx * batch
    want = 2 * (48 * (attn + router + (distinct + 1) * expert + kv) + V * H)
    got = bench.decode_step_bytes(cfg, 48, batch, ctx, distinct)
    assert abs(got - want) / want < 0.01, (got, want)
    json.dumps({"bytes": got})


def test_attention_work_lists_cut_a_step_into_decode_tokens_and_tiles():
    """What the attention parts ask the step function to upload: the tokens of entries of one
    token, and tiles of the longer entries: 64-token tiles while a step holds few prompt tokens,
    128-token tiles beyond; every token of a longer entry lies in exactly one tile, tiles do
    not cross entries."""
    import numpy as np
    from sharpinference_amd.parts.attention import SHORT_PROMPT_TOKENS, AttentionWorkLists
    from sharpinference_amd.parts.base import HostStep

    def plan(lens):
        cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
        host = HostStep(n_entries=len(lens), n_tokens=int(cu[-1]), lens=list(lens), starts=[7 * i for i in range(len(lens))], cu_tokens=cu)
        (dec, tiles), facts = AttentionWorkLists().plan(host)
        return cu, dec, tiles.reshape(-1, 3), facts

    cu, dec, tiles, facts = plan([1, 130, 1, 2, 64])
    assert dec.tolist() == [0, 131] and facts["n_dec"] == 2 and not facts["all_decode"]
    assert facts["tile"] == 64 and facts["n_tiles"] == len(tiles) == 3 + 1 + 1
    assert tiles.tolist() == [[1, 1, 64], [1, 65, 64], [1, 129, 2], [3, 132, 2], [4, 134, 64]]
    cu, dec, tiles, facts = plan([1, 1, 1])
    assert facts["all_decode"] and facts["n_tiles"] == 0 and tiles.size == 0 and dec.tolist() == [0, 1, 2]
    for lens in ([SHORT_PROMPT_TOKENS], [SHORT_PROMPT_TOKENS + 1], [700, 1, 900, 300], [4096, 5]):
        cu, dec, tiles, facts = plan(lens)
        assert facts["tile"] == (64 if sum(n for n in lens if n > 1) <= SHORT_PROMPT_TOKENS else 128)
        covered = np.zeros(int(cu[-1]), dtype=np.int32)
        for e, t0, rows in tiles.tolist():
            assert 1 <= rows <= facts["tile"] and cu[e] <= t0 and t0 + rows <= cu[e + 1]
            covered[t0:t0 + rows] += 1
        want = np.concatenate([np.full(n, 1 if n > 1 else 0) for n in lens])
        assert covered.tolist() == want.tolist()
    # under a graph's trial run the lists hold harmless contents of the same sizes
    host = HostStep(n_entries=3, n_tokens=3, lens=[1, 1, 1], starts=[5, 6, 7], cu_tokens=np.arange(4, dtype=np.int32))
    arrays, _ = AttentionWorkLists().plan(host)
    null = AttentionWorkLists().null(host, arrays)
    assert [a.size for a in null] == [a.size for a in arrays] and null[0].tolist() == [0, 1, 2]
