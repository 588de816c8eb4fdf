"""bin/trace_run as a user runs it: a subprocess fed steps on standard input."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import helpers as H
from tiny_configs import CONFIGS, make_model_dir

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _run_trace(model_dir, dtype, steps, out_dir, max_tokens):
    cmd = [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", model_dir, "--dtype", dtype,
           "--out", out_dir, "--max-tokens", str(max_tokens)]
    p = subprocess.Popen(cmd, stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True)
    for st in steps:                       # the next step only after `done <step>`
        p.stdin.write(json.dumps(st) + "\n")
        p.stdin.flush()
        line = p.stdout.readline().strip()
        assert line == f"done {st['step']}", f"trace_run answered {line!r}"
    p.stdin.close()
    assert p.wait(timeout=60) == 0


def _collect(steps, out_dir, vocab):
    got = {}
    for st in steps:
        wanted = sum(len(e["want"]) for e in st["entries"])
        path = os.path.join(out_dir, f"{st['step']}.f32")
        if not wanted:
            assert not os.path.exists(path)
            continue
        arr = np.fromfile(path, dtype="<f4").reshape(wanted, vocab)
        row = 0
        for e in st["entries"]:
            n = len(e["want"])
            if n:
                got.setdefault(e["id"], []).append(torch.from_numpy(arr[row:row + n].copy()))
                row += n
    return {k: torch.cat(v, 0) for k, v in got.items()}


@pytest.mark.parametrize("which,dtype", [("A", "float32"), ("B", "float32"), ("C", "bfloat16")])
def test_trace_run_mixed(which, dtype, tmp_path):
    d = make_model_dir(tmp_path, which, std=0.1)
    vocab = CONFIGS[which]["vocab_size"]
    reqs = {f"q{i}": H.random_tokens(n, vocab, 900 + i) for i, n in enumerate([45, 90, 33, 70, 58])}
    steps = H.mixed_trace(reqs, seed=4)
    # leave some places unwanted, and one step with nothing wanted at all
    for st in steps[::3]:
        for e in st["entries"]:
            e["want"] = e["want"][-1:]
    steps[1]["entries"] = [dict(e, want=[]) for e in steps[1]["entries"]]
    out = str(tmp_path / "out")
    _run_trace(d, dtype, steps, out, H.tokens_held(steps))
    got = _collect(steps, out, vocab)
    for rid, toks in reqs.items():
        places = []
        pos = 0
        for st in steps:
            for e in st["entries"]:
                if e["id"] == rid:
                    places += [pos + w for w in e["want"]]
                    pos += len(e["tokens"])
        if dtype == "float32":
            H.assert_close_fp32(got[rid], H.plain_logits(d, toks)[places], f"trace_run {which} {rid}")
        else:   # configuration C uses every expert for every token: no route can flip
            H.assert_close_bf16(got[rid], H.plain_logits(d, toks, bf16_storage=True)[places], f"trace_run {which} {rid}",
                                *H.bounds_of(d))


def test_trace_run_past_the_length_config_json_names(tmp_path):
    """A replay is bounded by --max-tokens, not by max_position_embeddings: given tokens need no trained positions."""
    d = make_model_dir(tmp_path, "A", std=0.1, max_position_embeddings=32)
    vocab = CONFIGS["A"]["vocab_size"]
    toks = H.random_tokens(100, vocab, 77)
    steps = [{"step": 0, "entries": [{"id": "x", "tokens": toks[:61], "want": [0, 31, 60]}], "end": []},
             {"step": 1, "entries": [{"id": "x", "tokens": toks[61:99], "want": [37]}], "end": []},
             {"step": 2, "entries": [{"id": "x", "tokens": toks[99:], "want": [0]}], "end": ["x"]}]
    out = str(tmp_path / "out")
    _run_trace(d, "float32", steps, out, 128)
    got = _collect(steps, out, vocab)["x"]
    H.assert_close_fp32(got, H.plain_logits(d, toks)[[0, 31, 60, 98, 99]], "trace_run past the named length")
