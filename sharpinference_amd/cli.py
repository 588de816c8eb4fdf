"""Command line in the manner of the reference's ``sharpi-cli`` (reference:
src/SharpInference.Cli/RunCommand.cs:23-300 for the options, 1907-1911 for the closing line
``Prefill: N tokens, X t/s | Decode: M tokens, Y t/s``).

Options keep the reference's names and meanings where it has them: -m/--model, -p/--prompt,
-f/--file, -n/--n-predict (512), --temp (0.7; 0 = greedy), --top-k (40), --top-p (0.95),
--min-p (0.05), -s/--seed (-1 = from the clock), -c/--ctx-size (0 = the model's), --kv-type,
--repeat-penalty/--rep-penalty (1.1), --repeat-last-n, --frequency-penalty, --presence-penalty,
--verbose-prompt, --no-display-prompt, --device (an index or a name), -g/--ngl (accepted: every
layer is on the GPU), --backend (auto).  -p and -f take text if the model folder has a
``tokenizer.json`` (the generated text is then printed as it comes); a prompt that is nothing
but numbers, ``--prompt-ids 1,2,3``, and every prompt for a folder without a tokenizer, are
token ids, and ``--prompt-len N`` makes N random ids.  Generation stops at the configuration's
``eos_token_id`` (``--ignore-eos`` switches that off; ``--stop-ids`` adds more).  ``-m`` names
a model folder (config.json + model.safetensors); with ``--random-weights`` the folder needs
only config.json.

Text prompts are put into the Llama 4 chat form (RunCommand.cs:2588-2596) when the folder's
tokenizer knows the form's marks, ``--system-prompt`` adds the system message of that form, and
``--raw-prompt`` leaves the text as it is.  Without any prompt option the command reads prompts
from standard input, one a line, until ``/exit``, ``/quit`` or the end of input (the reference's
interactive mode, RunCommand.cs:2185-2226: every turn starts from an empty cache); ``--single-turn``
ends after the first.  ``--profile`` launches every step part by part and prints milliseconds,
bytes and GB/s per kernel class at the end (the reference's SHARPI_CUDA_PROFILE buckets,
src/SharpInference.Engine/CudaForwardPass.cs:1523-1539).
"""
from __future__ import annotations

import argparse
import random
import re
import sys
import time
from typing import List, Optional


def _ids(text: str) -> List[int]:
    parts = [p for p in re.split(r"[,\s]+", text.strip()) if p]
    try:
        return [int(p) for p in parts]
    except ValueError:
        raise SystemExit(f"token ids expected (comma or space separated numbers), got {text[:40]!r}") from None


def prompt_ids(text: str, codec, system: Optional[str] = None, raw: bool = False) -> List[int]:
    """A prompt from the command line: numbers are token ids; anything else is text for the
    folder's tokenizer, in the chat form if the tokenizer knows its marks (and `raw` is not set)."""
    if re.fullmatch(r"[\d,\s]+", text) and re.search(r"\d", text):
        if system is not None:
            raise SystemExit("--system-prompt belongs to text prompts: token ids are taken as they are")
        return _ids(text)
    if codec is None:
        raise SystemExit("the model folder has no tokenizer.json: give the prompt as token ids, e.g. -p '1,2,3'")
    if not raw and codec.knows_chat_marks():
        return codec.encode_chat(text, system)
    if system is not None:
        raise SystemExit("--system-prompt needs the chat form, whose marks this folder's tokenizer does not know"
                         if not raw else "--system-prompt and --raw-prompt contradict each other")
    return codec.encode(text)


def parse_device(text: Optional[str]) -> str:
    """--device as the reference takes it (an index or a name, reference:
    src/SharpInference.Cli/RunCommand.cs:99-102) -> a torch device string; 'none' (the CPU) is refused."""
    if text is None or text == "" or text.lower() == "auto":
        return "cuda:0"
    t = text.strip().lower()
    if t == "none" or t == "cpu":
        raise SystemExit("--device none asks for the CPU: this engine has no CPU path")
    m = re.fullmatch(r"(?:cuda:?|hip:?|gpu:?)?(\d+)", t)
    if not m:
        raise SystemExit(f"--device {text!r}: give an index (0, 1, ...) or a name such as cuda:0")
    return f"cuda:{int(m.group(1))}"


def build_parser() -> argparse.ArgumentParser:
    ap = argparse.ArgumentParser(prog="sharpi-cli", description="Generate with a Llama 4 model folder on one MI355X.")
    ap.add_argument("-m", "--model", required=True, help="model folder (config.json, model.safetensors)")
    ap.add_argument("-p", "--prompt", help="prompt: text (the folder's tokenizer.json encodes it) or token ids "
                                           "(comma or space separated numbers)")
    ap.add_argument("-f", "--file", help="read the prompt (text or token ids) from a file")
    ap.add_argument("--prompt-ids", help="prompt as token ids (same as -p)")
    ap.add_argument("--prompt-len", type=int, help="a prompt of N random token ids")
    ap.add_argument("-n", "--n-predict", type=int, default=512, help="tokens to generate")
    ap.add_argument("--temp", type=float, default=0.7, help="temperature; 0 = greedy")
    ap.add_argument("--top-k", type=int, default=40)
    ap.add_argument("--top-p", type=float, default=0.95)
    ap.add_argument("--min-p", type=float, default=0.05)
    ap.add_argument("-s", "--seed", type=int, default=-1, help="sampling seed; -1 = from the clock")
    ap.add_argument("-c", "--ctx-size", type=int, default=0, help="longest sequence; 0 = the model's")
    ap.add_argument("--kv-type", default=None, choices=["fp32", "bf16"], help="cache dtype (follows --dtype)")
    ap.add_argument("--repeat-penalty", "--rep-penalty", dest="repeat_penalty", type=float, default=1.1)
    ap.add_argument("--repeat-last-n", type=int, default=256)
    ap.add_argument("--frequency-penalty", type=float, default=0.0)
    ap.add_argument("--presence-penalty", type=float, default=0.0)
    ap.add_argument("--verbose-prompt", action="store_true", help="print the prompt's token ids")
    ap.add_argument("--no-display-prompt", action="store_true")
    ap.add_argument("--single-turn", action="store_true", help="interactive mode: generate one response and exit")
    ap.add_argument("--system-prompt", default=None, help="system message of the chat form (text prompts)")
    ap.add_argument("--raw-prompt", action="store_true", help="text prompts as they are, without the chat form")
    ap.add_argument("--profile", action="store_true", help="launch steps part by part and print ms / bytes / GB/s per kernel class")
    ap.add_argument("--stop-ids", default="", help="token ids that end generation, beside the model's eos_token_id")
    ap.add_argument("--ignore-eos", action="store_true", help="do not stop at the model's eos_token_id")
    ap.add_argument("-g", "--ngl", "--n-gpu-layers", "--gpu-layers", dest="n_gpu_layers", type=int, default=-1,
                    help="accepted for the reference's sake: every layer runs on the GPU (-1 or any count > 0; 0 is refused)")
    ap.add_argument("--device", default=None, help="GPU to run on: an index (0, 1, ...) or a name (cuda:0); default 0")
    ap.add_argument("--backend", default="auto", choices=["auto", "hip"], help="there is one backend: HIP on gfx950")
    # this engine's own
    ap.add_argument("--dtype", default="bf16", choices=["bf16", "fp32", "bfloat16", "float32"])
    ap.add_argument("--random-weights", action="store_true", help="seeded random weights (folder needs config.json only)")
    ap.add_argument("--weight-seed", type=int, default=0)
    ap.add_argument("--parallel", type=int, default=1, help="generate this many copies of the prompt at once")
    ap.add_argument("--max-num-seqs", type=int, default=8)
    ap.add_argument("--max-tokens-per-step", type=int, default=2048)
    ap.add_argument("--kv-tokens", type=int, default=None, help="size of each page pool in tokens")
    ap.add_argument("--page-size", type=int, default=16)
    return ap


def main(argv: Optional[List[str]] = None) -> int:
    args = build_parser().parse_args(argv)
    from .config.base import load_config
    from .engine import Engine
    from .sampling.params import SamplingParams

    dtype = {"bf16": "bfloat16", "fp32": "float32"}.get(args.dtype, args.dtype)
    device = parse_device(args.device)
    if args.n_gpu_layers == 0:
        raise SystemExit("-g 0 asks for the CPU: this engine has no CPU path (leave -g out, or give -1)")
    if args.kv_type and {"bf16": "bfloat16", "fp32": "float32"}[args.kv_type] != dtype:
        raise SystemExit("--kv-type must equal --dtype: the cache is stored in the compute dtype")
    cfg = load_config(args.model)
    from .text import TextCodec
    codec = TextCodec.from_folder(args.model, cfg.bos_token_id)
    def text_prompt(text):
        return prompt_ids(text, codec, args.system_prompt, args.raw_prompt)

    interactive = False
    if args.file:
        with open(args.file) as f:
            prompt = text_prompt(f.read())
    elif args.prompt_ids:
        prompt = _ids(args.prompt_ids)
    elif args.prompt:
        prompt = text_prompt(args.prompt)
    elif args.prompt_len:
        rng = random.Random(args.weight_seed)
        prompt = [rng.randrange(cfg.vocab_size) for _ in range(args.prompt_len)]
    else:
        interactive, prompt = True, None
    ctx = args.ctx_size or None
    common = dict(dtype=dtype, device=device, max_model_len=ctx, max_num_seqs=max(args.max_num_seqs, args.parallel),
                  max_tokens_per_step=args.max_tokens_per_step, kv_tokens=args.kv_tokens, page_size=args.page_size,
                  decode_graphs=not args.profile)
    if args.random_weights:
        eng = Engine(config=cfg, weight_seed=args.weight_seed, **common)
    else:
        eng = Engine(args.model, **common)
    seed = args.seed if args.seed >= 0 else int(time.time() * 1000) & 0x7FFFFFFF

    def sampling(turn: int):
        return [SamplingParams(temperature=args.temp, top_k=args.top_k, top_p=args.top_p, min_p=args.min_p,
                               repetition_penalty=args.repeat_penalty, penalty_last_n=args.repeat_last_n,
                               frequency_penalty=args.frequency_penalty, presence_penalty=args.presence_penalty,
                               max_new_tokens=args.n_predict, stop_token_ids=() if args.ignore_eos else None,
                               additional_stop_token_ids=tuple(_ids(args.stop_ids)) if args.stop_ids else (),
                               seed=seed + turn * args.parallel + i) for i in range(args.parallel)]

    profiler = None
    if args.profile:
        from .ops.profile import Profiler

        profiler = Profiler()
        profiler.__enter__()

    def stream_one(ids: List[int], params) -> None:
        """One request: its tokens are printed as they come (the reference streams its chunks the same way)."""
        first = True
        stream = codec.streamer() if codec else None
        for c in eng.generate_chunks([ids], params):
            if c.kind == "token":
                piece = stream.push(c.token_id) if stream else ("" if first else " ") + str(c.token_id)
                print(piece, end="", flush=True)
                first = False
            elif c.kind == "stop":
                print((stream.flush() if stream else "") + f"  ({c.finish_reason})", flush=True)

    try:
        if interactive:
            # the reference's interactive chat (RunCommand.cs:2185-2226): a line a turn, every turn from an empty cache
            print("Interactive mode: a prompt a line (text, or token ids); /exit to quit.", flush=True)
            turn = 0
            while True:
                print("> ", end="", flush=True)
                line = sys.stdin.readline()
                if not line or line.strip() in ("/exit", "/quit"):
                    break
                if not line.strip():
                    continue
                ids = text_prompt(line.strip())
                if args.verbose_prompt:
                    print(f"prompt tokens ({len(ids)}): {ids}")
                stream_one(ids, sampling(turn)[:1])
                st = eng.last_stats
                rate = st.decode_tokens / st.decode_seconds if st.decode_seconds > 0 else 0.0
                print(f"{st.decode_tokens + 1} tokens, {rate:.1f} t/s\n", flush=True)
                turn += 1
                if args.single_turn:
                    break
        else:
            if args.verbose_prompt:
                print(f"prompt tokens ({len(prompt)}): {prompt}")
            elif not args.no_display_prompt:
                print(codec.decode(prompt) if codec else " ".join(str(t) for t in prompt))
            if args.parallel == 1:
                stream_one(prompt, sampling(0))
            else:
                for i, r in enumerate(eng.generate([prompt] * args.parallel, sampling(0))):
                    shown = codec.decode(r.token_ids) if codec else " ".join(str(t) for t in r.token_ids)
                    print(f"[{i}] {shown}  ({r.finish_reason})")
            st = eng.last_stats
            pre = st.prefill_tokens / st.prefill_seconds if st.prefill_seconds > 0 else 0.0
            dec = st.decode_tokens / st.decode_seconds if st.decode_seconds > 0 else 0.0
            print(f"Prefill: {st.prefill_tokens} tokens, {pre:.1f} t/s | Decode: {st.decode_tokens} tokens, {dec:.1f} t/s")
    finally:
        if profiler is not None:
            from .ops.profile import format_table

            profiler.__exit__(None, None, None)
            print(format_table(profiler.table(), "all steps of this run, launched part by part, by kernel class (event pairs):"),
                  file=sys.stderr, flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
