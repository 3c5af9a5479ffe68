"""Command line in the reference's manner (crates/server/src/main.rs:14-127, 216-294):

    rlis generate   --model DIR --prompt-ids 1,2,3 --max-tokens 128 --temperature 0 ...
    rlis perplexity --model DIR --ids-file tokens.txt --ctx 512 --max-windows 0

Option names, meanings and defaults are the reference's.  Differences: the model is a folder
of safetensors only; ``--dtype`` is ``f32`` or ``bf16`` (default bf16); prompts may be given
as token ids (``--prompt-ids``, ``--ids-file``) since a tokenizer is optional; a model with
seeded random weights can be built from a configuration (``--random-weights``); ``serve`` and
``--chat`` belong to the server side and are not part of this engine."""
from __future__ import annotations

import argparse
import json
import os
import sys
from typing import List, Optional

_DTYPES = {"f32": "float32", "fp32": "float32", "float32": "float32",
           "bf16": "bfloat16", "bfloat16": "bfloat16"}


def _dtype(name: str) -> str:
    if name in ("f16", "fp16", "float16", "half"):
        raise argparse.ArgumentTypeError(
            "f16 (the reference's default) is not built here: use bf16 or f32")
    if name not in _DTYPES:
        raise argparse.ArgumentTypeError(f"unknown dtype '{name}': one of {', '.join(sorted(_DTYPES))}")
    return name


def _add_model_args(p: argparse.ArgumentParser) -> None:
    p.add_argument("--model", help="a folder with config.json and *.safetensors")
    p.add_argument("--tokenizer", help="folder with tokenizer.json (needed for text prompts)")
    p.add_argument("--dtype", default="bf16", type=_dtype,
                   help="weight and activation dtype: bf16 (default) or f32 / fp32")
    p.add_argument("--device", default="hip", help="'hip' (the GPU); there is no CPU path")
    p.add_argument("--max-seq-len", type=int, default=2048,
                   help="longest prompt plus completion, in tokens")
    p.add_argument("--random-weights", action="store_true",
                   help="build the model from --config with seeded random weights")
    p.add_argument("--config", help="with --random-weights: a preset name or a config.json")
    p.add_argument("--weights-seed", type=int, default=0)


def _add_engine_args(p: argparse.ArgumentParser) -> None:
    p.add_argument("--kv-cache-gb", type=float, default=1.0, help="size of the page pool")
    p.add_argument("--num-pages", type=int, default=None, help="pool size in pages, overrides --kv-cache-gb")
    p.add_argument("--block-size", "--page-size", dest="block_size", type=int, default=16,
                   help="tokens per page")
    p.add_argument("--max-num-seqs", type=int, default=64, help="most sequences in one step")
    p.add_argument("--max-batched-tokens", type=int, default=2048,
                   help="most tokens in one step; longer prompts are prefilled in portions")
    p.add_argument("--scheduler", default="continuous", choices=["continuous", "static"])
    p.add_argument("--attention", default="v2", choices=["v1", "v2"],
                   help="v2: the specialised attention kernels; v1: the generic kernel only")
    p.add_argument("--no-prefix-caching", action="store_true",
                   help="accepted for compatibility; this engine has no prefix cache")


def _load(args):
    from .config import preset_dict, preset_names
    from .engine import load_model, random_model
    if args.device not in ("hip", "cuda", "gpu"):
        raise SystemExit(f"--device {args.device}: this engine runs on the GPU only ('hip')")
    dtype = _DTYPES[args.dtype]
    if args.random_weights:
        if not args.config:
            raise SystemExit("--random-weights needs --config (a preset name or a config.json)")
        if args.config in preset_names():
            cfg = preset_dict(args.config)
        else:
            with open(args.config) as f:
                cfg = json.load(f)
        return random_model(cfg, args.weights_seed, dtype, args.max_seq_len)
    if not args.model:
        raise SystemExit("--model is required (or --random-weights --config ...)")
    return load_model(args.model, dtype, args.max_seq_len)


def _tokenizer(args):
    folder = args.tokenizer or args.model
    path = os.path.join(folder or "", "tokenizer.json")
    if not (folder and os.path.exists(path)):
        return None
    from tokenizers import Tokenizer
    return Tokenizer.from_file(path)


def _parse_ids(text: str) -> List[int]:
    return [int(t) for t in text.replace(",", " ").split()]


def run_generate(args) -> int:
    from . import ops
    from .config import EngineConfig
    from .engine import Engine
    from .sampling import SamplingParams
    model = _load(args)
    tok = _tokenizer(args)
    if args.prompt_ids is not None:
        prompt = _parse_ids(args.prompt_ids)
    elif args.prompt is not None:
        if tok is None:
            raise SystemExit("--prompt needs a tokenizer.json (see --tokenizer); or use --prompt-ids")
        prompt = tok.encode(args.prompt).ids
    else:
        raise SystemExit("one of --prompt and --prompt-ids is required")
    if args.attention == "v1":
        ops.FORCE_ATTENTION = "generic"
    engine = Engine(model, EngineConfig(
        max_num_seqs=args.max_num_seqs, max_batched_tokens=args.max_batched_tokens,
        kv_cache_gb=args.kv_cache_gb, num_pages=args.num_pages, block_size=args.block_size,
        scheduler=args.scheduler, max_seq_len=args.max_seq_len))
    params = SamplingParams(temperature=args.temperature, top_p=args.top_p, top_k=args.top_k,
                            repetition_penalty=args.repetition_penalty, seed=args.seed,
                            max_tokens=args.max_tokens)
    seq_id = engine.add_request(prompt, params)
    first = True
    while engine.has_work():
        for _, token, _ in engine.step():
            if token is None:
                continue
            if tok is not None:
                sys.stdout.write(tok.decode([token]))
            else:
                sys.stdout.write(("" if first else " ") + str(token))
            sys.stdout.flush()
            first = False
    done = engine.pop_finished(seq_id)
    print(f"\n\nprompt {done.prompt_tokens} tok | output {done.completion_tokens} tok "
          f"({done.finish_reason}) | ttft {done.ttft * 1e3:.1f}ms | decode "
          f"{done.decode_tokens_per_sec:.1f} tok/s", file=sys.stderr)
    return 0


def run_perplexity(args) -> int:
    from .engine import ModelRunner
    from .engine.perplexity import perplexity
    model = _load(args)
    if args.ids_file:
        with open(args.ids_file) as f:
            tokens = _parse_ids(f.read())
        bos = args.bos if args.bos is not None else tokens[0]
    else:
        tok = _tokenizer(args)
        if tok is None:
            raise SystemExit("--file needs a tokenizer.json (see --tokenizer); or use --ids-file")
        with open(args.file, encoding="utf-8") as f:
            tokens = tok.encode(f.read()).ids
        bos = tokens[0]
    print(f"{len(tokens)} tokens", file=sys.stderr)
    runner = ModelRunner(model, num_pages=-(-args.ctx // args.block_size) + 1,
                         page_size=args.block_size, max_num_seqs=1)

    def progress(done, total, ppl):
        if done % 50 == 0 or done == total:
            print(f"[{done}/{total}] ppl {ppl:.4f}", file=sys.stderr)

    r = perplexity(runner, tokens, bos, args.ctx, args.max_windows, progress)
    print(f"PPL = {r.ppl:.4f} +/- {r.ppl_stderr:.4f} over {r.tokens_scored} tokens "
          f"({r.windows} windows of {r.ctx}) in {r.seconds:.1f}s", file=sys.stderr)
    print(json.dumps(r.to_dict()))
    return 0


def build_parser() -> argparse.ArgumentParser:
    ap = argparse.ArgumentParser(prog="rlis", description="Llama inference engine for MI355X")
    sub = ap.add_subparsers(dest="command", required=True)
    g = sub.add_parser("generate", help="generate a completion for one prompt")
    _add_model_args(g)
    _add_engine_args(g)
    g.add_argument("--prompt", help="prompt text (needs a tokenizer)")
    g.add_argument("--prompt-ids", help="prompt as token ids, comma or space separated")
    g.add_argument("--max-tokens", type=int, default=128)
    g.add_argument("--temperature", type=float, default=0.0)
    g.add_argument("--top-p", type=float, default=1.0)
    g.add_argument("--top-k", type=int, default=0)
    g.add_argument("--repetition-penalty", type=float, default=1.0)
    g.add_argument("--seed", type=int, default=None)
    p = sub.add_parser("perplexity", help="windowed perplexity of a token stream")
    _add_model_args(p)
    p.add_argument("--file", help="text file (needs a tokenizer)")
    p.add_argument("--ids-file", help="file of token ids, comma or space separated")
    p.add_argument("--bos", type=int, default=None, help="BOS id put at the start of each window")
    p.add_argument("--ctx", type=int, default=512, help="window length; the second half is scored")
    p.add_argument("--max-windows", type=int, default=0, help="score only the first N windows (0 = all)")
    p.add_argument("--block-size", "--page-size", dest="block_size", type=int, default=16)
    return ap


def main(argv: Optional[List[str]] = None) -> int:
    args = build_parser().parse_args(argv)
    return run_generate(args) if args.command == "generate" else run_perplexity(args)


if __name__ == "__main__":
    sys.exit(main())
