"""Command line in the manner of the reference's `quarrel` and `generate_text`
(cmd/quarrel/main_metal.go:24-36, cmd/generate_text/main.go:18-26): the same option
names and meanings where it has them.

    quarrel -model DIR -prompt "1 15 27 3" -n 20 -temp 0.7 -topk 40 -topp 0.95 -penalty 1.1 -stream

`-model` is a folder with config.json and model.safetensors (env QUARREL_MODEL if the
option is absent, as generate_text does).  `-prompt` is text when the folder has a
tokenizer.json, else token ids separated by blanks or commas; several prompts are
separated by `|` and run as one batch; `-prompt-file` reads them from a file instead, one prompt a
line; `-prompt-ids` always takes token ids.  `-stop-id` (repeatable) names ids that end a sequence beside
the configuration's own.  The beginning-of-sequence id of the
configuration is put in front of text prompts (the reference prepends id 1,
cmd/quarrel/main_metal.go:113-114).
"""
from __future__ import annotations

import argparse
import os
import sys
import time
from typing import List, Optional


def build_parser() -> argparse.ArgumentParser:
    ap = argparse.ArgumentParser(prog="quarrel", description="generate tokens with a model folder on one MI355X")
    ap.add_argument("-model", "--model", default=os.environ.get("QUARREL_MODEL", ""),
                    help="folder with config.json and model.safetensors (or env QUARREL_MODEL)")
    ap.add_argument("-prompt", "--prompt", default="1", help="text, or token ids; '|' separates several prompts")
    ap.add_argument("-prompt-ids", "--prompt-ids", dest="prompt_ids", default="",
                    help="token ids (blanks or commas between them), also where the folder has a tokenizer")
    ap.add_argument("-prompt-file", "--prompt-file", dest="prompt_file", default="",
                    help="a file with one prompt a line (in the place of -prompt)")
    ap.add_argument("-n", "--n", "-len", "--len", "-max-new-tokens", "--max-new-tokens", dest="n", type=int,
                    default=20, help="number of tokens to generate")
    ap.add_argument("-stop-id", "--stop-id", dest="stop_ids", type=int, action="append", default=[],
                    help="a token id that ends a sequence, beside the configuration's (may be given several times)")
    ap.add_argument("-kv-cache-size", "--kv-cache-size", dest="kv_cache_size", type=int, default=2048,
                    help="tokens the cache holds for each sequence of the batch")
    ap.add_argument("-temp", "--temp", type=float, default=0.7, help="temperature (0 = greedy)")
    ap.add_argument("-topk", "--topk", type=int, default=40, help="top-k (0 = off)")
    ap.add_argument("-topp", "--topp", type=float, default=0.95, help="top-p (1 = off)")
    ap.add_argument("-penalty", "--penalty", type=float, default=1.1, help="repetition penalty (1 = off)")
    ap.add_argument("-stream", "--stream", action="store_true", help="print tokens as they are generated")
    ap.add_argument("-seed", "--seed", type=int, default=0, help="seed of the sampler")
    ap.add_argument("-dtype", "--dtype", choices=["bfloat16", "float32"], default="bfloat16")
    ap.add_argument("-v", "--v", dest="verbose", action="store_true", help="timing details")
    ap.add_argument("-random-config", "--random-config", dest="random_config", default="",
                    help="a config.json to build a model with random weights from (instead of -model)")
    return ap


def _encode(prompt: str, tokenizer, bos: Optional[int]) -> List[int]:
    if tokenizer is not None:
        ids = tokenizer.encode(prompt, add_special_tokens=False).ids
        return ([bos] if bos is not None else []) + ids
    try:
        return [int(t) for t in prompt.replace(",", " ").split()]
    except ValueError:
        raise SystemExit("quarrel: the model folder has no tokenizer.json, so -prompt must be token ids "
                         "(for instance \"1 15 27 3\")")


def main(argv: Optional[List[str]] = None) -> int:
    args = build_parser().parse_args(argv)
    if not args.model and not args.random_config:
        print("Error: --model flag is required", file=sys.stderr)  # cmd/quarrel/main_metal.go:41-45
        return 1
    import json

    import longbow_quarrel_amd as lq

    as_ids = bool(args.prompt_ids)
    if args.prompt_file:
        try:
            with open(args.prompt_file) as f:
                prompts_text = [line.strip() for line in f if line.strip()]
        except OSError as e:
            print(f"Error: cannot read --prompt-file: {e}", file=sys.stderr)
            return 1
        if not prompts_text:
            print(f"Error: {args.prompt_file} holds no prompt", file=sys.stderr)
            return 1
    else:
        prompts_text = (args.prompt_ids or args.prompt).split("|")
    max_tokens = args.kv_cache_size * max(1, len(prompts_text))
    t0 = time.perf_counter()
    tokenizer = None
    if args.random_config:
        with open(args.random_config) as f:
            from longbow_quarrel_amd.registry import config_from_dict
            config = config_from_dict(json.load(f))
        engine = lq.random_engine(config, args.seed, dtype=args.dtype, max_tokens=max_tokens,
                                  max_sequence_tokens=args.kv_cache_size)
    else:
        engine = lq.load_engine(args.model, dtype=args.dtype, max_tokens=max_tokens,
                                max_sequence_tokens=args.kv_cache_size)
        tok_path = os.path.join(args.model, "tokenizer.json")
        if os.path.isfile(tok_path):
            from tokenizers import Tokenizer
            tokenizer = Tokenizer.from_file(tok_path)
    spec = engine.model.spec
    print("=== Longbow-Quarrel MI355X ===")
    print(f"Model: {args.model or args.random_config}")
    print(f"Architecture: {engine.config.architecture}")
    print(f"Layers: {len(spec.layers)}")
    print(f"Vocab: {spec.vocab_size}")
    if args.verbose:
        print(f"loaded in {time.perf_counter() - t0:.2f}s")

    prompts = [_encode(p.strip(), None if as_ids else tokenizer, spec.bos_id) for p in prompts_text]
    params = lq.SamplingParams(temperature=args.temp, top_k=args.topk, top_p=args.topp,
                               repetition_penalty=args.penalty, seed=args.seed)

    def show(ids: List[int]) -> str:
        return tokenizer.decode(ids) if tokenizer is not None else " ".join(str(i) for i in ids)

    callback = None
    if args.stream:
        print("Streaming output: ", end="", flush=True)

        def callback(request: int, token: int) -> None:
            prefix = f"[{request}]" if len(prompts) > 1 else ""
            print(prefix + show([token]), end=" ", flush=True)

    start = time.perf_counter()
    result = lq.generate(engine, prompts, args.n, params, callback=callback, extra_stop_ids=args.stop_ids)
    duration = time.perf_counter() - start
    if args.stream:
        print(" [END]")
    total = sum(len(t) for t in result.tokens)
    print("\n=== Complete ===")
    print(f"{total} tokens in {duration:.3f}s ({total / duration:.1f} t/s)\n")
    if args.verbose:
        print(f"prefill {result.prefill_tokens} tokens in {result.prefill_seconds:.3f}s, "
              f"{result.decode_steps} decode steps in {result.decode_seconds:.3f}s")
    for r, ids in enumerate(result.tokens):
        head = f"[{r}] " if len(prompts) > 1 else ""
        print(head + show(ids))
    return 0


if __name__ == "__main__":
    sys.exit(main())
