"""Command line in the manner of the reference's ``qwen3_infer [model_dir]``
(reference: demo/qwen3_infer.cpp:539-676): one positional model folder, generation
of up to ``--max-new-tokens`` tokens (the reference fixes 32, :542) with the
sampling options of its sampler (defaults from generation_config.json, :590-592),
and a tokens-per-second line at the end (:669-673).  There is no tokenizer in this
engine, so prompts are token ids.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time
from typing import List, Optional


def find_default_model_path() -> str:
    """Look upward from the working directory for a folder named ``model``
    (reference: demo/qwen3_infer.cpp:42-60)."""
    here = os.path.abspath(os.getcwd())
    while True:
        cand = os.path.join(here, "model")
        if os.path.isfile(os.path.join(cand, "config.json")):
            return cand
        parent = os.path.dirname(here)
        if parent == here:
            return "model"
        here = parent


def build_parser() -> argparse.ArgumentParser:
    p = argparse.ArgumentParser(prog="pulse_infer", description=__doc__.split("\n\n")[0])
    p.add_argument("model_dir", nargs="?", default=None, help="folder with config.json and *.safetensors")
    p.add_argument("--model", dest="model_opt", default=None, help="same as the positional model_dir")
    p.add_argument("--random-weights", action="store_true", help="ignore the folder's weights; make seeded random ones")
    p.add_argument("--seed", type=int, default=0, help="seed of random weights and of sampling")
    p.add_argument("--init", default="fan_in", help="random weights: 'fan_in' or a standard deviation such as 0.02")
    p.add_argument("--dtype", choices=["bfloat16", "float32", "bf16", "f32"], default="bfloat16")
    p.add_argument("--device", default="cuda:0")
    p.add_argument("--prompt-ids", action="append", default=[], help="comma separated token ids; may be repeated")
    p.add_argument("--prompt-file", default=None, help="JSON file: a list of lists of token ids")
    p.add_argument("--prompt-len", type=int, action="append", default=[], help="a prompt of N seeded random ids; may be repeated")
    p.add_argument("--max-new-tokens", type=int, default=32)
    p.add_argument("--temperature", type=float, default=None)
    p.add_argument("--top-k", type=int, default=None)
    p.add_argument("--top-p", type=float, default=None)
    p.add_argument("--presence-penalty", type=float, default=0.0)
    p.add_argument("--greedy", action="store_true", help="largest logit, whatever generation_config.json says")
    p.add_argument("--sample-seed", type=int, default=None)
    p.add_argument("--ignore-eos", action="store_true")
    p.add_argument("--page-size", type=int, default=16)
    p.add_argument("--num-pages", type=int, default=None)
    p.add_argument("--max-batch", type=int, default=8, help="most requests in one step")
    p.add_argument("--max-tokens", type=int, default=None, help="most tokens in one step (the budget)")
    p.add_argument("--chunk", type=int, default=256,
                   help="a prompt's portion of a step; what the step's budget (--max-tokens) has left when every "
                        "prompt has its portion extends the portions in order, unless --fixed-chunk is given")
    p.add_argument("--fixed-chunk", action="store_true", help="no prompt portion is longer than --chunk tokens")
    p.add_argument("--set", dest="overrides", action="append", default=[], metavar="FIELD=VALUE",
                   help="set a field of the model's configuration that is an option of the engine rather than a key of "
                        "config.json (for Qwen3: rope_pairing=half, the channels a rotation pairs); may be repeated")
    p.add_argument("--strict", action="store_true", help="a tensor that no part of the model asks for is an error")
    p.add_argument("--stats", action="store_true")
    p.add_argument("--own-products", choices=["none", "swiglu", "all"], default=None,
                   help="which bfloat16 products of 256 and more rows run as this package's tiled product instead of the "
                        "vendor library's: gate and up with SwiGLU inside, all of them, or none "
                        "(default: $PULSE_OWN_PRODUCTS, else none)")
    p.add_argument("--log-level", default=None, help="trace, debug, info, warn, error, critical or off "
                                                     "(default: $PULSE_LOG_LEVEL, else info); messages go to standard error")
    return p


def parse_args(argv: Optional[List[str]] = None) -> argparse.Namespace:
    """Options of the program, then those that the model's architecture declares (``engine_options`` of its
    configuration class, e.g. ``--rope-pairing`` for Qwen3): they are known only once config.json has been read."""
    parser = build_parser()
    args, rest = parser.parse_known_args(argv)
    args.model_path = args.model_opt or args.model_dir or find_default_model_path()
    args.config = None
    if rest or os.path.isfile(os.path.join(args.model_path, "config.json")):
        from .config import load_config

        args.config = load_config(args.model_path)
        extra = argparse.ArgumentParser(prog="pulse_infer", add_help=False, allow_abbrev=False)
        for field, keywords in args.config.engine_options.items():
            extra.add_argument("--" + field.replace("_", "-"), dest=field, default=None, **keywords)
        known, unknown = extra.parse_known_args(rest)
        if unknown:
            parser.error(f"unrecognized arguments: {' '.join(unknown)} (options of '{args.config.architecture}': "
                         f"{', '.join('--' + f.replace('_', '-') for f in args.config.engine_options) or 'none'})")
        args.architecture_options = {k: v for k, v in vars(known).items() if v is not None}
    else:
        args.architecture_options = {}
    return args


def parse_overrides(items: List[str]) -> dict:
    """``FIELD=VALUE`` pairs; a value is read as JSON where it is JSON (numbers, true, null), else as a string."""
    out = {}
    for item in items:
        key, sep, text = item.partition("=")
        if not sep or not key.strip():
            raise SystemExit(f"pulse_infer: --set expects FIELD=VALUE, got '{item}'")
        try:
            value = json.loads(text)
        except json.JSONDecodeError:
            value = text
        out[key.strip()] = value
    return out


def main(argv: Optional[List[str]] = None) -> int:
    args = parse_args(argv)
    model_dir = args.model_path
    if args.log_level:
        from . import log
        log.set_level(args.log_level)
    if args.own_products:
        from .parts import linear
        linear.OWN_MANY_ROWS = args.own_products
    dtype = {"bf16": "bfloat16", "f32": "float32"}.get(args.dtype, args.dtype)

    import torch

    if not torch.cuda.is_available():
        print("pulse_infer: no GPU is visible; this engine has no CPU path", file=sys.stderr)
        return 3
    from .config import load_config
    from .engine.engine import LLM
    from .sampling.params import SamplingParams

    config = args.config or load_config(model_dir)
    overrides = dict(parse_overrides(args.overrides), **args.architecture_options)
    config.apply_overrides(overrides, "the command line")
    options = dict(max_batch_size=args.max_batch, chunk_size=args.chunk, page_size=args.page_size,
                   num_pages=args.num_pages, max_num_batched_tokens=args.max_tokens, seed=args.seed,
                   extend_portions=not args.fixed_chunk)
    if args.random_weights:
        init = args.init if args.init == "fan_in" else float(args.init)
        llm = LLM.from_config_random(config, weights_seed=args.seed, init=init, dtype=dtype, device=args.device, **options)
    else:
        llm = LLM.from_pretrained(model_dir, dtype=dtype, device=args.device, config_overrides=overrides,
                                  strict=args.strict, **options)

    prompts: List[List[int]] = [[int(t) for t in s.split(",") if t.strip()] for s in args.prompt_ids]
    if args.prompt_file:
        with open(args.prompt_file) as fh:
            prompts.extend([[int(t) for t in row] for row in json.load(fh)])
    gen = torch.Generator().manual_seed(args.seed)
    for n in args.prompt_len:
        prompts.append(torch.randint(0, config.vocab_size, (n,), generator=gen).tolist())
    if not prompts:
        prompts.append(torch.randint(0, config.vocab_size, (16,), generator=gen).tolist())

    temperature = 0.0 if args.greedy else (args.temperature if args.temperature is not None else config.temperature)
    params = [SamplingParams(
        temperature=temperature,
        top_k=args.top_k if args.top_k is not None else config.top_k,
        top_p=args.top_p if args.top_p is not None else config.top_p,
        presence_penalty=args.presence_penalty,
        seed=None if args.sample_seed is None else args.sample_seed + i,
        ignore_eos=args.ignore_eos or not config.eos_token_ids) for i in range(len(prompts))]

    torch.cuda.synchronize()
    t0 = time.perf_counter()
    outputs = llm.generate(prompts, max_new_tokens=args.max_new_tokens, sampling=params)
    torch.cuda.synchronize()
    seconds = time.perf_counter() - t0
    for i, (prompt, out) in enumerate(zip(prompts, outputs)):
        print(json.dumps({"request": i, "prompt_len": len(prompt), "output_ids": out}))
    total = sum(len(o) for o in outputs)
    print(f"Generated {total} tokens in {seconds:.3f} s ({total / seconds if seconds > 0 else 0.0:.2f} tokens/s)")
    if args.stats:
        s = llm.engine.get_stats()
        print(json.dumps({"steps": s.num_steps, "preemptions": s.num_preemptions, "tokens_computed": s.tokens_computed,
                          "tokens_generated": s.tokens_generated, "pages_high_water": s.pages_high_water}))
    return 0


if __name__ == "__main__":
    sys.exit(main())
