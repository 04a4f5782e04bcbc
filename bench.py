#!/usr/bin/env python3
"""Decode and prefill throughput of the Qwen3-8B shape on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A "step" is one decode step of the whole batch: the step function on one token
per request, the argmax kernel, and the tokens' way back to the host and into
the next step.  Weights are random (made on the GPU), token ids are seeded
synthetic ids, and the cache of the context before the timed steps is filled
with random keys and values instead of being computed (its content does not
change the work of a decode step).  Prints one JSON line.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E, published
PEAK_FLOPS = {"bf16": 2.5e15, "fp16": 2.5e15, "fp8": 5.0e15, "fp32": 157.3e12}  # dense MFMA, published

QWEN3_8B = dict(
    architectures=["Qwen3ForCausalLM"], vocab_size=151936, hidden_size=4096, intermediate_size=12288,
    num_hidden_layers=36, num_attention_heads=32, num_key_value_heads=8, head_dim=128,
    max_position_embeddings=40960, rms_norm_eps=1e-6, rope_theta=1e6, tie_word_embeddings=False,
    torch_dtype="bfloat16", use_sliding_window=False)
# the other shapes of the benchmark list: selected with --model, never the default
SHAPES = {
    "8b": QWEN3_8B,
    "14b": dict(QWEN3_8B, hidden_size=5120, intermediate_size=17408, num_hidden_layers=40, num_attention_heads=40),
    "32b": dict(QWEN3_8B, hidden_size=5120, intermediate_size=25600, num_hidden_layers=64, num_attention_heads=64),
}


def parse_args() -> argparse.Namespace:
    p = argparse.ArgumentParser()
    p.add_argument("--gpus", type=int, default=1)
    p.add_argument("--steps", type=int, default=64)
    p.add_argument("--warmup", type=int, default=8)
    p.add_argument("--batch", type=int, default=8)
    p.add_argument("--context", type=int, default=4096, help="context length the timed decode steps end at")
    p.add_argument("--model", choices=sorted(SHAPES), default="8b", help="layer sizes: Qwen3-8B (the default), 14B or 32B")
    p.add_argument("--layers", type=int, default=None, help="fewer layers than the model has, if memory or time needs it")
    p.add_argument("--workload", choices=["decode", "serving"], default="decode",
                   help="decode: fixed batch at a fixed context; serving: continuous batching of requests with "
                        "seeded prompt lengths, chunked prefill mixed with decoding")
    p.add_argument("--requests", type=int, default=32, help="serving: number of requests")
    p.add_argument("--prompt-range", type=int, nargs=2, default=[128, 2048], help="serving: prompt lengths drawn from [lo, hi]")
    p.add_argument("--output-tokens", type=int, default=256, help="serving: tokens generated per request")
    p.add_argument("--chunk", type=int, default=512, help="serving: longest prompt portion in a step")
    p.add_argument("--token-budget", type=int, default=None,
                   help="serving: most tokens a step computes (default: four portions)")
    p.add_argument("--temperature", type=float, default=0.7, help="serving: sampling temperature")
    p.add_argument("--prefill-tokens", type=int, default=2048)
    p.add_argument("--page-size", type=int, default=16)
    p.add_argument("--dtype", choices=["bfloat16", "float32"], default="bfloat16")
    p.add_argument("--no-points", action="store_true", help="skip the batch 1 and batch 64 points")
    p.add_argument("--no-prefill", action="store_true")
    p.add_argument("--seed", type=int, default=0)
    return p.parse_args()


def weight_bytes(cfg, element_size: int) -> int:
    """Bytes of every weight a decode step reads once: all layers and the head."""
    h, i, d = cfg.hidden_size, cfg.intermediate_size, cfg.head_dim
    nq, nkv = cfg.num_attention_heads, cfg.num_key_value_heads
    per_layer = (nq + 2 * nkv) * d * h + h * nq * d + 2 * i * h + h * i + 2 * h + 2 * d
    return (per_layer * cfg.num_hidden_layers + cfg.vocab_size * h + h) * element_size


def kv_bytes_per_token(cfg, element_size: int) -> int:
    return 2 * cfg.num_hidden_layers * cfg.num_key_value_heads * cfg.head_dim * element_size


def prefill_flops(cfg, tokens: int) -> float:
    """Multiply-adds of one prompt of ``tokens`` tokens, times two; logits for the last row only."""
    h, i, d = cfg.hidden_size, cfg.intermediate_size, cfg.head_dim
    nq, nkv = cfg.num_attention_heads, cfg.num_key_value_heads
    linear = (nq + 2 * nkv) * d * h + h * nq * d + 3 * i * h
    attn = 4 * nq * d * tokens * (tokens + 1) / 2          # QK^T and PV over the causal triangle
    return cfg.num_hidden_layers * (2.0 * tokens * linear + attn) + 2.0 * cfg.vocab_size * h


def serving(args, cfg, model, full_layers: int) -> int:
    """Continuous batching end to end: every request through the scheduler, the step function and the sampler."""
    import torch

    from pulse_infer_amd.engine.engine import ContinuousBatchEngine
    from pulse_infer_amd.sampling.params import SamplingParams

    gen = torch.Generator().manual_seed(args.seed)
    lo, hi = args.prompt_range
    lengths = torch.randint(lo, hi + 1, (args.requests,), generator=gen).tolist()
    per_request = hi + args.output_tokens + args.page_size
    pages = args.requests * ((per_request + args.page_size - 1) // args.page_size)
    engine = ContinuousBatchEngine(model, max_batch_size=args.requests, chunk_size=args.chunk, page_size=args.page_size,
                                   num_pages=pages, max_sequences=args.requests,
                                   max_num_batched_tokens=args.token_budget or 4 * args.chunk, seed=args.seed)
    for i, n in enumerate(lengths):
        prompt = torch.randint(0, cfg.vocab_size, (n,), generator=gen).tolist()
        engine.add_request(prompt, args.output_tokens,
                           SamplingParams(temperature=args.temperature, seed=args.seed + i, ignore_eos=True))
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    engine.run_until_complete()
    torch.cuda.synchronize()
    seconds = time.perf_counter() - t0
    stats = engine.get_stats()
    total = stats.tokens_generated
    print(json.dumps({
        "metric": f"qwen3_{args.model}_serving_output_tokens_per_s", "value": round(total / seconds, 2), "unit": "tokens/s",
        "n_gpus": 1, "steps": stats.num_steps, "warmup": 0, "ms_per_step": round(seconds * 1e3 / max(1, stats.num_steps), 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"model": f"Qwen3-{args.model.upper()} shape, random weights", "global_batch": args.requests,
                   "seq_len": hi + args.output_tokens, "parallelism": "single GPU", "layers": args.layers,
                   "layers_full_model": full_layers, "requests": args.requests, "prompt_min": lo, "prompt_max": hi,
                   "output_tokens": args.output_tokens, "chunk": args.chunk, "token_budget": engine.scheduler.max_num_batched_tokens,
                   "temperature": args.temperature,
                   "prompt_tokens": sum(lengths), "preemptions": stats.num_preemptions},
        "seconds": round(seconds, 3), "tokens_computed": stats.tokens_computed}))
    return 0


def main() -> int:
    args = parse_args()
    if args.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not supported")
        return 2

    import torch

    sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
    from pulse_infer_amd.config import Qwen3Config
    from pulse_infer_amd.engine.runner import ModelRunner, StepEntry
    from pulse_infer_amd.models.causal_lm import expected_tensors
    from pulse_infer_amd.models.factory import build_model
    from pulse_infer_amd.sampling.sampler import Sampler
    from pulse_infer_amd.sampling.params import SamplingParams
    from pulse_infer_amd.weights.random_init import RandomSource

    torch.backends.cuda.matmul.allow_tf32 = False
    device = torch.device("cuda:0")
    shape = SHAPES[args.model]
    full_layers = shape["num_hidden_layers"]
    if args.layers is None:
        args.layers = full_layers
    cfg_dict = dict(shape, num_hidden_layers=args.layers)
    cfg = Qwen3Config.from_dict(cfg_dict, "<bench>")
    element = 2 if args.dtype == "bfloat16" else 4
    source = RandomSource(expected_tensors(cfg.model_spec()), args.seed, 0.02, torch.bfloat16, device=device)
    model = build_model(cfg, source, mode=args.dtype, device=device)

    if args.workload == "serving":
        return serving(args, cfg, model, full_layers)

    batches = [args.batch] if args.no_points else sorted({1, args.batch, 64})
    max_batch = max(batches)
    pages_per_request = (args.context + args.page_size - 1) // args.page_size + 1
    prefill_pages = (args.prefill_tokens + args.page_size - 1) // args.page_size + 1
    runner = ModelRunner(model, page_size=args.page_size, num_pages=max(max_batch * pages_per_request, prefill_pages),
                         max_requests=max_batch + 1)
    for g in runner.cache.groups:  # a cache that looks computed: random keys and values
        g.keys.normal_(0.0, 1.0)
        g.values.normal_(0.0, 1.0)
    sampler = Sampler(cfg.vocab_size, max_batch + 1, device)
    gen = torch.Generator().manual_seed(args.seed)

    def decode_run(batch: int, steps: int, warmup: int):
        """Time ``steps`` decode steps of ``batch`` requests whose contexts end at ``args.context``."""
        start = args.context - (steps + warmup)
        if start < 1:
            raise SystemExit(f"--context {args.context} is too short for {steps} + {warmup} steps")
        names = [f"d{batch}_{i}" for i in range(batch)]
        for n in names:
            runner.add_request(n)
            runner.reserve(n, args.context)
            runner.cache.advance(n, start)          # the context so far counts as computed
        tokens = torch.randint(0, cfg.vocab_size, (batch,), generator=gen).tolist()
        greedy = [SamplingParams()] * batch
        slots = [runner.cache.slot_of(n) for n in names]

        def one_step(toks):
            logits = runner.step([StepEntry(n, [t], [0]) for n, t in zip(names, toks)])
            return sampler.sample(logits, greedy, slots, [0] * batch, [0] * batch)

        for _ in range(warmup):
            tokens = one_step(tokens)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            tokens = one_step(tokens)
        torch.cuda.synchronize()
        seconds = time.perf_counter() - t0
        for n in names:
            runner.free_request(n)
        return seconds / steps

    def prefill_run(tokens: int, repeats: int = 3):
        ids = torch.randint(0, cfg.vocab_size, (tokens,), generator=gen).tolist()
        best = None
        for r in range(repeats + 1):  # the first run warms up
            runner.add_request("p")
            runner.reserve("p", tokens)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            logits = runner.step([StepEntry("p", ids, [tokens - 1])])
            sampler.sample(logits, [SamplingParams()], [0], [0], [0])
            torch.cuda.synchronize()
            seconds = time.perf_counter() - t0
            runner.free_request("p")
            if r > 0:
                best = seconds if best is None else min(best, seconds)
        return best

    step_s = decode_run(args.batch, args.steps, args.warmup)
    value = args.batch / step_s
    mean_ctx = args.context - args.steps / 2.0
    step_bytes = weight_bytes(cfg, element) + args.batch * mean_ctx * kv_bytes_per_token(cfg, element)
    achieved = step_bytes / step_s / 1e9
    result = {
        "metric": f"qwen3_{args.model}_decode_tokens_per_s_batch{args.batch}", "value": round(value, 2), "unit": "tokens/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(step_s * 1e3, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16" if args.dtype == "bfloat16" else "fp32", "data": "synthetic",
        "config": {
            "model": f"Qwen3-{args.model.upper()} shape, random weights", "global_batch": args.batch, "seq_len": args.context,
            "parallelism": "single GPU", "layers": args.layers, "layers_full_model": full_layers,
            "hidden_size": cfg.hidden_size, "intermediate_size": cfg.intermediate_size,
            "num_attention_heads": cfg.num_attention_heads, "num_key_value_heads": cfg.num_key_value_heads,
            "head_dim": cfg.head_dim, "vocab_size": cfg.vocab_size, "rope_theta": cfg.rope_theta,
            "rms_norm_eps": cfg.rms_norm_eps, "tie_word_embeddings": cfg.tie_word_embeddings,
            "page_size": args.page_size, "prefill_tokens": args.prefill_tokens,
        },
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4)},
    }
    if not args.no_prefill:
        pf_s = prefill_run(args.prefill_tokens)
        peak = PEAK_FLOPS["bf16" if args.dtype == "bfloat16" else "fp32"]
        result["prefill"] = {"value": round(args.prefill_tokens / pf_s, 1), "tokens": args.prefill_tokens,
                             "ms": round(pf_s * 1e3, 3),
                             "frac": round(prefill_flops(cfg, args.prefill_tokens) / pf_s / peak, 4)}
    if not args.no_points:
        points = {}
        for b in (1, 64):
            steps = max(8, min(args.steps, 32))
            points[f"decode_b{b}"] = round(b / decode_run(b, steps, min(args.warmup, 4)), 2)
        result["points"] = points
    print(json.dumps(result))
    return 0


if __name__ == "__main__":
    sys.exit(main())
