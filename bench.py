#!/usr/bin/env python3
"""Decode and prefill throughput of the Qwen3-8B shape on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A "step" is one decode step of the whole batch, as the engine's own serving loop
runs it (``ContinuousBatchEngine.run_until_complete``): the scheduler's decision,
the step function on one token per request, the argmax kernel, and the tokens'
way back to the host and into the next step, which is queued while this one is
computed.  Weights are random (made on the GPU), token ids are seeded synthetic
ids, and for the fixed-context points the requests are admitted with the context
before the timed steps counting as computed, over a cache filled with random
keys and values (its content does not change the work of a decode step).  Every
point is timed three times and the median is reported; ``value`` is the batch
over the median step time of ``--steps`` steps at contexts ending at
``--context``.  ``trajectory`` is the workload as stated, end to end: every
request a prompt of ``--prefill-tokens`` tokens and as many greedy tokens;
``serving`` is continuous batching of 32 requests with seeded prompt lengths.
Bytes and arithmetic of the rooflines come from the model's own description
(``models/cost.py``), not from formulas of one architecture.
``--kernels`` prints where one decode step's time goes, entry point by entry
point.  Prints one JSON line.
"""
from __future__ import annotations

import argparse
import json
import os
import statistics
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
    p.add_argument("--workload", choices=["decode", "serving", "long-prompt"], default="decode",
                   help="decode: fixed batch at a fixed context; serving: continuous batching of requests with "
                        "seeded prompt lengths, chunked prefill mixed with decoding; long-prompt: one prompt of "
                        "--prompt-tokens tokens in portions of --chunk tokens")
    p.add_argument("--prompt-tokens", type=int, default=16384, help="long-prompt: length of the prompt")
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
    p.add_argument("--no-points", action="store_true",
                   help="skip the further points (batch 1 / 16 / 32 / 64, batch 8 at a context of 16,384, prompts of "
                        "512 and 8,192 tokens)")
    p.add_argument("--more-points", action="store_true",
                   help="points that need a larger cache pool: batch 8 at contexts of 1,024 and 40,000, batch 128")
    p.add_argument("--no-serving", action="store_true", help="skip the serving workload at the end of the default run")
    p.add_argument("--no-prefill", action="store_true")
    p.add_argument("--no-trajectory", action="store_true",
                   help="skip the end-to-end run (prompt + as many greedy tokens per request through the scheduler)")
    p.add_argument("--trajectory-tokens", type=int, default=None,
                   help="greedy tokens per request of the end-to-end run (default: --prefill-tokens)")
    p.add_argument("--runs", type=int, default=3, help="timed runs per point; the median is reported")
    p.add_argument("--kernels", action="store_true",
                   help="print where one decode step's time goes by entry point (eager, GPU events) and exit")
    p.add_argument("--seed", type=int, default=0)
    return p.parse_args()


def trajectory(args, cfg, model, batch: int, prompt_tokens: int, new_tokens: int) -> dict:
    """The stated workload end to end: ``batch`` requests of ``prompt_tokens`` tokens each, ``new_tokens`` greedy
    tokens each, through scheduler, step function and sampler (prompts in portions of 512 under a budget of 2,048
    tokens a step).  Returns output tokens a second over the whole run and over its decoding steps alone."""
    import torch

    from pulse_infer_amd.engine.engine import ContinuousBatchEngine
    from pulse_infer_amd.sampling.params import SamplingParams

    gen = torch.Generator().manual_seed(args.seed + 17)
    pages = batch * ((prompt_tokens + new_tokens + args.page_size - 1) // args.page_size + 1)
    engine = ContinuousBatchEngine(model, max_batch_size=batch, chunk_size=512, page_size=args.page_size,
                                   num_pages=pages, max_sequences=batch, max_num_batched_tokens=2048, seed=args.seed)
    for _ in range(batch):
        engine.add_request(torch.randint(0, cfg.vocab_size, (prompt_tokens,), generator=gen).tolist(), new_tokens,
                           SamplingParams(ignore_eos=True))
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    # the prompts step by step (so that the moment the last one is through can be told), then the engine's own loop
    while engine.scheduler.has_work() and any(r.is_prefill for r in engine.scheduler.running + list(engine.scheduler.waiting)):
        if engine.step().empty():
            break
    torch.cuda.synchronize()
    t_decode = time.perf_counter()
    steps_before = engine.get_stats().num_steps
    engine.run_until_complete()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    stats = engine.get_stats()
    total = stats.tokens_generated
    assert total == batch * new_tokens, (total, batch, new_tokens)
    decode_s = t1 - t_decode
    decode_steps = stats.num_steps - steps_before
    del engine
    torch.cuda.empty_cache()
    return {"value": round(total / (t1 - t0), 2), "decode_value": round(batch * decode_steps / decode_s, 2),
            "batch": batch, "prompt_tokens": prompt_tokens, "new_tokens": new_tokens, "seconds": round(t1 - t0, 3),
            "decode_ms_per_step": round(decode_s * 1e3 / max(1, decode_steps), 4), "steps": stats.num_steps}


def serving(args, cfg, model, full_layers: int) -> dict:
    """Continuous batching end to end: every request through the scheduler, the step function and the sampler.
    Returns the record of the run (the whole JSON line of ``--workload serving``)."""
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
    # one short request before the clock starts: the first step of a process loads the libraries and their kernels
    # (0.4 s), which a server has behind it; the recordings of the run's own steps stay inside the timed part
    engine.add_request(torch.randint(0, cfg.vocab_size, (args.chunk + 8,), generator=gen).tolist(), 2,
                       SamplingParams(temperature=args.temperature, seed=args.seed, ignore_eos=True))
    engine.run_until_complete()
    before = engine.get_stats()
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
    stats.num_steps -= before.num_steps
    stats.tokens_computed -= before.tokens_computed
    total = stats.tokens_generated - before.tokens_generated
    record = {
        "metric": f"qwen3_{args.model}_serving_output_tokens_per_s", "value": round(total / seconds, 2), "unit": "tokens/s",
        "n_gpus": 1, "steps": stats.num_steps, "warmup": before.num_steps, "ms_per_step": round(seconds * 1e3 / max(1, stats.num_steps), 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"model": f"Qwen3-{args.model.upper()} shape, random weights", "global_batch": args.requests,
                   "seq_len": hi + args.output_tokens, "parallelism": "single GPU", "layers": args.layers,
                   "layers_full_model": full_layers, "requests": args.requests, "prompt_min": lo, "prompt_max": hi,
                   "output_tokens": args.output_tokens, "chunk": args.chunk, "token_budget": engine.scheduler.max_num_batched_tokens,
                   "temperature": args.temperature,
                   "prompt_tokens": sum(lengths), "preemptions": stats.num_preemptions},
        "seconds": round(seconds, 3), "tokens_computed": stats.tokens_computed,
        "steps_recorded": engine.runner.graph_records, "steps_replayed": engine.runner.graph_replays}
    del engine
    torch.cuda.empty_cache()
    return record


def long_prompt(args, cfg, model, full_layers: int) -> int:
    """One prompt of ``--prompt-tokens`` tokens computed in portions of ``--chunk`` tokens (every portion attends to
    all the keys before it: few workgroups with long walks, the split prompt-portion kernel's case)."""
    import torch

    from pulse_infer_amd.engine.runner import ModelRunner, StepEntry
    from pulse_infer_amd.models.cost import step_cost

    tokens, chunk, page = args.prompt_tokens, args.chunk, args.page_size
    runner = ModelRunner(model, page_size=page, num_pages=(tokens + page - 1) // page + 1, max_requests=2)
    ids = torch.randint(0, cfg.vocab_size, (tokens,), generator=torch.Generator().manual_seed(args.seed)).tolist()
    element = 2 if args.dtype == "bfloat16" else 4
    spec = cfg.model_spec()
    flops = sum(step_cost(spec, [(p, min(chunk, tokens - p))], 0, element, element).flops for p in range(0, tokens, chunk))
    times = []
    for r in range(args.runs + 1):          # the first run warms up
        runner.add_request("p")
        runner.reserve("p", tokens)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for p in range(0, tokens, chunk):
            part = ids[p:p + chunk]
            runner.step([StepEntry("p", part, [len(part) - 1] if p + chunk >= tokens else [])])
        torch.cuda.synchronize()
        if r > 0:
            times.append(time.perf_counter() - t0)
        runner.free_request("p")
    seconds = statistics.median(times)
    peak = PEAK_FLOPS["bf16" if args.dtype == "bfloat16" else "fp32"]
    steps = (tokens + chunk - 1) // chunk
    print(json.dumps({
        "metric": f"qwen3_{args.model}_long_prompt_tokens_per_s", "value": round(tokens / seconds, 1), "unit": "tokens/s",
        "n_gpus": 1, "steps": steps, "warmup": steps, "ms_per_step": round(seconds * 1e3 / steps, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16" if args.dtype == "bfloat16" else "fp32", "data": "synthetic",
        "config": {"model": f"Qwen3-{args.model.upper()} shape, random weights", "global_batch": 1, "seq_len": tokens,
                   "parallelism": "single GPU", "layers": args.layers, "layers_full_model": full_layers, "chunk": chunk},
        "runs": args.runs, "seconds": round(seconds, 4), "frac_of_peak": round(flops / seconds / peak, 4)}))
    return 0


def main() -> int:
    args = parse_args()
    if args.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not supported")
        return 2

    import torch

    sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
    from pulse_infer_amd.config import Qwen3Config
    from pulse_infer_amd.engine.engine import ContinuousBatchEngine
    from pulse_infer_amd.models.causal_lm import expected_tensors
    from pulse_infer_amd.models.factory import build_model
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
        print(json.dumps(serving(args, cfg, model, full_layers)))
        return 0
    if args.workload == "long-prompt":
        return long_prompt(args, cfg, model, full_layers)

    from pulse_infer_amd.models.cost import step_cost

    spec = cfg.model_spec()
    peak_flops = PEAK_FLOPS["bf16" if args.dtype == "bfloat16" else "fp32"]
    # (batch, context) of every decode point, prompt lengths of every prefill point
    decode_points, prefill_points = {}, {}
    if not args.no_points:
        decode_points = {"decode_b1": (1, args.context), "decode_b64": (64, args.context),
                         "decode_b16": (16, args.context), "decode_b32": (32, args.context),
                         "decode_b8_ctx16384": (8, 16384)}
        prefill_points = {"prefill_512": 512, "prefill_8192": 8192}
    if args.more_points:
        for ctx in (1024, 40000):
            decode_points[f"decode_b8_ctx{ctx}"] = (8, ctx)
        decode_points["decode_b128"] = (128, args.context)
    shapes = [(args.batch, args.context)] + list(decode_points.values())
    max_batch = max(b for b, _ in shapes)
    page = args.page_size
    prompts = [args.prefill_tokens] + list(prefill_points.values())
    pool = max([b * ((c + page - 1) // page + 1) for b, c in shapes] + [(n + page - 1) // page + 1 for n in prompts])
    # every point runs through the engine's own serving loop; a prompt that has a step to itself runs in one portion
    engine = ContinuousBatchEngine(model, max_batch_size=max_batch, chunk_size=512, page_size=page, num_pages=pool,
                                   max_sequences=max_batch, max_num_batched_tokens=max(prompts), seed=args.seed)
    runner = engine.runner
    for g in runner.cache.groups:  # a cache that looks computed: random keys and values
        for t in g.spec.tensors(g.storage):
            t.normal_(0.0, 1.0)
    gen = torch.Generator().manual_seed(args.seed)
    greedy = SamplingParams(ignore_eos=True)

    def decode_run(batch: int, context: int, steps: int, warmup: int, runs: int):
        """``runs`` timings of ``steps`` decode steps of ``batch`` requests whose contexts end at ``context`` (every run
        walks the same contexts), through ``run_until_complete``.  Returns (median seconds a step by the host's clock
        between two synchronisations, the same by GPU events, every run's host figure)."""
        start = context - (steps + warmup)
        if start < 1:
            raise SystemExit(f"a context of {context} is too short for {steps} + {warmup} steps")
        host, events = [], []
        for _ in range(runs):
            for _ in range(batch):
                rid = engine.add_request(torch.randint(0, cfg.vocab_size, (start + 1,), generator=gen).tolist(),
                                         steps + warmup, greedy)
                engine.admit_as_computed(rid, start)        # the context so far counts as computed
            if warmup:
                assert engine.run_until_complete(max_steps=warmup) == warmup
            first, last = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            first.record()
            ran = engine.run_until_complete()
            last.record()
            torch.cuda.synchronize()
            assert ran == steps and not engine.scheduler.has_work(), (ran, steps)
            host.append((time.perf_counter() - t0) / steps)
            events.append(first.elapsed_time(last) * 1e-3 / steps)
        return statistics.median(host), statistics.median(events), host

    def decode_bytes(batch: int, context: int, steps: int) -> float:
        """What a decode step of the timed run has to read: every weight once and the live requests' cache, at the
        run's mean context."""
        cost = step_cost(spec, [(int(context - steps / 2.0) - 1, 1)] * batch, batch, element, element)
        return cost.weight_bytes + cost.cache_bytes

    def prefill_run(tokens: int, runs: int):
        ids = torch.randint(0, cfg.vocab_size, (tokens,), generator=gen).tolist()
        times = []
        for r in range(runs + 1):  # the first run warms up
            engine.add_request(ids, 1, greedy)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            ran = engine.run_until_complete()    # one step of the whole prompt, its last row's token back on the host
            torch.cuda.synchronize()
            seconds = time.perf_counter() - t0
            assert ran == 1, ran
            if r > 0:
                times.append(seconds)
        return statistics.median(times)

    if args.kernels:
        return kernel_table(args, cfg, runner, engine.sampler, gen)

    step_s, step_gpu_s, all_runs = decode_run(args.batch, args.context, args.steps, args.warmup, args.runs)
    value = args.batch / step_s
    achieved = decode_bytes(args.batch, args.context, args.steps) / step_s / 1e9
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
        "runs": args.runs, "ms_per_step_runs": [round(t * 1e3, 4) for t in all_runs],
        "ms_per_step_gpu_events": round(step_gpu_s * 1e3, 4),
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4)},
    }
    if not args.no_prefill:
        pf_s = prefill_run(args.prefill_tokens, args.runs)
        flops = step_cost(spec, [(0, args.prefill_tokens)], 1, element, element).flops
        result["prefill"] = {"value": round(args.prefill_tokens / pf_s, 1), "tokens": args.prefill_tokens,
                             "ms": round(pf_s * 1e3, 3), "frac": round(flops / pf_s / peak_flops, 4)}
    if decode_points or prefill_points:
        points, fracs = {}, {}
        for name, (b, ctx) in decode_points.items():
            steps = max(8, min(args.steps, 32))
            t, _, _ = decode_run(b, ctx, steps, min(args.warmup, 4), args.runs)
            points[name] = round(b / t, 2)
            fracs[name] = round(decode_bytes(b, ctx, steps) / t / 1e9 / HBM_PEAK_GBS, 4)
        for name, n in prefill_points.items():
            t = prefill_run(n, args.runs)
            points[name] = round(n / t, 1)
            fracs[name] = round(step_cost(spec, [(0, n)], 1, element, element).flops / t / peak_flops, 4)
        result["points"] = points
        result["points_frac"] = fracs     # of 8 TB/s for decoding, of the dense matrix-core peak for prompts
    del runner, engine
    torch.cuda.empty_cache()
    if not args.no_trajectory:
        new_tokens = args.trajectory_tokens or args.prefill_tokens
        result["trajectory"] = trajectory(args, cfg, model, args.batch, args.prefill_tokens, new_tokens)
    if not args.no_serving:
        record = serving(args, cfg, model, full_layers)
        result["serving"] = {"value": record["value"], "unit": "output tokens/s", "requests": args.requests,
                             "prompt_min": args.prompt_range[0], "prompt_max": args.prompt_range[1],
                             "output_tokens": args.output_tokens, "chunk": args.chunk,
                             "token_budget": record["config"]["token_budget"], "temperature": args.temperature,
                             "seconds": record["seconds"], "steps": record["steps"],
                             "preemptions": record["config"]["preemptions"]}
    print(json.dumps(result))
    return 0


def kernel_table(args, cfg, runner, sampler, gen) -> int:
    """Where the time of one decode step goes, by entry point: every launch of an eager step is bracketed by GPU
    events (``ops/timing.py``), over a few steps; printed as a table, most expensive first."""
    import torch

    from pulse_infer_amd.engine.runner import StepEntry
    from pulse_infer_amd.ops import timing
    from pulse_infer_amd.sampling.params import SamplingParams

    runner.use_graphs = False
    batch, context, steps = args.batch, args.context, 6
    names = [f"k{i}" for i in range(batch)]
    for n in names:
        runner.add_request(n)
        runner.reserve(n, context)
        runner.cache.advance(n, context - steps - 2)
    tokens = torch.randint(0, cfg.vocab_size, (batch,), generator=gen).tolist()
    slots = [runner.cache.slot_of(n) for n in names]

    def one_step(toks):
        logits = runner.step([StepEntry(n, [t], [0]) for n, t in zip(names, toks)])
        return sampler.sample(logits, [SamplingParams()] * batch, slots, [0] * batch, [0] * batch)

    for _ in range(2):
        tokens = one_step(tokens)
    with timing.record() as table:
        for _ in range(steps):
            tokens = one_step(tokens)
    print(f"# decode step, batch {batch}, contexts ending at {context}, {args.layers} layers, eager launches, "
          f"mean of {steps} steps")
    print(table.format(per=steps))
    return 0


if __name__ == "__main__":
    sys.exit(main())
