"""A sweep over seeded random configurations of the architecture (head sizes in steps of 16, any grouping of heads,
windows on some layers, widths that are multiples of 128 so that every product kernel has its turn, vocabularies that
are no power of two, several page sizes): the engine whole, with the last 32 tokens one by one and in portions of
17 to 150 tokens, against the plain implementation in 32-bit and in bfloat16; and continuous batching with small
portions and a pool so tight that requests are preempted, in 32-bit against each request alone and against the plain
implementation's greedy choice."""
import random

import pytest
import torch

from conftest import token_ids
from plain.qwen3_plain import PlainQwen3
from test_gpu_model import TOL, SPLIT_TOL, close, run_alone

pytestmark = pytest.mark.gpu


def random_config(rng, hidden_choices, max_positions=1024):
    """(config.json's keys, options of the engine): windows on the later layers of some configurations are the latter."""
    d = rng.choice([16, 32, 48, 64, 80, 96, 112, 128])
    nkv = rng.choice([1, 2, 3, 4])
    group = rng.choice([1, 2, 3, 4, 5, 7, 8])
    window = rng.choice([None, None, 20, 70])
    cfg = dict(architectures=["Qwen3ForCausalLM"], model_type="qwen3", vocab_size=rng.choice([300, 1000, 2053]),
               hidden_size=rng.choice(hidden_choices), intermediate_size=rng.choice([128, 160, 256, 1056]),
               num_hidden_layers=rng.choice([1, 2, 3]), num_attention_heads=nkv * group, num_key_value_heads=nkv,
               head_dim=d, max_position_embeddings=max_positions, rms_norm_eps=rng.choice([1e-6, 1e-5]),
               rope_theta=rng.choice([1e4, 1e6]), tie_word_embeddings=rng.random() < 0.5, torch_dtype="bfloat16",
               attention_bias=False, hidden_act="silu", use_sliding_window=False)
    options = None
    if window is not None:
        first = rng.choice([0, 1])
        options = {"layer_windows": [window if i >= first else None for i in range(cfg["num_hidden_layers"])]}
    return cfg, options


@pytest.mark.parametrize("seed", range(8))
def test_random_configurations_whole_tail_and_portions(tmp_path, seed):
    if not torch.cuda.is_available():
        pytest.skip("no GPU visible")
    from pulse_infer_amd.config import Qwen3Config
    from pulse_infer_amd.engine.runner import ModelRunner
    from pulse_infer_amd.models.factory import load_model
    from pulse_infer_amd.weights import write_model_folder

    rng = random.Random(1000 + seed)
    cfg, options = random_config(rng, [128, 256, 384, 1024])
    windows = (options or {}).get("layer_windows")
    page, length = rng.choice([16, 32, 64]), rng.choice([90, 200, 333])
    folder = write_model_folder(Qwen3Config.from_dict(cfg), str(tmp_path / "m"), seed=seed)
    ids = token_ids(cfg["vocab_size"], length, seed=seed)
    want = PlainQwen3.from_folder(folder, windows=windows).logits(ids)
    what = f"{cfg} {options} page {page} length {length}"
    for dtype in ("float32", "bfloat16"):
        _, model = load_model(folder, mode=dtype, config_overrides=options)
        runner = ModelRunner(model, page_size=page, num_pages=(length + page - 1) // page + 2, max_requests=2)
        whole = run_alone(runner, ids, [length])
        close(whole, want, dtype, f"whole: {what}")
        tail = run_alone(runner, ids, [length - 32] + [1] * 32)
        close(tail, want, dtype, f"tail: {what}")
        close(tail, whole, dtype, f"tail against whole: {what}", SPLIT_TOL)
        cuts, left, sizes = [], length, [40, 2, 17, 64, 3, 100, 5, 19, 150]
        while left:
            n = min(sizes[len(cuts) % len(sizes)], left)
            if left - n == 1:
                n += 1
            cuts.append(n)
            left -= n
        portions = run_alone(runner, ids, cuts)
        close(portions, want, dtype, f"portions {cuts}: {what}")
        close(portions, whole, dtype, f"portions against whole: {what}", SPLIT_TOL)
        del runner, model
    torch.cuda.empty_cache()


@pytest.mark.parametrize("seed", range(4))
def test_random_configurations_continuous_batching_and_preemption(tmp_path, seed):
    """In 32-bit the greedy choice does not depend on the batch: what a request generates beside others, in small
    portions, and after being preempted and recomputed, is what it generates alone and what the plain
    implementation generates."""
    if not torch.cuda.is_available():
        pytest.skip("no GPU visible")
    from pulse_infer_amd import LLM
    from pulse_infer_amd.config import Qwen3Config
    from pulse_infer_amd.weights import write_model_folder

    rng = random.Random(2000 + seed)
    cfg, options = random_config(rng, [128, 256], max_positions=512)
    windows = (options or {}).get("layer_windows")
    page = rng.choice([16, 32])
    folder = write_model_folder(Qwen3Config.from_dict(cfg), str(tmp_path / "m"), seed=50 + seed)
    prompts = [token_ids(cfg["vocab_size"], rng.choice([1, 5, 18, 40, 77]), seed=seed * 10 + i)
               for i in range(rng.choice([3, 5, 7]))]
    new = rng.choice([8, 20])
    make = lambda **kw: LLM.from_pretrained(folder, dtype="float32", page_size=page, config_overrides=options, **kw)
    alone = [make(max_batch_size=1, chunk_size=256, num_pages=64).generate([p], max_new_tokens=new, ignore_eos=True)[0]
             for p in prompts]
    plain = PlainQwen3.from_folder(folder, windows=windows)
    assert alone[:2] == [plain.greedy(p, new) for p in prompts[:2]]
    roomy = make(max_batch_size=4, chunk_size=rng.choice([8, 16, 50]), num_pages=64,
                 max_num_batched_tokens=rng.choice([24, 64]))
    assert roomy.generate(prompts, max_new_tokens=new, ignore_eos=True) == alone
    need = max((len(p) + new + page - 1) // page for p in prompts)
    tight = make(max_batch_size=4, chunk_size=16, num_pages=need + 2)       # room for little more than one request
    assert tight.generate(prompts, max_new_tokens=new, ignore_eos=True) == alone
    tight.engine.runner.cache.check()


@pytest.mark.parametrize("seed", range(6))
def test_random_workloads_through_the_loop_one_step_ahead_and_step_by_step(tmp_path, seed):
    """Random requests (sampling options of every kind, seeded; lengths from none to thirty; end-of-sequence ids that
    are drawn often; banned ids; a pool that holds little more than the longest request, so requests are preempted,
    some of them while their last token is still on the device) through the serving loop that queues a step ahead
    and through the loop that waits for every step, in 32-bit: the same tokens, finish reasons and results."""
    if not torch.cuda.is_available():
        pytest.skip("no GPU visible")
    from pulse_infer_amd import SamplingParams
    from pulse_infer_amd.config import Qwen3Config
    from pulse_infer_amd.engine.engine import ContinuousBatchEngine
    from pulse_infer_amd.models.factory import load_model
    from pulse_infer_amd.weights import write_model_folder

    rng = random.Random(5000 + seed)
    cfg, options = random_config(rng, [64, 128], max_positions=512)
    vocab = cfg["vocab_size"]
    folder = write_model_folder(Qwen3Config.from_dict(cfg), str(tmp_path / "m"), seed=80 + seed)
    _, model = load_model(folder, mode="float32", config_overrides=options)
    page = rng.choice([8, 16])
    count = rng.randint(4, 12)
    prompts = [token_ids(vocab, rng.randint(1, 60), seed=seed * 100 + i) for i in range(count)]
    lengths = [rng.randint(0, 30) for _ in range(count)]
    eos = rng.sample(range(vocab), k=rng.choice([0, vocab // 12, vocab // 5]))
    banned = rng.sample(range(vocab), k=rng.choice([0, 3]))

    def options_of(i):
        r = random.Random(seed * 1000 + i)
        kind = r.choice(["greedy", "temperature", "top_k", "top_p", "both", "penalty"])
        common = dict(seed=r.randint(0, 10 ** 6), ignore_eos=r.random() < 0.2)
        if kind == "greedy":
            return SamplingParams(ignore_eos=common["ignore_eos"], presence_penalty=r.choice([0.0, 3.0]))
        t = r.uniform(0.5, 1.5)
        return {"temperature": SamplingParams(temperature=t, **common),
                "top_k": SamplingParams(temperature=t, top_k=r.choice([1, 5, 40]), **common),
                "top_p": SamplingParams(temperature=t, top_p=r.uniform(0.3, 0.95), **common),
                "both": SamplingParams(temperature=t, top_k=r.choice([3, 20]), top_p=r.uniform(0.5, 0.95), **common),
                "penalty": SamplingParams(temperature=t, presence_penalty=r.uniform(0.5, 4.0), **common)}[kind]

    longest = max(len(p) + n for p, n in zip(prompts, lengths))
    pages = max((longest + page - 1) // page + 1, rng.choice([4, 6, 8]))
    batch, chunk = rng.choice([2, 4, 8]), rng.choice([4, 16, 64])
    results = []
    for ahead in (True, False):
        engine = ContinuousBatchEngine(model, max_batch_size=batch, chunk_size=chunk, page_size=page, num_pages=pages,
                                       max_sequences=8, eos_token_ids=eos, banned_tokens=banned or None, seed=5)
        ids = [engine.add_request(p, n, options_of(i)) for i, (p, n) in enumerate(zip(prompts, lengths))]
        engine.run_until_complete(one_step_ahead=ahead)
        stats = engine.get_stats()
        assert stats.num_finished == count and stats.num_running == 0 and stats.num_waiting == 0
        engine.runner.cache.check()
        assert all(g.pool.num_held == 0 for g in engine.runner.cache.groups)
        results.append([(engine.get_request(i).generated_tokens, engine.get_request(i).finish_reason,
                         engine.get_result(i)) for i in ids])
    assert results[0] == results[1]


@pytest.mark.parametrize("seed", range(6))
def test_random_configurations_mixed_batches_with_page_reuse(tmp_path, seed):
    """Up to four live requests, portions of some beside single tokens of others, in a pool of 256 tokens whose
    pages are used again, for random configurations in both storage types."""
    if not torch.cuda.is_available():
        pytest.skip("no GPU visible")
    from pulse_infer_amd.config import Qwen3Config
    from pulse_infer_amd.engine.runner import ModelRunner, StepEntry
    from pulse_infer_amd.models.factory import load_model
    from pulse_infer_amd.weights import write_model_folder
    from test_gpu_model import mixed_trace

    rng = random.Random(3000 + seed)
    cfg, options = random_config(rng, [128, 256, 1024])
    windows = (options or {}).get("layer_windows")
    page = rng.choice([16, 32, 64])
    folder = write_model_folder(Qwen3Config.from_dict(cfg), str(tmp_path / "m"), seed=70 + seed)
    plain = PlainQwen3.from_folder(folder, windows=windows)
    ids, steps = mixed_trace(cfg["vocab_size"], seed=20 + seed)
    want = {k: plain.logits(v) for k, v in ids.items()}
    for dtype in ("float32", "bfloat16"):
        _, model = load_model(folder, mode=dtype, config_overrides=options)
        runner = ModelRunner(model, page_size=page, num_pages=256 // page, max_requests=4)
        got = {k: [] for k in ids}
        for step in steps:
            entries = []
            for e in step["entries"]:
                if not runner.cache.has_request(e["id"]):
                    runner.add_request(e["id"])
                runner.reserve(e["id"], runner.cache.computed(e["id"]) + len(e["tokens"]))
                entries.append(StepEntry(e["id"], e["tokens"], e["want"]))
            logits = runner.step(entries)
            row = 0
            for e in step["entries"]:
                got[e["id"]].append(logits[row:row + len(e["want"])])
                row += len(e["want"])
            for k in step["end"]:
                runner.free_request(k)
            runner.cache.check()
        for k, parts in got.items():
            close(torch.cat(parts), want[k], dtype, f"mixed request {k}: {cfg} {options} page {page}")
        del runner, model
    torch.cuda.empty_cache()


@pytest.mark.parametrize("seed", range(4))
def test_random_traces_with_recorded_steps_over_small_context_buckets(tmp_path, seed):
    """Random traces, random configurations (widths whose decoding steps run without norm kernels among them): up to
    six live requests, prompt portions of random sizes beside decoded tokens, requests left out of steps, and long
    runs of steps of decoded tokens only, which are recorded at once and replayed, over context buckets so small that
    the requests walk through many of them (another recording, another number of splits each time, every replay told
    its own longest context); few pages, so that they are used again.  Every wanted row against the plain
    implementation, in bfloat16 (recorded) and in 32-bit (eager)."""
    if not torch.cuda.is_available():
        pytest.skip("no GPU visible")
    from pulse_infer_amd.config import Qwen3Config
    from pulse_infer_amd.engine.runner import ModelRunner, StepEntry
    from pulse_infer_amd.models.factory import load_model
    from pulse_infer_amd.weights import write_model_folder

    rng = random.Random(4000 + seed)
    cfg, options = random_config(rng, [256, 1024, 1024, 2048], max_positions=2048)
    cfg["num_hidden_layers"] = min(cfg["num_hidden_layers"], 2)
    if options:
        options = {"layer_windows": options["layer_windows"][:cfg["num_hidden_layers"]]}
        if not any(options["layer_windows"]):
            options = None
    windows = (options or {}).get("layer_windows")
    page = rng.choice([16, 32])
    folder = write_model_folder(Qwen3Config.from_dict(cfg), str(tmp_path / "m"), seed=80 + seed)
    plain = PlainQwen3.from_folder(folder, windows=windows)
    lengths = [rng.choice([3, 20, 70, 150, 300]) + rng.randint(0, 30) for _ in range(rng.randint(2, 6))]
    ids = {r: token_ids(cfg["vocab_size"], n, seed=seed * 10 + r) for r, n in enumerate(lengths)}
    want = {r: plain.logits(ids[r]) for r in ids}
    for dtype in ("bfloat16", "float32"):
        trace = random.Random(5000 + seed)            # the same trace for both
        _, model = load_model(folder, mode=dtype, config_overrides=options)
        runner = ModelRunner(model, page_size=page, num_pages=sum((n + page - 1) // page for n in lengths) + 1,
                             max_requests=len(lengths))
        runner.GRAPH_AFTER_STEPS = 1
        runner.GRAPH_CONTEXT_BUCKET = trace.choice([64, 256])
        fed = {r: 0 for r in ids}
        live, got = set(), {r: [] for r in ids}
        prompt_end = {r: trace.randint(1, lengths[r]) for r in ids}      # up to here in portions, then token by token
        while any(fed[r] < lengths[r] for r in ids):
            todo = [r for r in ids if fed[r] < lengths[r]]
            decode_only = trace.random() < 0.6
            entries, rows = [], []
            for r in todo:
                if trace.random() < 0.2 and len(todo) > 1:
                    continue                                              # left out of this step
                if fed[r] >= prompt_end[r] or (decode_only and fed[r] > 0):
                    n = 1
                elif decode_only:
                    continue
                else:
                    n = min(trace.choice([2, 5, 16, 17, 40, 64, 130]), prompt_end[r] - fed[r])
                if r not in live:
                    runner.add_request(r)
                    live.add(r)
                runner.reserve(r, fed[r] + n)
                wanted = [n - 1] if n == 1 or trace.random() < 0.7 else [0, n - 1]
                entries.append(StepEntry(r, ids[r][fed[r]:fed[r] + n], wanted))
                rows += [(r, fed[r] + w) for w in wanted]
                fed[r] += n
            if not entries:
                continue
            for (r, pos), row in zip(rows, runner.step(entries)):
                got[r].append((pos, row))
            for r in list(live):
                if fed[r] >= lengths[r]:
                    runner.free_request(r)
                    live.discard(r)
            runner.cache.check()
        if dtype == "bfloat16":
            assert runner.graph_records >= 2 and runner.graph_replays >= 10
        for r, pairs in got.items():
            mine = torch.stack([row for _, row in pairs])
            ref = torch.stack([want[r][pos] for pos, _ in pairs])
            close(mine, ref, dtype, f"request {r} of {lengths}: {cfg} {options} page {page}")
        del runner, model
    torch.cuda.empty_cache()
