"""Generation through the entry points: greedy against the plain implementation, long decoding,
continuous batching with portions, preemption when pages run out, seeded sampling, the command line."""
import json

import pytest
import torch

from conftest import OVERRIDES, TINY, WINDOW_W, token_ids

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def gpu():
    if not torch.cuda.is_available():
        pytest.skip("no GPU visible")


def make_llm(folder, dtype="float32", name=None, **options):
    from pulse_infer_amd import LLM
    return LLM.from_pretrained(folder, dtype=dtype, config_overrides=OVERRIDES.get(name), **options)


@pytest.mark.parametrize("name", ["A", "B", "W"])
def test_greedy_generation_matches_the_plain_implementation(gpu, model_folders, plain_models, name):
    cfg, page = TINY[name]
    prompts = [token_ids(cfg["vocab_size"], n, seed=20 + n) for n in (5, 11, 17)]
    llm = make_llm(model_folders[name], "float32", name, max_batch_size=3, chunk_size=8, page_size=page, num_pages=64)
    got = llm.generate(prompts, max_new_tokens=8, ignore_eos=True)
    for prompt, out in zip(prompts, got):
        assert out == plain_models[name].greedy(prompt, 8)
    llm.engine.runner.cache.check()
    assert not llm.engine.runner.cache.requests                       # everything was given back
    # bfloat16: the same tokens wherever the plain top-two margin is clear of bfloat16's error
    llm16 = make_llm(model_folders[name], "bfloat16", name, max_batch_size=3, chunk_size=8, page_size=page, num_pages=64)
    clear = 0
    for prompt, out in zip(prompts, llm16.generate(prompts, max_new_tokens=8, ignore_eos=True)):
        assert len(out) == 8
        rows = plain_models[name].logits(list(prompt) + out)[len(prompt) - 1:-1]   # along the engine's own path
        for tok, row in zip(out, rows):
            top = torch.topk(row, 2)
            if float(top.values[0] - top.values[1]) > 0.25:
                assert tok == int(top.indices[0])
                clear += 1
            assert float(row[tok]) >= float(row.max()) - 3e-2 * float(row.abs().max())   # never far from the best
    assert clear >= 5, f"only {clear} of 24 tokens had a margin that bfloat16 cannot blur: the check says too little"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_token_by_token(gpu, model_folders, plain_logits, dtype):
    """240 positions one token at a time (W has windows that pass many pages meanwhile)."""
    from pulse_infer_amd.engine.runner import ModelRunner, StepEntry
    from pulse_infer_amd.models.factory import load_model
    from test_gpu_model import close

    for name in ("B", "W"):
        cfg, page = TINY[name]
        ids = token_ids(cfg["vocab_size"], 240, seed=33)
        _, model = load_model(model_folders[name], mode=dtype, config_overrides=OVERRIDES[name])
        runner = ModelRunner(model, page_size=page, num_pages=256 // page, max_requests=2)
        runner.add_request("r")
        rows = []
        for i, tok in enumerate(ids):
            runner.reserve("r", i + 1)
            rows.append(runner.step([StepEntry("r", [tok], [0])]))
        if name == "W":
            held = [p for p in runner.cache.table(1, "r") if p >= 0]
            assert len(held) <= WINDOW_W // page + 2      # the window's pages only
        runner.free_request("r")
        close(torch.cat(rows), plain_logits(name, ids), dtype, f"{name} long decoding")


def test_continuous_batching_gives_what_each_request_gives_alone(gpu, model_folders):
    cfg, page = TINY["B"]
    prompts = [token_ids(cfg["vocab_size"], n, seed=40 + n) for n in (1, 9, 33, 70)]
    alone = []
    for p in prompts:
        alone.append(make_llm(model_folders["B"], max_batch_size=1, chunk_size=256, page_size=page,
                              num_pages=32).generate([p], max_new_tokens=12, ignore_eos=True)[0])
    llm = make_llm(model_folders["B"], max_batch_size=4, chunk_size=16, page_size=page, num_pages=32,
                   max_num_batched_tokens=24)
    assert llm.generate(prompts, max_new_tokens=12, ignore_eos=True) == alone
    stats = llm.engine.get_stats()
    assert stats.num_finished == 4 and stats.tokens_generated == 48 and stats.num_preemptions == 0


def test_preemption_reproduces_the_outputs(gpu, model_folders):
    cfg, page = TINY["A"]                                              # pages of 4 tokens
    prompts = [token_ids(cfg["vocab_size"], n, seed=50 + n) for n in (14, 15, 13)]
    roomy = make_llm(model_folders["A"], max_batch_size=3, chunk_size=8, page_size=page, num_pages=64)
    want = roomy.generate(prompts, max_new_tokens=20, ignore_eos=True)
    tight = make_llm(model_folders["A"], max_batch_size=3, chunk_size=8, page_size=page, num_pages=17)
    got = tight.generate(prompts, max_new_tokens=20, ignore_eos=True)
    stats = tight.engine.get_stats()
    assert stats.num_preemptions > 0, "the pool was meant to run out"
    assert got == want
    tight.engine.runner.cache.check()
    assert tight.engine.runner.cache.free_pages() == [17]


def test_eos_and_max_new_tokens(gpu, model_folders, plain_models):
    cfg, page = TINY["A"]
    prompt = token_ids(cfg["vocab_size"], 9, seed=61)
    path = plain_models["A"].greedy(prompt, 6)
    from pulse_infer_amd.engine.engine import ContinuousBatchEngine
    from pulse_infer_amd.models.factory import load_model
    _, model = load_model(model_folders["A"], mode="float32")
    engine = ContinuousBatchEngine(model, 2, 8, page_size=page, num_pages=32, eos_token_ids=[path[3]])
    rid = engine.add_request(prompt, 6)
    assert engine.get_result(rid) == []                               # nothing while it runs
    engine.run_until_complete()
    first_eos = path.index(path[3])
    assert engine.get_request(rid).generated_tokens == path[:first_eos + 1]   # the end-of-sequence id is kept ...
    assert engine.get_result(rid) == path[:first_eos]                         # ... and cut from the result
    assert engine.get_request(rid).finish_reason == "eos"
    with pytest.raises(ValueError, match="vocabulary"):
        engine.add_request([cfg["vocab_size"]], 2)


def test_seeded_sampling_does_not_depend_on_the_batch(gpu, model_folders):
    from pulse_infer_amd import SamplingParams
    cfg, page = TINY["B"]
    prompts = [token_ids(cfg["vocab_size"], n, seed=70 + n) for n in (4, 21, 9)]
    params = [SamplingParams(temperature=0.8, seed=100 + i, ignore_eos=True) for i in range(3)]
    together = make_llm(model_folders["B"], max_batch_size=3, chunk_size=16, page_size=page, num_pages=32).generate(
        prompts, max_new_tokens=12, sampling=params)
    for i in (2, 0):
        alone = make_llm(model_folders["B"], max_batch_size=1, chunk_size=5, page_size=page, num_pages=32).generate(
            [prompts[i]], max_new_tokens=12, sampling=[params[i]])[0]
        assert alone == together[i]
    other = make_llm(model_folders["B"], max_batch_size=3, chunk_size=16, page_size=page, num_pages=32).generate(
        prompts, max_new_tokens=12, sampling=[SamplingParams(temperature=0.8, seed=900 + i, ignore_eos=True) for i in range(3)])
    assert other != together                                          # another seed, another path
    # requests with options of different kinds in one batch: each draws what it draws alone (which kernels choose a
    # row's token depends on the row's own options)
    kinds = [SamplingParams(temperature=0.9, seed=31, ignore_eos=True),
             SamplingParams(temperature=0.9, top_k=7, seed=32, ignore_eos=True),
             SamplingParams(temperature=1.1, top_k=20, top_p=0.9, seed=33, ignore_eos=True),
             SamplingParams(temperature=1.0, top_p=0.8, seed=34, ignore_eos=True),
             SamplingParams(ignore_eos=True),
             SamplingParams(temperature=0.7, presence_penalty=1.5, seed=36, ignore_eos=True)]
    many = [token_ids(cfg["vocab_size"], n, seed=40 + n) for n in (6, 13, 3, 18, 8, 11)]
    mixed = make_llm(model_folders["B"], max_batch_size=6, chunk_size=16, page_size=page, num_pages=48).generate(
        many, max_new_tokens=10, sampling=kinds)
    for i in range(6):
        alone = make_llm(model_folders["B"], max_batch_size=1, chunk_size=16, page_size=page, num_pages=32).generate(
            [many[i]], max_new_tokens=10, sampling=[kinds[i]])[0]
        assert alone == mixed[i], i
    # temperature near zero is greedy; top_k = 1 is greedy whatever the temperature
    greedy = make_llm(model_folders["B"], page_size=page, num_pages=32).generate(prompts, max_new_tokens=6, ignore_eos=True)
    topk1 = make_llm(model_folders["B"], page_size=page, num_pages=32).generate(
        prompts, max_new_tokens=6, sampling=[SamplingParams(temperature=1.3, top_k=1, seed=5, ignore_eos=True)] * 3)
    assert topk1 == greedy
    # with a presence penalty large enough no token is generated twice
    fresh = make_llm(model_folders["B"], page_size=page, num_pages=32).generate(
        [prompts[1]], max_new_tokens=30, sampling=[SamplingParams(presence_penalty=1000.0, ignore_eos=True)])[0]
    assert len(set(fresh)) == 30 and not set(fresh) & set(prompts[1])


@pytest.mark.parametrize("name,dtype", [("B", "float32"), ("B", "bfloat16"), ("W", "float32")])
def test_the_loop_one_step_ahead_gives_what_the_loop_step_by_step_gives(gpu, model_folders, name, dtype):
    """``run_until_complete`` queues a step before it has seen the tokens of the step before (they are fed to it on
    the device).  Requests of every kind: ended by an end-of-sequence id that is drawn often, by their length, by
    both at once, with a presence penalty, greedy and seeded, in a pool so small that requests are preempted and
    computed again: every request's tokens, reasons and results are those of the loop that waits for every step.
    In 32-bit, where a draw does not depend on what else a step holds; in bfloat16 (recorded steps, whose ids are fed
    on the device) no request ends early and the pool is large, so that both loops run the same steps.  "W": layers
    with a window, whose pages go back to the pool while requests run."""
    from pulse_infer_amd import SamplingParams
    from pulse_infer_amd.engine.engine import ContinuousBatchEngine
    from pulse_infer_amd.models.factory import load_model

    cfg, page = TINY[name]
    _, model = load_model(model_folders[name], mode=dtype, config_overrides=OVERRIDES.get(name))
    vocab = cfg["vocab_size"]
    exact = dtype == "float32"
    eos = list(range(0, vocab, 9)) if exact else []   # one id in nine ends a request: many end early, at any step
    prompts = [token_ids(vocab, n, seed=200 + n) for n in (5, 33, 17, 2, 40, 11, 26, 8, 19, 3)]
    kinds = [SamplingParams(temperature=0.9, seed=11), SamplingParams(), SamplingParams(temperature=1.2, top_k=12, seed=12),
             SamplingParams(temperature=0.8, presence_penalty=2.0, seed=13), SamplingParams(temperature=1.0, top_p=0.9, seed=14),
             SamplingParams(temperature=0.9, seed=15, ignore_eos=True), SamplingParams(presence_penalty=50.0),
             SamplingParams(temperature=1.5, top_k=30, top_p=0.8, seed=16), SamplingParams(temperature=0.7, seed=17),
             SamplingParams(temperature=1.1, seed=18, ignore_eos=True)]
    lengths = [30, 12, 25, 40, 9, 16, 33, 1, 22, 14]
    results = []
    for ahead in (True, False):
        engine = ContinuousBatchEngine(model, max_batch_size=6, chunk_size=8, page_size=page,
                                       num_pages=(80 // page if exact else 64),
                                       max_sequences=6, eos_token_ids=eos, seed=3)
        engine.runner.GRAPH_AFTER_STEPS = 1
        ids = [engine.add_request(p, n, k) for p, n, k in zip(prompts, lengths, kinds)]
        engine.run_until_complete(one_step_ahead=ahead)
        stats = engine.get_stats()
        assert stats.num_finished == len(ids) and stats.num_running == 0 and stats.num_waiting == 0
        engine.runner.cache.check()
        assert all(g.pool.num_held == 0 for g in engine.runner.cache.groups)
        results.append([(engine.get_request(i).generated_tokens, engine.get_request(i).finish_reason,
                         engine.get_result(i)) for i in ids])
        if ahead and exact:
            assert stats.num_preemptions > 0                       # the pool of 5 pages made requests give way
        if not exact:
            assert engine.runner.graph_replays > 20
    for i, (a, b) in enumerate(zip(*results)):
        assert a == b, i
    reasons = {reason for _, reason, _ in results[0]}
    assert ({"eos", "length"} if exact else {"length"}) <= reasons


def _sweep_model(tmp_path, seed):
    """A seeded random configuration of the architecture (as the sweep's), its folder and its plain twin."""
    import random
    from plain.qwen3_plain import PlainQwen3
    from pulse_infer_amd.config import Qwen3Config
    from pulse_infer_amd.weights import write_model_folder
    from test_gpu_sweep import random_config

    rng = random.Random(seed)
    cfg, options = random_config(rng, [128, 256], max_positions=512)
    folder = write_model_folder(Qwen3Config.from_dict(cfg), str(tmp_path / "m"), seed=seed)
    plain = PlainQwen3.from_folder(folder, windows=(options or {}).get("layer_windows"))
    return cfg, options, folder, plain, rng.choice([16, 32])


@pytest.mark.parametrize("which", ["B", "sweep"])
def test_the_loop_one_step_ahead_in_bfloat16_with_recorded_steps_early_ends_and_preemption(
        gpu, model_folders, plain_models, tmp_path, which):
    """The serving loop as it serves (reference loop: src/scheduler/continuous_batch_engine.cpp:186-252): bfloat16,
    every step of single tokens recorded at once and replayed with its ids fed on the device, end-of-sequence ids that
    are drawn often (a request ends while the step that already holds its next token is queued) and a pool so tight
    that requests are preempted and computed again (some with their last token still on the device).  In bfloat16 the
    tokens need not be those of the loop that waits for every step, so what must hold is asserted instead: every
    request finishes, everything is given back, an end-of-sequence id is only ever a request's last token, and every
    greedy token, along the engine's own path, is the plain implementation's best or within bfloat16's error of it."""
    from pulse_infer_amd import SamplingParams
    from pulse_infer_amd.engine.engine import ContinuousBatchEngine
    from pulse_infer_amd.models.factory import load_model

    if which == "B":
        (cfg, page), options, folder, plain = TINY["B"], None, model_folders["B"], plain_models["B"]
    else:
        cfg, options, folder, plain, page = _sweep_model(tmp_path, 7003)
    vocab = cfg["vocab_size"]
    _, model = load_model(folder, mode="bfloat16", config_overrides=options)
    eos = list(range(0, vocab, 9))
    sizes = (5, 33, 17, 2, 40, 11, 26, 8, 19, 3, 30, 14)
    prompts = [token_ids(vocab, n, seed=600 + n) for n in sizes]
    lengths = [30, 12, 25, 40, 9, 16, 33, 1, 22, 14, 35, 28]
    kinds = [SamplingParams() for _ in sizes]
    kinds[3] = SamplingParams(ignore_eos=True)
    kinds[6] = SamplingParams(ignore_eos=True)
    kinds[2] = SamplingParams(temperature=0.9, top_k=12, seed=21)              # three that draw: their tokens are
    kinds[5] = SamplingParams(temperature=0.8, presence_penalty=2.0, seed=22)  # checked for form only
    kinds[9] = SamplingParams(temperature=1.1, top_p=0.9, seed=23)
    longest = max(len(p) + n for p, n in zip(prompts, lengths))
    pages = (longest + page - 1) // page + 1
    engine = ContinuousBatchEngine(model, max_batch_size=6, chunk_size=8, page_size=page, num_pages=pages,
                                   max_sequences=6, eos_token_ids=eos, seed=3)
    engine.runner.GRAPH_AFTER_STEPS = 1
    ids = [engine.add_request(p, n, k) for p, n, k in zip(prompts, lengths, kinds)]
    engine.run_until_complete(one_step_ahead=True)
    stats = engine.get_stats()
    assert stats.num_finished == len(ids) and stats.num_running == 0 and stats.num_waiting == 0
    engine.runner.cache.check()
    assert all(g.pool.num_held == 0 for g in engine.runner.cache.groups) and not engine.runner.cache.requests
    assert engine.runner.graph_records > 0 and engine.runner.graph_replays > 0
    assert stats.num_preemptions > 0, "the pool was meant to run out"
    reasons, checked = set(), 0
    for rid, prompt, most, kind in zip(ids, prompts, lengths, kinds):
        request = engine.get_request(rid)
        out = request.generated_tokens
        reasons.add(request.finish_reason)
        assert 1 <= len(out) <= most and all(0 <= t < vocab for t in out)
        if kind.ignore_eos:
            assert len(out) == most and request.finish_reason == "length"
        else:
            assert not any(t in eos for t in out[:-1])                   # an end-of-sequence id ends its request
            assert (out[-1] in eos) == (request.finish_reason == "eos")
            assert len(out) == most or request.finish_reason == "eos"
            assert engine.get_result(rid) == (out[:-1] if out[-1] in eos else out)
        if kind.greedy and kind.presence_penalty == 0.0:
            rows = plain.logits(list(prompt) + out)[len(prompt) - 1:-1]
            for t, (tok, row) in enumerate(zip(out, rows)):
                slack = 3e-2 * float(row.abs().max())
                assert float(row[tok]) >= float(row.max()) - slack, (
                    f"request {rid}, token {t}: logit {float(row[tok]):.4f} against the best {float(row.max()):.4f}")
                checked += 1
    assert {"eos", "length"} <= reasons and checked > 60


def test_a_fed_token_that_is_no_token_spoils_only_its_own_request(gpu, model_folders, plain_logits):
    """A request for which no token is allowed draws -1, and the loop one step ahead has by then queued a step that is
    fed that -1 on the device: its embedding row is NaN and so are the key and value that the step writes into the
    request's page.  The request ends there; nothing of it may reach another request, neither the one beside it in
    the step nor the one that gets its pages next (whose slots beyond its own context still hold the NaN).  Eager and
    recorded steps, against the plain implementation."""
    from pulse_infer_amd.engine.runner import ModelRunner, StepEntry
    from pulse_infer_amd.models.factory import load_model
    from test_gpu_model import close

    cfg, page = TINY["B"]
    vocab = cfg["vocab_size"]
    ids = {k: token_ids(vocab, n, seed=800 + n) for k, n in (("good", 60), ("bad", 41), ("next", 47))}
    want = {k: plain_logits("B", v) for k, v in ids.items() if k != "bad"}
    for dtype, graphs in (("float32", False), ("bfloat16", False), ("bfloat16", True)):
        _, model = load_model(model_folders["B"], mode=dtype)
        runner = ModelRunner(model, page_size=page, num_pages=8, max_requests=3, use_graphs=graphs)
        runner.GRAPH_AFTER_STEPS = 1
        for k, n in (("good", 30), ("bad", 37)):
            runner.add_request(k)
            runner.reserve(k, 60 if k == "good" else n + 4)
            runner.step([StepEntry(k, ids[k][:n], [])])
        none = torch.tensor([7, -1], dtype=torch.int32, device=model.device)    # what the step before "drew"
        got = []
        for s in range(4):         # "bad" is fed -1 from the device in every one of them; the host holds a valid id
            feed = (none, [1], [1])
            logits = runner.step([StepEntry("good", [ids["good"][30 + s]], [0]), StepEntry("bad", [0], [0])], feed=feed)
            got.append(logits[0])
            assert bool(torch.isnan(logits[1]).all())            # no token can be chosen from this row
        assert model.embedding.saw_bad_id()
        bad_pages = set(runner.cache.table(0, "bad"))
        runner.free_request("bad")
        runner.add_request("next")
        runner.reserve("next", 47)
        assert bad_pages & set(runner.cache.table(0, "next"))    # the pages with NaN in them are used again
        first = runner.step([StepEntry("next", ids["next"][:21], list(range(21)))])
        rest = [runner.step([StepEntry("good", [ids["good"][34 + s]], [0]),
                             StepEntry("next", [ids["next"][21 + s]], [0])]) for s in range(26)]
        if graphs:
            assert runner.graph_replays >= 20
        close(torch.stack(got + [r[0] for r in rest]), want["good"][30:60], dtype, f"beside the spoiled request ({dtype})")
        close(torch.cat([first, torch.stack([r[1] for r in rest])]), want["next"], dtype,
              f"in the spoiled request's pages ({dtype})")
        runner.cache.reset()
        runner.cache.check()


def test_command_line(gpu, model_folders, plain_models, capsys):
    from pulse_infer_amd import cli
    cfg, page = TINY["A"]
    prompt = token_ids(cfg["vocab_size"], 7, seed=81)
    code = cli.main([model_folders["A"], "--dtype", "f32", "--prompt-ids", ",".join(map(str, prompt)),
                     "--max-new-tokens", "5", "--page-size", str(page), "--num-pages", "32", "--ignore-eos", "--stats"])
    lines = capsys.readouterr().out.strip().splitlines()
    assert code == 0 and json.loads(lines[0])["output_ids"] == plain_models["A"].greedy(prompt, 5)
    assert lines[1].startswith("Generated 5 tokens in ") and "tokens/s" in lines[1]
    assert json.loads(lines[2])["tokens_generated"] == 5
    code = cli.main(["--model", model_folders["A"], "--random-weights", "--seed", "3", "--prompt-len", "6",
                     "--max-new-tokens", "4", "--temperature", "0.7", "--top-k", "20", "--top-p", "0.95",
                     "--sample-seed", "1", "--num-pages", "32"])
    assert code == 0 and len(json.loads(capsys.readouterr().out.splitlines()[0])["output_ids"]) == 4


def test_captured_decode_steps_replay_like_eager_ones(gpu, model_folders, plain_logits):
    """Decode steps are recorded once per (batch, context bucket), when the shape comes for the fourth time, and
    replayed from then on.  Every replay is checked against the eager step and the plain implementation, with eager
    prompt portions of other requests in between."""
    from pulse_infer_amd.engine.runner import ModelRunner, StepEntry
    from pulse_infer_amd.models.factory import load_model
    from test_gpu_model import SPLIT_TOL, close

    cfg, page = TINY["B"]
    _, model = load_model(model_folders["B"], mode="bfloat16")
    runners = [ModelRunner(model, page_size=16, num_pages=32, max_requests=4, use_graphs=flag) for flag in (True, False)]
    ids = {k: token_ids(cfg["vocab_size"], n, seed=90 + n) for k, n in (("a", 60), ("b", 75), ("c", 50))}
    got = [{k: [] for k in ids} for _ in runners]
    for which, runner in enumerate(runners):
        fed = {k: 0 for k in ids}

        def feed(pairs):
            entries = []
            for k, n in pairs:
                if not runner.cache.has_request(k):
                    runner.add_request(k)
                runner.reserve(k, fed[k] + n)
                entries.append(StepEntry(k, ids[k][fed[k]:fed[k] + n], [n - 1]))
                fed[k] += n
            logits = runner.step(entries)
            for row, (k, _) in enumerate(pairs):
                got[which][k].append((fed[k] - 1, logits[row]))

        feed([("a", 20), ("b", 31)])
        for _ in range(10):
            feed([("a", 1), ("b", 1)])                   # three eager steps, recorded at the fourth, replayed six times
        feed([("c", 17)])                                 # eager work between replays
        for _ in range(8):
            feed([("a", 1), ("b", 1), ("c", 1)])         # another batch size: another recording
        feed([("c", 9)])
        for _ in range(12):
            feed([("b", 1), ("a", 1)])                   # the first recording again, entries in another order
        assert runner.use_graphs == (which == 0) and runner.graph_records == (2 if which == 0 else 0)
    for k in ids:
        want = plain_logits("B", ids[k])
        for (pos_g, row_g), (pos_e, row_e) in zip(got[0][k], got[1][k]):
            assert pos_g == pos_e
            close(row_g[None], want[pos_g][None], "bfloat16", f"captured {k}@{pos_g}")
            close(row_g[None], row_e[None], "bfloat16", f"captured against eager {k}@{pos_g}", SPLIT_TOL)


def test_steps_of_uneven_contexts_are_recorded_apart(gpu, model_folders, plain_logits):
    """When the longest context of a decoding step is well above the mean, attention shares its work out by a plan
    made on the device (every request cut by its own length, the longest walks first), and such a step has a recording
    of its own.  A batch that goes from uneven to even and back, with another request in between: three recordings,
    every replay against the eager step and the plain implementation."""
    from pulse_infer_amd.engine.runner import ModelRunner, StepEntry
    from pulse_infer_amd.models.factory import load_model
    from test_gpu_model import SPLIT_TOL, close

    cfg, page = TINY["B"]
    _, model = load_model(model_folders["B"], mode="bfloat16")
    lens = {"a": 200, "b": 20, "c": 24, "d": 18, "e": 150, "f": 25}
    ids = {k: token_ids(cfg["vocab_size"], n + 30, seed=70 + n) for k, n in lens.items()}
    got = []
    for graphs in (True, False):
        runner = ModelRunner(model, page_size=16, num_pages=40, max_requests=4, use_graphs=graphs)
        runner.GRAPH_AFTER_STEPS = 1
        fed, rows = {}, []

        def start(k):
            runner.add_request(k)
            runner.reserve(k, lens[k] + 30)
            runner.step([StepEntry(k, ids[k][:lens[k]], [])])
            fed[k] = lens[k]

        def decode(names, steps):
            for _ in range(steps):
                logits = runner.step([StepEntry(k, ids[k][fed[k]:fed[k] + 1], [0]) for k in names])
                for row, k in enumerate(names):
                    rows.append((k, fed[k], logits[row]))
                    fed[k] += 1

        for k in "abcd":
            start(k)
        decode("abcd", 5)            # uneven: one of 200 among three of 20
        runner.free_request("a")
        decode("bcd", 5)             # even
        start("e")
        decode("ebcd", 5)            # uneven again, another request in another place: the first recording
        runner.free_request("e")
        start("f")
        decode("bcdf", 5)            # four even ones
        assert runner.graph_records == (3 if graphs else 0)
        assert runner.graph_replays == (20 - 3 if graphs else 0)
        for k in "bcdf":
            runner.free_request(k)
        runner.cache.check()
        got.append(rows)
    assert any(name.startswith("attention.plan") for name, _ in model.workspace._flat)   # the eager steps planned too
    for (k, pos, recorded), (k2, pos2, eager) in zip(*got):
        assert (k, pos) == (k2, pos2)
        want = plain_logits("B", ids[k])                 # (causal: the logits at pos do not see what follows)
        close(recorded[None], want[pos][None], "bfloat16", f"uneven {k}@{pos}")
        close(recorded[None], eager[None], "bfloat16", f"uneven against eager {k}@{pos}", SPLIT_TOL)


def test_the_collector_rests_while_a_step_is_recorded(gpu, model_folders):
    """No graph may be destroyed while a stream records, and Python's collector, which may find dropped recordings (of
    a step function that is no longer used, of the caller), runs whenever it likes: the step function keeps it off
    while it records.  A dropped step function itself goes at once: nothing points back at it
    in a circle."""
    import gc
    import weakref
    from pulse_infer_amd.engine.runner import ModelRunner, StepEntry
    from pulse_infer_amd.models.factory import load_model

    cfg, page = TINY["B"]
    _, model = load_model(model_folders["B"], mode="bfloat16")
    ids = token_ids(cfg["vocab_size"], 40, seed=5)
    seen = []
    forward = model.forward

    def watched(ctx, views):
        seen.append((torch.cuda.is_current_stream_capturing(), gc.isenabled()))
        return forward(ctx, views)

    model.forward = watched
    try:
        runner = ModelRunner(model, page_size=16, num_pages=8, max_requests=2)
        runner.GRAPH_AFTER_STEPS = 1
        runner.add_request("a")
        runner.reserve("a", 40)
        runner.step([StepEntry("a", ids[:30], [29])])
        for t in range(30, 34):
            runner.step([StepEntry("a", ids[t:t + 1], [0])])
    finally:
        model.forward = forward
    assert runner.graph_records == 1 and runner.graph_replays == 3
    assert (True, False) in seen                      # it was recorded, with the collector off
    assert all(on for capturing, on in seen if not capturing) and not any(on for capturing, on in seen if capturing)
    assert gc.isenabled()
    gone = weakref.ref(runner)
    del runner
    assert gone() is None                             # no circle: the recordings went with it, not at the collector's whim


def test_recorded_steps_while_a_window_gives_pages_back_and_after_eviction(gpu, model_folders, plain_logits):
    """Tiny W (windows of 24 keys on some layers, pages of 16): two requests decode far past window + page while
    their steps are replayed, so the windowed group gives pages back under a live recording and its table rows hold
    -1 there.  Only one recording is kept, and the batch alternates between two and one request, so every change
    evicts the recording and the next step of that shape records again.  Against the plain implementation and the
    eager steps."""
    from pulse_infer_amd.engine.runner import ModelRunner, StepEntry
    from pulse_infer_amd.models.factory import load_model
    from test_gpu_model import SPLIT_TOL, close

    cfg, _ = TINY["W"]
    _, model = load_model(model_folders["W"], mode="bfloat16", config_overrides=OVERRIDES["W"])
    ids = {"a": token_ids(cfg["vocab_size"], 120, seed=71), "b": token_ids(cfg["vocab_size"], 100, seed=72)}
    start = {"a": 20, "b": 9}
    outs = []
    for graphs in (True, False):
        runner = ModelRunner(model, page_size=16, num_pages=24, max_requests=2, use_graphs=graphs)
        runner.GRAPH_AFTER_STEPS, runner.GRAPH_LIMIT = 1, 1
        fed, got = dict(start), {k: [] for k in ids}
        for k, n in start.items():
            runner.add_request(k)
            runner.reserve(k, len(ids[k]))
            runner.step([StepEntry(k, ids[k][:n], [])])
        windowed = next(g for g in runner.cache.groups if g.spec.window is not None)
        for s in range(80):
            who = ["a", "b"] if (s // 5) % 2 == 0 else ["a"]          # five steps of two, five of one, ...
            logits = runner.step([StepEntry(k, [ids[k][fed[k]]], [0]) for k in who])
            for row, k in enumerate(who):
                got[k].append(logits[row])
                fed[k] += 1
        assert -1 in windowed.tables["a"] and -1 in windowed.tables["b"]          # pages were given back on the way
        if graphs:
            assert runner.graph_records == 16 and runner.graph_replays == 80 - 16    # every change of batch records anew
        outs.append({k: torch.stack(v) for k, v in got.items()})
        runner.cache.reset()
        runner.cache.check()
    for k in ids:
        n = outs[0][k].shape[0]
        want = plain_logits("W", ids[k])[start[k]:start[k] + n]
        close(outs[0][k], want, "bfloat16", f"recorded under a window, request {k}")
        close(outs[0][k], outs[1][k], "bfloat16", f"recorded against eager under a window, request {k}", SPLIT_TOL)
