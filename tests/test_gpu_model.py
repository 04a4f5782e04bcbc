"""The engine against the plain implementation, in 32-bit and in bfloat16: each request alone and whole;
most of it in one step and the last 32 tokens one by one; in portions of changing size down to two
tokens; and mixed, up to four live requests, portions of some beside decoded tokens of others, with so
few pages that they are used again.  Tolerances are fixed here once and are not to be widened."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

from conftest import OVERRIDES, ROOT, TINY, token_ids

pytestmark = pytest.mark.gpu

# max |engine - plain| relative to the largest |logit| of the sequence
TOL = {"float32": 3e-5, "bfloat16": 3e-2}
# two ways of cutting the same request, same dtype: only the order of float32 sums differs
SPLIT_TOL = {"float32": 1e-5, "bfloat16": 2e-2}


def close(got, want, dtype, what, tol=TOL):
    got, want = got.double().cpu(), want.double().cpu()
    assert got.shape == want.shape, (what, got.shape, want.shape)
    scale = max(1.0, float(want.abs().max()))
    err = float((got - want).abs().max())
    assert err <= tol[dtype] * scale, f"{what}: max error {err:.3e} exceeds {tol[dtype] * scale:.3e}"


@pytest.fixture(scope="module")
def engines(model_folders):
    """(name, dtype) -> ModelRunner with a deliberately small pool."""
    if not torch.cuda.is_available():
        pytest.skip("no GPU visible")
    from pulse_infer_amd.engine.runner import ModelRunner
    from pulse_infer_amd.models.factory import load_model

    made = {}

    def get(name, dtype, page=None, tokens=256):
        page = page or TINY[name][1]
        key = (name, dtype, page)
        if key not in made:
            _, model = load_model(model_folders[name], mode=dtype, config_overrides=OVERRIDES[name])
            made[key] = ModelRunner(model, page_size=page, num_pages=tokens // page, max_requests=4)
        return made[key]

    return get


def run_alone(runner, ids, cuts, rid="r"):
    """Feed ids in portions of the given sizes, wanting every position; returns [len(ids), vocab]."""
    from pulse_infer_amd.engine.runner import StepEntry

    assert sum(cuts) == len(ids)
    runner.add_request(rid)
    outs, p = [], 0
    for n in cuts:
        runner.reserve(rid, p + n)
        outs.append(runner.step([StepEntry(rid, ids[p:p + n], list(range(n)))]))
        p += n
    runner.free_request(rid)
    runner.cache.check()
    return torch.cat(outs)


LENGTH = {"A": 100, "B": 150, "W": 170}
# (configuration, page size): each configuration's own small page and pages of 16 and more, which in bfloat16
# take the matrix-core attention kernel
CASES = [("A", 4), ("A", 16), ("B", 16), ("B", 64), ("W", 8), ("W", 16)]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name,page", CASES)
def test_whole_tail_and_portions(engines, plain_logits, name, page, dtype):
    cfg = TINY[name][0]
    ids = token_ids(cfg["vocab_size"], LENGTH[name], seed=3)
    want = plain_logits(name, ids)
    runner = engines(name, dtype, page)
    whole = run_alone(runner, ids, [len(ids)])
    close(whole, want, dtype, f"{name} whole")
    tail = run_alone(runner, ids, [len(ids) - 32] + [1] * 32)
    close(tail, want, dtype, f"{name} last 32 one by one")
    close(tail, whole, dtype, f"{name} tail against whole", SPLIT_TOL)
    cuts, left, sizes = [], len(ids), [7, 2, 16, 3, 2, 33, 5, 2, 64, 11, 2]
    while left:
        n = min(sizes[len(cuts) % len(sizes)], left)
        if left - n == 1:          # keep every portion at two tokens or more
            n += 1
        cuts.append(n)
        left -= n
    portions = run_alone(runner, ids, cuts)
    close(portions, want, dtype, f"{name} portions {cuts}")
    close(portions, whole, dtype, f"{name} portions against whole", SPLIT_TOL)
    first = run_alone(runner, ids[:3], [1, 1, 1])                    # the first tokens of a sequence
    close(first, want[:3], dtype, f"{name} first tokens")


def mixed_trace(vocab, seed, sizes=(2, 3, 5, 8, 13, 21)):
    """Six requests, at most four live, over a pool that holds 256 tokens: pages of finished requests are
    used again by later ones.  Steps mix prompt portions of some (of the given sizes) with single tokens of others."""
    rng = np.random.RandomState(seed)
    lengths = {"a": 60, "b": 45, "c": 64, "d": 30, "e": 50, "f": 58}
    ids = {k: token_ids(vocab, n, seed=seed * 10 + i) for i, (k, n) in enumerate(lengths.items())}
    fed = {k: 0 for k in lengths}
    waiting, live, steps = list(lengths), [], []
    while waiting or live:
        held = sum((fed[k] + 63) // 64 * 64 for k in live)
        while waiting and len(live) < 4 and held + (lengths[waiting[0]] + 63) // 64 * 64 <= 256:
            k = waiting.pop(0)
            live.append(k)
            held += (lengths[k] + 63) // 64 * 64
        entries, end = [], []
        for k in list(live):
            if rng.rand() < 0.2 and len(live) > 1:
                continue                                             # a request may sit a step out
            left = lengths[k] - fed[k]
            if fed[k] >= lengths[k] - 12:
                n = 1                                                # its last tokens come one by one
            else:
                n = int(min(left - 12, rng.choice(list(sizes))))
                n = max(n, 1)
            entries.append({"id": k, "tokens": ids[k][fed[k]:fed[k] + n], "want": list(range(n))})
            fed[k] += n
            if fed[k] == lengths[k]:
                end.append(k)
                live.remove(k)
        if entries:
            steps.append({"step": len(steps), "entries": entries, "end": end})
    return ids, steps


def run_mixed(runner, steps):
    """Drive the steps of ``mixed_trace`` through a runner: per request the logits of all its places, the pages it
    ever held, and the most requests that were live at once."""
    from pulse_infer_amd.engine.runner import StepEntry

    got, pages_seen, most_live = {}, {}, 0
    for step in steps:
        entries = []
        for e in step["entries"]:
            if not runner.cache.has_request(e["id"]):
                runner.add_request(e["id"])
            runner.reserve(e["id"], runner.cache.computed(e["id"]) + len(e["tokens"]))
            entries.append(StepEntry(e["id"], e["tokens"], e["want"]))
            pages_seen.setdefault(e["id"], set()).update(p for p in runner.cache.table(0, e["id"]) if p >= 0)
        most_live = max(most_live, len(runner.cache.requests))
        logits = runner.step(entries)
        row = 0
        for e in step["entries"]:
            got.setdefault(e["id"], []).append(logits[row:row + len(e["want"])])
            row += len(e["want"])
        for k in step["end"]:
            runner.free_request(k)
        runner.cache.check()
    return {k: torch.cat(parts) for k, parts in got.items()}, pages_seen, most_live


def pages_were_used_again(pages_seen):
    names = list(pages_seen)
    return any(pages_seen[a] & pages_seen[b] for i, a in enumerate(names) for b in names[i + 1:])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name,page", CASES)
def test_mixed_batches_with_page_reuse(engines, plain_logits, name, page, dtype):
    cfg = TINY[name][0]
    ids, steps = mixed_trace(cfg["vocab_size"], seed=5)
    runner = engines(name, dtype, page)
    got, pages_seen, most_live = run_mixed(runner, steps)
    assert most_live == 4 and any(len(s["entries"]) >= 3 for s in steps)
    assert any(len(e["tokens"]) > 1 for s in steps for e in s["entries"]) and \
        any(len(e["tokens"]) == 1 and len(s["entries"]) > 1 for s in steps for e in s["entries"])
    assert pages_were_used_again(pages_seen), "no page was used again"
    for k, mine in got.items():
        close(mine, plain_logits(name, ids[k]), dtype, f"{name} mixed request {k}")


# The layer sizes of the benchmark's model (Qwen3-8B: 32 query heads over 8 kv heads of 128, hidden 4096, feed-forward
# 12288) with two layers and a small vocabulary: the sizes at which the serving kernels run (the streaming product with
# K = 4096 and 12288, 128-wide heads in groups of four), against the plain implementation.
LAYER_SHAPE = dict(
    architectures=["Qwen3ForCausalLM"], model_type="qwen3", vocab_size=1032, hidden_size=4096, intermediate_size=12288,
    num_hidden_layers=2, num_attention_heads=32, num_key_value_heads=8, head_dim=128, max_position_embeddings=4096,
    rms_norm_eps=1e-6, rope_theta=1e6, tie_word_embeddings=False, torch_dtype="bfloat16", attention_bias=False,
    use_sliding_window=False, hidden_act="silu")


@pytest.fixture(scope="module")
def layer_shape(tmp_path_factory):
    if not torch.cuda.is_available():
        pytest.skip("no GPU visible")
    from plain.qwen3_plain import PlainQwen3
    from pulse_infer_amd.config import Qwen3Config
    from pulse_infer_amd.weights import write_model_folder

    folder = str(tmp_path_factory.mktemp("layer_shape"))
    write_model_folder(Qwen3Config.from_dict(LAYER_SHAPE), folder, seed=41)
    ids = token_ids(LAYER_SHAPE["vocab_size"], 150, seed=42)
    plain = PlainQwen3.from_folder(folder)
    return folder, ids, plain.logits(ids), plain


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_benchmark_layer_sizes(layer_shape, dtype):
    from pulse_infer_amd.engine.runner import ModelRunner
    from pulse_infer_amd.models.factory import load_model

    folder, ids, want, _ = layer_shape
    _, model = load_model(folder, mode=dtype)
    runner = ModelRunner(model, page_size=16, num_pages=24, max_requests=4)
    whole = run_alone(runner, ids, [len(ids)])
    close(whole, want, dtype, "layer sizes, whole")
    tail = run_alone(runner, ids, [len(ids) - 32] + [1] * 32)
    close(tail, want, dtype, "layer sizes, last 32 one by one")
    close(tail, whole, dtype, "layer sizes, tail against whole", SPLIT_TOL)
    portions = run_alone(runner, ids, [40, 2, 17, 64, 3, 5, 19])
    close(portions, want, dtype, "layer sizes, portions")
    close(portions, whole, dtype, "layer sizes, portions against whole", SPLIT_TOL)
    if dtype == "bfloat16":
        assert runner.graph_replays >= 1           # the single tokens ran as recorded steps
    del runner, model
    torch.cuda.empty_cache()


@pytest.mark.parametrize("policy", ["swiglu", "all"])
def test_benchmark_layer_sizes_with_this_packages_products_for_many_rows(layer_shape, policy, monkeypatch):
    """A prompt of 600 tokens at the benchmark's layer sizes, whole and in portions of 300, 260 and 40 tokens, with the
    products of 256 and more rows in this package's tiled product (gate and up with SwiGLU inside; or all of them, o
    and down in shares of the inner dimension) against the plain implementation and against the library's products."""
    from pulse_infer_amd.engine.runner import ModelRunner
    from pulse_infer_amd.models.factory import load_model
    from pulse_infer_amd.parts import linear

    folder, _, _, plain = layer_shape
    ids = token_ids(LAYER_SHAPE["vocab_size"], 600, seed=44)
    want = plain.logits(ids)
    _, model = load_model(folder, mode="bfloat16")
    runner = ModelRunner(model, page_size=16, num_pages=40, max_requests=2)
    monkeypatch.setattr(linear, "OWN_MANY_ROWS", "none")      # (whatever PULSE_OWN_PRODUCTS says)
    library = run_alone(runner, ids, [len(ids)])
    monkeypatch.setattr(linear, "OWN_MANY_ROWS", policy)
    whole = run_alone(runner, ids, [len(ids)])
    close(whole, want, "bfloat16", f"own products ({policy}), whole")
    close(whole, library, "bfloat16", f"own products ({policy}) against the library's", SPLIT_TOL)
    assert not torch.equal(whole, library)                 # (another kernel did run)
    portions = run_alone(runner, ids, [300, 260, 40])
    close(portions, want, "bfloat16", f"own products ({policy}), portions")
    close(portions, whole, "bfloat16", f"own products ({policy}), portions against whole", SPLIT_TOL)
    del runner, model
    torch.cuda.empty_cache()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_benchmark_layer_sizes_mixed_with_page_reuse(layer_shape, dtype):
    """Up to four live requests at the benchmark model's layer sizes over a pool of 256 tokens: steps that hold a
    portion of 16 tokens and more (the prompt-portion attention kernel) beside single decoded tokens (the split
    kernel) and steps of 17 to 64 rows (the products for those row counts, the shares of o and down), which no
    single request alone ever makes."""
    from pulse_infer_amd.engine.runner import ModelRunner
    from pulse_infer_amd.models.factory import load_model

    folder, _, _, plain = layer_shape
    ids, steps = mixed_trace(LAYER_SHAPE["vocab_size"], seed=4, sizes=(2, 3, 16, 21, 34))
    rows = [sum(len(e["tokens"]) for e in s["entries"]) for s in steps]
    assert any(17 <= r <= 64 for r in rows) and any(13 <= r <= 16 for r in rows)
    assert any(any(len(e["tokens"]) >= 16 for e in s["entries"]) and any(len(e["tokens"]) == 1 for e in s["entries"])
               for s in steps), "no step holds a portion of 16 tokens beside a single token"
    assert any(len(s["entries"]) == 4 and all(len(e["tokens"]) == 1 for e in s["entries"]) for s in steps)
    _, model = load_model(folder, mode=dtype)
    runner = ModelRunner(model, page_size=16, num_pages=16, max_requests=4)
    got, pages_seen, most_live = run_mixed(runner, steps)
    assert most_live == 4 and pages_were_used_again(pages_seen)
    for k, mine in got.items():
        close(mine, plain.logits(ids[k]), dtype, f"layer sizes, mixed request {k}")
    del runner, model
    torch.cuda.empty_cache()


@pytest.mark.parametrize("batch", [8, 3, 24, 40])
def test_benchmark_layer_sizes_recorded_decode_steps(layer_shape, batch):
    """Recorded steps at the benchmark's attention shape (heads of 128 in groups of four, the decode kernel writing
    keys and values from inside the graph): eight (and three) requests of unequal contexts, from 5 to more than a
    thousand keys, so that some of the splits chosen for the context bucket are empty for the short ones; the longest
    walks across a multiple of 1,024 on the way, which takes a new recording with a wider block table.  With 24 and 40
    requests the step's products are those for 17 to 64 rows (qkv and the logits among them: no library call, or the
    step would not be recorded).  Every replay against the eager step and the plain implementation."""
    from pulse_infer_amd.engine.runner import ModelRunner, StepEntry
    from pulse_infer_amd.models.factory import load_model

    folder, _, _, plain = layer_shape
    lengths = ([1018, 5, 700, 300, 1000, 64, 513, 17] + [20 + (7 * i) % 31 for i in range(32)])[:batch]
    steps = 12
    vocab = LAYER_SHAPE["vocab_size"]
    ids = [token_ids(vocab, n + steps, seed=300 + i) for i, n in enumerate(lengths)]
    _, model = load_model(folder, mode="bfloat16")
    results = []
    for graphs in (True, False):
        runner = ModelRunner(model, page_size=16, num_pages=sum((n + steps + 15) // 16 for n in lengths) + 2,
                             max_requests=batch, use_graphs=graphs)
        runner.GRAPH_AFTER_STEPS = 1                     # record at once: all other single-token steps are replays
        for r, n in enumerate(lengths):
            runner.add_request(r)
            runner.reserve(r, n + steps)
            runner.step([StepEntry(r, ids[r][:n], [])])
        got = [runner.step([StepEntry(r, [ids[r][n + s]], [0]) for r, n in enumerate(lengths)]) for s in range(steps)]
        results.append(torch.stack(got))                 # [steps, batch, vocab]
        assert runner.graph_replays == (steps - 2 if graphs else 0)
        assert runner.graph_records == (2 if graphs else 0)      # contexts up to 1,024, then up to 2,048
        for r in range(batch):
            runner.free_request(r)
        runner.cache.check()
        del runner
    recorded, eager = results
    for r, n in enumerate(lengths):
        want = plain.logits(ids[r], rows=list(range(n, n + steps)))
        close(recorded[:, r], want, "bfloat16", f"recorded, request {r} ({n} keys)")
        close(eager[:, r], want, "bfloat16", f"eager, request {r} ({n} keys)")
        close(recorded[:, r], eager[:, r], "bfloat16", f"recorded against eager, request {r}", SPLIT_TOL)
    del model
    torch.cuda.empty_cache()


# One layer of the benchmark's sizes under the benchmark's vocabulary: the head's products at the size they are timed
# at (151,936 rows of 4,096), and contexts up to the model's 4,096 positions.
HEAD_SHAPE = dict(LAYER_SHAPE, num_hidden_layers=1, vocab_size=151936)


@pytest.fixture(scope="module")
def head_shape(tmp_path_factory):
    if not torch.cuda.is_available():
        pytest.skip("no GPU visible")
    from plain.qwen3_plain import PlainQwen3
    from pulse_infer_amd.config import Qwen3Config
    from pulse_infer_amd.weights import write_model_folder

    folder = str(tmp_path_factory.mktemp("head_shape"))
    write_model_folder(Qwen3Config.from_dict(HEAD_SHAPE), folder, seed=43)
    return folder, PlainQwen3.from_folder(folder)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_the_head_at_the_benchmark_vocabulary(head_shape, dtype):
    """The logits of the last row of a whole prompt, of a step of 8 decoded tokens and of a step of 24 (in bfloat16
    three products: the streaming one for few rows, the same at 8 rows, the one for 17 to 64 rows with a float32
    result), at a vocabulary of 151,936, against the plain implementation."""
    from pulse_infer_amd.engine.runner import ModelRunner, StepEntry
    from pulse_infer_amd.models.factory import load_model

    folder, plain = head_shape
    vocab = HEAD_SHAPE["vocab_size"]
    _, model = load_model(folder, mode=dtype)
    runner = ModelRunner(model, page_size=16, num_pages=80, max_requests=24)
    prompt = token_ids(vocab, 70, seed=44)
    runner.add_request("p")
    runner.reserve("p", 70)
    got = runner.step([StepEntry("p", prompt, [69])])
    runner.free_request("p")
    assert got.shape == (1, vocab)
    close(got, plain.logits(prompt, rows=[69]), dtype, "head, last row of a prompt")
    for batch in (8, 24):
        lengths = [3 + (11 * i) % 29 for i in range(batch)]
        ids = [token_ids(vocab, n + 1, seed=500 + 10 * batch + i) for i, n in enumerate(lengths)]
        for r, n in enumerate(lengths):
            runner.add_request(r)
            runner.reserve(r, n + 1)
        runner.step([StepEntry(r, ids[r][:n], []) for r, n in enumerate(lengths)])
        got = runner.step([StepEntry(r, [ids[r][n]], [0]) for r, n in enumerate(lengths)])
        assert got.shape == (batch, vocab)
        want = torch.cat([plain.logits(ids[r], rows=[n]) for r, n in enumerate(lengths)])
        close(got, want, dtype, f"head, {batch} decoded rows")
        assert torch.equal(got.argmax(dim=1).cpu(), want.argmax(dim=1)) or dtype == "bfloat16"
        for r in range(batch):
            runner.free_request(r)
    runner.cache.check()
    del runner, model
    torch.cuda.empty_cache()


def test_recorded_decode_steps_at_the_benchmark_contexts(head_shape):
    """Three requests decode from 3,065 to 3,085 keys and, after a prompt portion each, from 4,075 to 4,090: into and
    inside the context bucket of 4,096 keys, the model's last positions, whose recording cuts every request's keys into
    the splits chosen for 4,096.  Every replay against the eager step and the plain implementation."""
    from pulse_infer_amd.engine.runner import ModelRunner, StepEntry
    from pulse_infer_amd.models.factory import load_model

    folder, plain = head_shape
    vocab = HEAD_SHAPE["vocab_size"]
    legs = ((3065, 20), (4075, 15))
    shift = (0, 1, 40)                           # the requests' contexts differ a little
    ids = [token_ids(vocab, 4090 - s, seed=700 + r) for r, s in enumerate(shift)]
    _, model = load_model(folder, mode="bfloat16")
    results, rows_of = [], {r: [] for r in range(3)}
    for graphs in (True, False):
        runner = ModelRunner(model, page_size=16, num_pages=3 * 256 + 2, max_requests=3, use_graphs=graphs)
        runner.GRAPH_AFTER_STEPS = 1
        fed, got = [0, 0, 0], {r: [] for r in range(3)}
        for r in range(3):
            runner.add_request(r)
            runner.reserve(r, len(ids[r]))
        for start, steps in legs:
            for r, s in enumerate(shift):
                runner.step([StepEntry(r, ids[r][fed[r]:start - s], [])])
                fed[r] = start - s
            for _ in range(steps):
                logits = runner.step([StepEntry(r, [ids[r][fed[r]]], [0]) for r in range(3)])
                for r in range(3):
                    got[r].append(logits[r])
                    if graphs:
                        rows_of[r].append(fed[r])
                    fed[r] += 1
        assert fed == [len(x) for x in ids]
        # (the first leg walks from the bucket of 3,072 keys into that of 4,096: two recordings)
        assert runner.graph_records == (2 if graphs else 0) and runner.graph_replays == (33 if graphs else 0)
        results.append({r: torch.stack(v) for r, v in got.items()})
        runner.cache.reset()
        runner.cache.check()
        del runner
    recorded, eager = results
    for r in range(3):
        want = plain.logits(ids[r], rows=rows_of[r])
        close(recorded[r], want, "bfloat16", f"recorded at the benchmark's contexts, request {r}")
        close(eager[r], want, "bfloat16", f"eager at the benchmark's contexts, request {r}")
        close(recorded[r], eager[r], "bfloat16", f"recorded against eager at the benchmark's contexts, request {r}",
              SPLIT_TOL)
    del model
    torch.cuda.empty_cache()


FAR_PAGES = dict(
    architectures=["Qwen3ForCausalLM"], model_type="qwen3", vocab_size=300, hidden_size=512, intermediate_size=768,
    num_hidden_layers=1, num_attention_heads=16, num_key_value_heads=8, head_dim=128, max_position_embeddings=512,
    rms_norm_eps=1e-6, rope_theta=1e4, tie_word_embeddings=False, torch_dtype="bfloat16", attention_bias=False,
    use_sliding_window=False, hidden_act="silu")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_pages_beyond_two_to_the_31_elements(tmp_path, dtype):
    """A pool of more than 131,072 pages of 8 heads x 16 slots x 128 channels: the low pages are held by idle
    requests, so that every page of the tested request starts past element 2^31 of the key and value arrays, where
    an offset computed in 32 bits would wrap (the reference computes them in 64 bits,
    src/ops/kernels/cuda/paged_attention.cu:96-98).  Whole, the last 32 tokens one by one, and portions of 64 tokens
    and more, against the plain implementation."""
    from plain.qwen3_plain import PlainQwen3
    from pulse_infer_amd.config import Qwen3Config
    from pulse_infer_amd.engine.runner import ModelRunner
    from pulse_infer_amd.models.factory import load_model
    from pulse_infer_amd.weights import write_model_folder

    if not torch.cuda.is_available():
        pytest.skip("no GPU visible")
    folder = write_model_folder(Qwen3Config.from_dict(FAR_PAGES), str(tmp_path / "m"), seed=61)
    ids = token_ids(FAR_PAGES["vocab_size"], 230, seed=62)
    want = PlainQwen3.from_folder(folder).logits(ids)
    page_elems = 8 * 16 * 128
    low = (1 << 31) // page_elems                          # pages that start below element 2^31
    _, model = load_model(folder, mode=dtype)
    runner = ModelRunner(model, page_size=16, num_pages=low + 24, max_requests=4)
    for half in ("idle0", "idle1"):                        # they hold every low page and are never stepped
        runner.add_request(half)
        runner.reserve(half, low // 2 * 16)
    assert runner.cache.groups[0].pool.num_free == 24

    def far(rid="r"):
        table = runner.cache.table(0, rid)
        assert table and min(table) >= low and min(table) * page_elems >= 1 << 31
    from pulse_infer_amd.engine.runner import StepEntry
    for cuts in ([230], [198] + [1] * 32, [100, 64, 66]):
        runner.add_request("r")
        outs, p = [], 0
        for n in cuts:
            runner.reserve("r", p + n)
            far()
            outs.append(runner.step([StepEntry("r", ids[p:p + n], list(range(n)))]))
            p += n
        runner.free_request("r")
        close(torch.cat(outs), want, dtype, f"far pages, cuts {cuts[:3]}")
    runner.cache.check()
    del runner, model
    torch.cuda.empty_cache()


def test_step_refuses_what_it_cannot_run(engines):
    from pulse_infer_amd.engine.runner import StepEntry, StepError

    runner = engines("A", "float32")
    with pytest.raises(StepError, match="at least one entry"):
        runner.step([])
    with pytest.raises(StepError, match="not live"):
        runner.step([StepEntry("nobody", [1], [0])])
    runner.add_request("x")
    try:
        with pytest.raises(StepError, match="reserved"):
            runner.step([StepEntry("x", [1, 2], [0])])
        runner.reserve("x", 2)
        with pytest.raises(StepError, match="outside the vocabulary"):
            runner.step([StepEntry("x", [1, 256], [0])])
        with pytest.raises(StepError, match="wanted place"):
            runner.step([StepEntry("x", [1, 2], [2])])
        with pytest.raises(StepError, match="twice"):
            runner.step([StepEntry("x", [1], []), StepEntry("x", [2], [])])
        with pytest.raises(StepError, match="no tokens"):
            runner.step([StepEntry("x", [], [])])
        assert runner.step([StepEntry("x", [1, 2], [])]).shape == (0, 256)      # nothing wanted: nothing returned
        assert runner.cache.computed("x") == 2
    finally:
        runner.free_request("x")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_program(model_folders, plain_logits, tmp_path, dtype):
    """bin/trace_run as a user runs it: JSON lines in, <step>.f32 files and `done <step>` lines out."""
    name = "B"
    cfg = TINY[name][0]
    ids, steps = mixed_trace(cfg["vocab_size"], seed=7)
    out = tmp_path / "out"
    proc = subprocess.run(
        [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", model_folders[name], "--dtype", dtype,
         "--out", str(out), "--max-tokens", "256"],
        input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert [l for l in proc.stdout.splitlines() if l.startswith("done ")] == [f"done {s['step']}" for s in steps]
    got = {k: [] for k in ids}
    for s in steps:
        data = np.fromfile(out / f"{s['step']}.f32", dtype="<f4").reshape(-1, cfg["vocab_size"])
        assert data.shape[0] == sum(len(e["want"]) for e in s["entries"])
        row = 0
        for e in s["entries"]:
            got[e["id"]].append(torch.from_numpy(data[row:row + len(e["want"])].copy()))
            row += len(e["want"])
    for k, parts in got.items():
        close(torch.cat(parts), plain_logits(name, ids[k]), dtype, f"trace_run request {k}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name,page", [("A", 4), ("B", 16)])
def test_half_pairing_option(model_folders, plain_models, name, page, dtype):
    """``rope_pairing="half"`` (an option of the engine, no key of config.json) rotates (i, i + d/2): whole, then the
    tail token by token (which in bfloat16 rotates inside the decode attention kernel), against the plain
    implementation under the same pairing; and it is another function of the same weights than the default."""
    from plain.qwen3_plain import PlainQwen3
    from pulse_infer_amd.engine.runner import ModelRunner
    from pulse_infer_amd.models.factory import load_model

    cfg = TINY[name][0]
    ids = token_ids(cfg["vocab_size"], 90, seed=8)
    plain = PlainQwen3.from_folder(model_folders[name], pairing="half")
    want = plain.logits(ids)
    config, model = load_model(model_folders[name], mode=dtype, config_overrides={"rope_pairing": "half"})
    assert config.rope_pairing == "half"
    runner = ModelRunner(model, page_size=page, num_pages=256 // page, max_requests=4)
    close(run_alone(runner, ids, [len(ids)]), want, dtype, "whole, half pairing")
    close(run_alone(runner, ids, [len(ids) - 32] + [1] * 32), want, dtype, "tail, half pairing")
    other = plain_models[name].logits(ids)
    assert float((other - want).abs().max()) > 0.05 * float(want.abs().max())
    with pytest.raises(ValueError):
        load_model(model_folders[name], mode=dtype, config_overrides={"no_such_field": 1})


LONG = dict(
    architectures=["Qwen3ForCausalLM"], model_type="qwen3", vocab_size=300, hidden_size=128, intermediate_size=160,
    num_hidden_layers=2, num_attention_heads=4, num_key_value_heads=2, head_dim=64, max_position_embeddings=2048,
    rms_norm_eps=1e-6, rope_theta=1e4, tie_word_embeddings=True, torch_dtype="bfloat16", attention_bias=False,
    use_sliding_window=False, hidden_act="silu")


def test_long_prompts_walk_their_keys_in_splits(tmp_path):
    """A prompt of 1,300 tokens whole, and in portions that come late in a long context: few work items with long
    walks, which the prompt-portion kernel cuts into splits (asserted), against the plain implementation."""
    from plain.qwen3_plain import PlainQwen3
    from pulse_infer_amd.config import Qwen3Config
    from pulse_infer_amd.engine.runner import ModelRunner
    from pulse_infer_amd.models.factory import load_model
    from pulse_infer_amd.ops import attention_mfma as M
    from pulse_infer_amd.weights import write_model_folder

    if not torch.cuda.is_available():
        pytest.skip("no GPU visible")
    folder = write_model_folder(Qwen3Config.from_dict(LONG), str(tmp_path / "m"), seed=31)
    ids = token_ids(LONG["vocab_size"], 1300, seed=12)
    want = PlainQwen3.from_folder(folder).logits(ids)

    class E:
        def __init__(self, start, count):
            self.start, self.count = start, count
    portion = M.portion_tokens(2, 64)
    for start, count in ((0, 1300), (1000, 300), (1236, 64)):
        assert M.choose_prefill_splits([(0, E(start, count))], portion, 2, 2, 64, 0)[1] > 1
    _, model = load_model(folder, mode="bfloat16")
    runner = ModelRunner(model, page_size=16, num_pages=90, max_requests=2)
    whole = run_alone(runner, ids, [1300])
    close(whole, want, "bfloat16", "whole, in splits")
    portions = run_alone(runner, ids, [1000, 236, 64])
    close(portions, want, "bfloat16", "late portions, in splits")
    close(portions, whole, "bfloat16", "late portions against whole", SPLIT_TOL)


WIDE = dict(
    architectures=["Qwen3ForCausalLM"], model_type="qwen3", vocab_size=211, hidden_size=128, intermediate_size=8192,
    num_hidden_layers=2, num_attention_heads=2, num_key_value_heads=1, head_dim=32, max_position_embeddings=512,
    rms_norm_eps=1e-6, rope_theta=1e4, tie_word_embeddings=False, torch_dtype="bfloat16", attention_bias=False,
    use_sliding_window=False, hidden_act="silu")


def test_a_wide_feed_forward_shares_out_its_down_product(tmp_path):
    """An intermediate size of 8,192 and prompts of a few hundred tokens: the down product runs as the library's
    batch over shares of its inner dimension (asserted), and the norms, the last one with gathered rows too, add the
    shares up; whole, in portions and with a decoded tail, against the plain implementation."""
    from plain.qwen3_plain import PlainQwen3
    from pulse_infer_amd.config import Qwen3Config
    from pulse_infer_amd.engine.runner import ModelRunner, StepEntry
    from pulse_infer_amd.models.factory import load_model
    from pulse_infer_amd.weights import write_model_folder

    if not torch.cuda.is_available():
        pytest.skip("no GPU visible")
    folder = write_model_folder(Qwen3Config.from_dict(WIDE), str(tmp_path / "m"), seed=41)
    ids = token_ids(WIDE["vocab_size"], 400, seed=13)
    want = PlainQwen3.from_folder(folder).logits(ids)
    _, model = load_model(folder, mode="bfloat16")
    down = model.blocks[0].ffn.down
    assert down.library_shares_for(torch.empty(400, 8192, dtype=torch.bfloat16, device=model.device)) == 4
    runner = ModelRunner(model, page_size=16, num_pages=40, max_requests=2)
    whole = run_alone(runner, ids, [400])
    close(whole, want, "bfloat16", "whole, down in shares")
    cut = run_alone(runner, ids, [250, 118] + [1] * 32)
    close(cut, want, "bfloat16", "portions and a tail, down in shares")
    # only the last row wanted: the final norm gathers rows of a residual whose last update is still in shares
    runner.add_request("g")
    runner.reserve("g", 400)
    last = runner.step([StepEntry("g", ids, [399, 7])])
    runner.free_request("g")
    close(last, want[[399, 7]], "bfloat16", "gathered rows, down in shares")


MANY = dict(
    architectures=["Qwen3ForCausalLM"], model_type="qwen3", vocab_size=300, hidden_size=256, intermediate_size=512,
    num_hidden_layers=2, num_attention_heads=4, num_key_value_heads=2, head_dim=64, max_position_embeddings=256,
    rms_norm_eps=1e-6, rope_theta=1e4, tie_word_embeddings=False, torch_dtype="bfloat16", attention_bias=False,
    use_sliding_window=False, hidden_act="silu")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("requests", [14, 24, 70, 200])
def test_many_requests_decode_together(tmp_path, requests, dtype):
    """Steps of 14, 24, 70 and 200 decoded tokens (the products for up to 16 and for 17 to 192 rows and the library's beyond, attention
    over many short contexts of different lengths): every request's logits are those of the plain implementation
    for its own sequence, whatever stands beside it."""
    from plain.qwen3_plain import PlainQwen3
    from pulse_infer_amd.config import Qwen3Config
    from pulse_infer_amd.engine.runner import ModelRunner, StepEntry
    from pulse_infer_amd.models.factory import load_model
    from pulse_infer_amd.weights import write_model_folder

    if not torch.cuda.is_available():
        pytest.skip("no GPU visible")
    folder = write_model_folder(Qwen3Config.from_dict(MANY), str(tmp_path / "m"), seed=51)
    plain = PlainQwen3.from_folder(folder)
    steps = 4
    lengths = [1 + (7 * i) % 40 for i in range(requests)]
    ids = [token_ids(MANY["vocab_size"], n + steps, seed=100 + i) for i, n in enumerate(lengths)]
    _, model = load_model(folder, mode=dtype)
    runner = ModelRunner(model, page_size=16, num_pages=requests * 4, max_requests=requests)
    for i in range(0, requests, 8):          # prompts, eight requests a step
        batch = []
        for r in range(i, min(i + 8, requests)):
            runner.add_request(r)
            runner.reserve(r, lengths[r] + steps)
            batch.append(StepEntry(r, ids[r][:lengths[r]], []))
        runner.step(batch)
    got = []
    for s in range(steps):                   # then every request's next token in one step
        got.append(runner.step([StepEntry(r, [ids[r][lengths[r] + s]], [0]) for r in range(requests)]))
    for r in range(0, requests, max(1, requests // 12)):
        want = plain.logits(ids[r])[lengths[r]:]
        mine = torch.stack([g[r] for g in got])
        close(mine, want, dtype, f"request {r} of {requests}")
    for r in range(requests):
        runner.free_request(r)
    runner.cache.check()
