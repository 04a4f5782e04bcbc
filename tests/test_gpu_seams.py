"""The seams for another architecture, shown with toys that live in this file alone: a mixer that pages ONE row of
some width per token (a cache spec class of its own: what the manager allocates and what view a run gets are the
spec's answers), an embedding that scales its rows and an output head with a bias (looked up by kind like every other
part).  The toy architecture is registered, loaded from a folder, stepped in mixed batches with page reuse, and run
through ``LLM`` and the command line, against plain formulas.  The toys are torch code: they show interfaces, they are
no kernels and no model of anyone's."""
import json
from dataclasses import dataclass
from typing import Optional

import pytest
import torch

from conftest import token_ids
from plain import qwen3_plain as P

pytestmark = pytest.mark.gpu
F64 = torch.float64

ROWS = dict(architectures=["RowsForCausalLM"], vocab=157, width=64, depth=3, latent=24, inner=96, heads=4, kv_heads=2,
            head_width=16, most_positions=256, eps=3e-6, theta=2e4, row_window=11, scale=1.7)


@pytest.fixture(scope="module")
def gpu():
    if not torch.cuda.is_available():
        pytest.skip("no GPU visible")


@dataclass(frozen=True)
class PagedRowSpec:
    """One float32 row of ``width`` per token, in pages: [runs, pages, page, width]."""

    width: int
    window: Optional[int] = None
    per_token = True

    def bytes_per_token(self, element_size):
        return 4 * self.width

    def allocate(self, runs, units, page_size, device, dtype):
        return torch.full((runs, units, page_size, self.width), float("nan"), dtype=torch.float32, device=device)

    def view(self, storage, index, group, page_size, writable):
        return RowsView(storage[index], group, page_size)

    def tensors(self, storage):
        return [storage]


@dataclass
class RowsView:
    rows: torch.Tensor      # [pages, page, width]
    group: int
    page_size: int


def register_row_toys():
    from pulse_infer_amd.config import JsonReader, ModelConfig, register_architecture
    from pulse_infer_amd.models.spec import LayerSpec, ModelSpec, PartSpec, RunSpec
    from pulse_infer_amd.parts.base import EMBEDDINGS, HEADS, MIXERS, Part
    from pulse_infer_amd.parts.linear import Linear
    from pulse_infer_amd.weights import TensorSpec

    @MIXERS.register("toy_paged_rows", replace=True)
    class PagedRows(Part):
        """c_t = x_t A^T is written to the token's place in the request's pages; the output is the mean of the rows
        c_j of the keys j <= t (of the last ``window`` of them), times B^T."""

        @classmethod
        def weight_specs(cls, params):
            h, w = params["hidden_size"], params["latent"]
            return {"in.weight": TensorSpec((w, h), fan_in=h), "out.weight": TensorSpec((h, w), fan_in=w)}

        def __init__(self, params, prefix, build):
            self.latent, self.window = params["latent"], params["window"]
            self.a = build.loader.get(f"{prefix}.in.weight").float()
            self.b = build.loader.get(f"{prefix}.out.weight").float()
            self.act = build.act_dtype

        def cache_spec(self):
            return PagedRowSpec(self.latent, self.window)

        def forward(self, x, ctx, cache):
            c = x.float() @ self.a.t()
            table = ctx.block_tables[cache.group]
            page = cache.page_size
            out = torch.empty(x.shape[0], self.latent, dtype=torch.float32, device=x.device)
            for i, e in enumerate(ctx.entries):
                new = torch.arange(e.start, e.start + e.count, device=x.device)
                cache.rows[table[i, new // page].long(), new % page] = c[e.first_row:e.first_row + e.count]
                lowest = 0 if self.window is None else max(0, e.start - self.window + 1)
                held = torch.arange(lowest, e.start + e.count, device=x.device)
                rows = cache.rows[table[i, held // page].long(), held % page]
                for t in range(e.count):
                    p = e.start + t
                    lo = 0 if self.window is None else max(0, p - self.window + 1)
                    out[e.first_row + t] = rows[lo - lowest:p + 1 - lowest].mean(dim=0)
            return (out @ self.b.t()).to(self.act)

    @EMBEDDINGS.register("toy_scaled_embedding", replace=True)
    class ScaledEmbedding(Part):
        @classmethod
        def weight_specs(cls, params):
            return {params["name"]: TensorSpec((params["vocab_size"], params["hidden_size"]), kind="embedding",
                                               fan_in=params["hidden_size"])}

        def __init__(self, params, build):
            self.table = build.loader.get(params["name"]).float()
            self.scale = params["scale"]

        def forward(self, ids, out):
            out.copy_(self.table.index_select(0, ids.long()) * self.scale)
            return out

    @HEADS.register("toy_biased_head", replace=True)
    class BiasedHead(Part):
        @classmethod
        def weight_specs(cls, params):
            return {params["name"]: TensorSpec((params["vocab_size"], params["hidden_size"]), fan_in=params["hidden_size"]),
                    params["bias"]: TensorSpec((params["vocab_size"],), kind="norm")}

        def __init__(self, params, build, embedding):
            self.linear = Linear(build.loader.get(params["name"]), build.mode)
            self.bias = build.loader.get(params["bias"]).float()

        def forward(self, x, out):
            self.linear.forward(x, out)
            out.add_(self.bias)
            return out

    @dataclass
    class RowsConfig(ModelConfig):
        vocab_size: int
        width: int
        depth: int
        latent: int
        inner: int
        heads: int
        kv_heads: int
        head_width: int
        most_positions: int
        eps: float
        theta: float
        row_window: int
        scale: float
        architecture: str = "RowsForCausalLM"

        @classmethod
        def from_dict(cls, data, origin="<dict>", generation=None, generation_origin="<dict>"):
            r = JsonReader(data, origin)
            cfg = cls(vocab_size=r.integer("vocab"), width=r.integer("width"), depth=r.integer("depth"),
                      latent=r.integer("latent"), inner=r.integer("inner"), heads=r.integer("heads"),
                      kv_heads=r.integer("kv_heads"), head_width=r.integer("head_width"),
                      most_positions=r.integer("most_positions"), eps=r.number("eps"), theta=r.number("theta"),
                      row_window=r.integer("row_window"), scale=r.number("scale"))
            cfg.read_generation_defaults(generation, generation_origin)
            cfg.validate(origin)
            return cfg

        def validate(self, origin="<config>"):
            pass

        def to_dict(self):
            return dict(architectures=[self.architecture], vocab=self.vocab_size, width=self.width, depth=self.depth,
                        latent=self.latent, inner=self.inner, heads=self.heads, kv_heads=self.kv_heads,
                        head_width=self.head_width, most_positions=self.most_positions, eps=self.eps, theta=self.theta,
                        row_window=self.row_window, scale=self.scale)

        def model_spec(self):
            rms = PartSpec("rmsnorm", {"size": self.width, "eps": self.eps})
            ffn = PartSpec("gated_mlp", {"hidden_size": self.width, "intermediate_size": self.inner, "prefix": "mlp"})
            layers = []
            for i in range(self.depth):
                if i % 2 == 0:      # rows of all keys in layer 0, of a window in layer 2: two groups of pages
                    mixer = PartSpec("toy_paged_rows", {"hidden_size": self.width, "latent": self.latent,
                                                        "window": self.row_window if i else None, "prefix": "rows"})
                else:
                    mixer = PartSpec("attention", {
                        "hidden_size": self.width, "num_heads": self.heads, "num_kv_heads": self.kv_heads,
                        "head_dim": self.head_width, "qk_norm": True, "qk_norm_eps": self.eps,
                        "scale": self.head_width ** -0.5, "window": None, "position": "rope", "prefix": "self_attn"})
                layers.append(LayerSpec(f"model.layers.{i}", mixer, ffn, {"mixer_norm": rms, "ffn_norm": rms}))
            return ModelSpec(
                architecture=self.architecture, vocab_size=self.vocab_size, hidden_size=self.width,
                max_positions=self.most_positions,
                embedding=PartSpec("toy_scaled_embedding", {"vocab_size": self.vocab_size, "hidden_size": self.width,
                                                            "name": "model.embed_tokens.weight", "scale": self.scale}),
                layers=layers, order=[RunSpec(i) for i in range(self.depth)], final_norm=rms,
                head=PartSpec("toy_biased_head", {"vocab_size": self.vocab_size, "hidden_size": self.width,
                                                  "name": "lm_head.weight", "bias": "lm_head.bias"}),
                positions={"rope": PartSpec("rope", {"theta": self.theta, "rotary_dim": self.head_width,
                                                     "head_dim": self.head_width, "pairing": "interleaved"})})

    register_architecture("RowsForCausalLM", RowsConfig, replace=True)
    return RowsConfig


def unregister_row_toys():
    from pulse_infer_amd.config import unregister_architecture
    from pulse_infer_amd.parts.base import EMBEDDINGS, HEADS, MIXERS

    unregister_architecture("RowsForCausalLM")
    MIXERS.unregister("toy_paged_rows")
    EMBEDDINGS.unregister("toy_scaled_embedding")
    HEADS.unregister("toy_biased_head")


def rows_plain(folder):
    from safetensors.torch import load_file
    c = dict(num_attention_heads=ROWS["heads"], num_key_value_heads=ROWS["kv_heads"], head_dim=ROWS["head_width"],
             hidden_size=ROWS["width"], rms_norm_eps=ROWS["eps"], rope_theta=ROWS["theta"],
             num_hidden_layers=ROWS["depth"], vocab_size=ROWS["vocab"])
    return P.PlainQwen3(c, load_file(f"{folder}/model.safetensors"))


def plain_rows_logits(plain, ids):
    c, w = plain.c, plain.w
    h = P.embedding(w["model.embed_tokens.weight"], ids) * ROWS["scale"]
    pos = list(range(len(ids)))
    for i in range(c["num_hidden_layers"]):
        if i % 2 == 1:
            h = plain.layer(h, i, pos)
            continue
        p = f"model.layers.{i}."
        a = P.rms_norm(h, w[p + "input_layernorm.weight"], c["rms_norm_eps"])
        rows = a @ w[p + "rows.in.weight"].T
        window = ROWS["row_window"] if i else None
        mixed = torch.stack([rows[(0 if window is None else max(0, t - window + 1)):t + 1].mean(dim=0)
                             for t in range(len(ids))])
        h = h + mixed @ w[p + "rows.out.weight"].T
        m = P.rms_norm(h, w[p + "post_attention_layernorm.weight"], c["rms_norm_eps"])
        h = h + P.gated_mlp(m, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"], w[p + "mlp.down_proj.weight"])
    return P.linear(P.rms_norm(h, w["model.norm.weight"], c["rms_norm_eps"]), w["lm_head.weight"]) + w["lm_head.bias"]


def plain_rows_greedy(plain, prompt, steps):
    ids, out = list(prompt), []
    for _ in range(steps):
        out.append(int(torch.argmax(plain_rows_logits(plain, ids)[-1])))
        ids.append(out[-1])
    return out


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_mixer_that_pages_rows_of_its_own_and_a_biased_head_step_in_mixed_batches(gpu, tmp_path, dtype):
    from pulse_infer_amd.engine.runner import ModelRunner
    from pulse_infer_amd.models.factory import load_model
    from pulse_infer_amd.parts.base import EntryMeta
    from pulse_infer_amd.weights import write_model_folder
    from test_gpu_model import close, mixed_trace, pages_were_used_again, run_mixed

    config_class = register_row_toys()
    try:
        folder = write_model_folder(config_class.from_dict(ROWS), str(tmp_path / "rows"), seed=71)
        plain = rows_plain(folder)
        config, model = load_model(folder, mode=dtype)
        assert type(config) is config_class
        assert type(model.embedding).__name__ == "ScaledEmbedding" and type(model.head).__name__ == "BiasedHead"
        runner = ModelRunner(model, page_size=16, num_pages=16, max_requests=4)
        specs = [g.spec for g in runner.cache.groups]
        assert [type(s).__name__ for s in specs] == ["PagedRowSpec", "PagedKVSpec", "PagedRowSpec"]
        assert (specs[0].window, specs[2].window) == (None, ROWS["row_window"])
        assert runner.views[0].rows.shape == (16, 16, ROWS["latent"]) and runner.views[1].keys.shape[0] == 16
        assert not model.recordable([EntryMeta("r", 0, 3, 1, 0)])           # a part did not say that it records
        ids, steps = mixed_trace(ROWS["vocab"], seed=6)
        got, pages_seen, most_live = run_mixed(runner, steps)
        assert most_live == 4 and pages_were_used_again(pages_seen)
        windowed = runner.cache.groups[2]
        assert windowed.pool.high_water < runner.cache.groups[0].pool.high_water   # the window gave pages back
        for k, mine in got.items():
            close(mine, plain_rows_logits(plain, ids[k]), dtype, f"rows toy, mixed request {k}")
        assert runner.graph_records == 0
    finally:
        unregister_row_toys()


def test_the_row_toy_runs_through_the_entry_points(gpu, tmp_path, capsys):
    from pulse_infer_amd import LLM, cli
    from pulse_infer_amd.weights import write_model_folder

    config_class = register_row_toys()
    try:
        folder = write_model_folder(config_class.from_dict(ROWS), str(tmp_path / "rows"), seed=73)
        plain = rows_plain(folder)
        prompts = [token_ids(ROWS["vocab"], n, seed=50 + n) for n in (7, 26, 13)]
        llm = LLM.from_pretrained(folder, dtype="float32", max_batch_size=3, chunk_size=8, page_size=16, num_pages=12)
        assert llm.generate(prompts, max_new_tokens=6, ignore_eos=True) == [plain_rows_greedy(plain, p, 6) for p in prompts]
        llm.engine.runner.cache.check()
        assert all(g.pool.num_held == 0 for g in llm.engine.runner.cache.groups)
        code = cli.main([folder, "--dtype", "f32", "--prompt-ids", ",".join(map(str, prompts[1])), "--max-new-tokens",
                         "4", "--num-pages", "16", "--ignore-eos"])
        assert code == 0
        assert json.loads(capsys.readouterr().out.splitlines()[0])["output_ids"] == plain_rows_greedy(plain, prompts[1], 4)
    finally:
        unregister_row_toys()
