"""Each part alone against its plain formula, models whose order names a layer twice or shares a cache,
and toy parts (a mixer with state of its own, a feed-forward that routes tokens to experts, another position
encoding) that are registered, built and stepped from here without a change to the framework's files."""
import math

import pytest
import torch

from conftest import token_ids
from plain import qwen3_plain as P

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
F64 = torch.float64


@pytest.fixture(scope="module")
def gpu():
    if not torch.cuda.is_available():
        pytest.skip("no GPU visible")


def rnd(*shape, seed=0, scale=1.0):
    return (torch.randn(*shape, generator=torch.Generator().manual_seed(seed)) * scale).to(torch.bfloat16)


def build_ctx(tensors, mode, positions=None):
    from pulse_infer_amd.parts.base import BuildContext, Workspace
    from pulse_infer_amd.weights import DictSource, TensorSpec, WeightLoader
    expected = {n: TensorSpec(tuple(t.shape)) for n, t in tensors.items()}
    loader = WeightLoader(DictSource(tensors), expected, mode, DEV)
    act = torch.float32 if mode == "float32" else torch.bfloat16
    return BuildContext(loader=loader, mode=mode, device=torch.device(DEV), act_dtype=act,
                        workspace=Workspace(torch.device(DEV)), positions=positions or {})


def step_ctx(build, positions, entry, tables, counts=None):
    from pulse_infer_amd.parts.base import EntryMeta, StepContext
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)
    n_entries = max(entry) + 1
    starts = [min(p for p, e in zip(positions, entry) if e == i) for i in range(n_entries)]
    counts = [entry.count(i) for i in range(n_entries)]
    first = [entry.index(i) for i in range(n_entries)]
    metas = [EntryMeta(i, i, starts[i], counts[i], first[i]) for i in range(n_entries)]
    return StepContext(num_tokens=len(positions), entries=metas, token_ids=i32([0] * len(positions)),
                       positions=i32(positions), token_entry=i32(entry), entry_start=i32(starts),
                       entry_count=i32(counts), entry_first_row=i32(first + [len(positions)]),
                       entry_slot=i32(list(range(n_entries))), block_tables={0: i32(tables)},
                       want_rows=i32([]), num_wanted=0, workspace=build.workspace,
                       max_count=max(counts), max_context=max(positions) + 1)


TOL = {"float32": dict(atol=3e-5, rtol=3e-5), "bfloat16": dict(atol=3e-2, rtol=3e-2)}


@pytest.mark.parametrize("mode", ["float32", "bfloat16"])
def test_norm_part(gpu, mode):
    from pulse_infer_amd.parts.base import NORMS
    w = (1 + 0.1 * rnd(70, seed=1).float()).to(torch.bfloat16)
    build = build_ctx({"n.weight": w}, mode)
    norm = NORMS.get("rmsnorm")({"size": 70, "eps": 1e-4}, "n", build)
    h = torch.randn(5, 70, generator=torch.Generator().manual_seed(2)).to(DEV)
    out = torch.empty(5, 70, dtype=build.act_dtype, device=DEV)
    norm.apply(h, None, out)
    assert torch.allclose(out.cpu().to(F64), P.rms_norm(h.cpu().to(F64), w.to(F64), 1e-4), **TOL[mode])


@pytest.mark.parametrize("rows,n,splits", [(300, 768, 4), (700, 768, 4), (1800, 2048, 2)])
def test_linear_adds_into_the_residual_through_shares_of_the_library_product(gpu, rows, n, splits, monkeypatch):
    """Many rows, a wide inner dimension and few output tiles: ``Linear.add_into`` runs the library's product as a
    batch over shares of the inner dimension and hands back their float32 results, which the norm's kernel (and the
    plain addition) add to the residual in order."""
    from pulse_infer_amd.ops import kernels
    from pulse_infer_amd.parts.base import Workspace
    from pulse_infer_amd.parts import linear
    from pulse_infer_amd.parts.linear import Linear
    monkeypatch.setattr(linear, "OWN_MANY_ROWS", "none")      # (whatever PULSE_OWN_PRODUCTS says)
    k = 8192
    w = rnd(n, k, seed=3, scale=k ** -0.5).to(DEV)
    x = rnd(rows, k, seed=4).to(DEV)
    lin = Linear(w, "bfloat16")
    assert lin.library_shares_for(x) == splits
    h = torch.randn(rows, n, generator=torch.Generator().manual_seed(5)).to(DEV)
    parts = lin.add_into(x, h, torch.empty(rows, n, dtype=torch.bfloat16, device=DEV), Workspace(torch.device(DEV)))
    assert parts.shape == (splits, rows, n) and parts.dtype == torch.float32
    want = x.double() @ w.double().T
    assert torch.allclose(parts.double().sum(0), want, atol=2e-3, rtol=2e-3)
    share = k // splits
    assert torch.allclose(parts[1].double(), x[:, share:2 * share].double() @ w[:, share:2 * share].double().T,
                          atol=2e-3, rtol=2e-3)
    norm_w = torch.ones(n, dtype=torch.bfloat16, device=DEV)
    out = torch.empty(rows, n, dtype=torch.bfloat16, device=DEV)
    h2 = h.clone()
    kernels.add_rmsnorm(h2, parts, norm_w, 1e-6, out)
    assert torch.allclose(h2.double(), h.double() + want, atol=3e-3, rtol=3e-3)
    h3 = h.clone()
    kernels.residual_add(h3, parts)
    assert torch.equal(h3, h2)


@pytest.mark.parametrize("mode", ["float32", "bfloat16"])
def test_feed_forward_part(gpu, mode):
    from pulse_infer_amd.parts.base import FEED_FORWARDS
    hidden, inter = 72, 200
    ws = {"m.gate_proj.weight": rnd(inter, hidden, seed=3, scale=hidden ** -0.5),
          "m.up_proj.weight": rnd(inter, hidden, seed=4, scale=hidden ** -0.5),
          "m.down_proj.weight": rnd(hidden, inter, seed=5, scale=inter ** -0.5)}
    build = build_ctx(ws, mode)
    mlp = FEED_FORWARDS.get("gated_mlp")({"hidden_size": hidden, "intermediate_size": inter, "activation": "silu"}, "m", build)
    x = rnd(9, hidden, seed=6).to(build.act_dtype).to(DEV)
    ctx = step_ctx(build, list(range(9)), [0] * 9, [[0]])
    out = mlp.forward(x, ctx)
    want = P.gated_mlp(x.cpu().to(F64), *(ws[f"m.{n}_proj.weight"].to(F64) for n in ("gate", "up", "down")))
    assert torch.allclose(out.cpu().to(F64), want, **TOL[mode])
    with pytest.raises(ValueError, match="activation"):
        FEED_FORWARDS.get("gated_mlp")({"hidden_size": hidden, "intermediate_size": inter, "activation": "relu"}, "m", build)


@pytest.mark.parametrize("policy", ["none", "swiglu", "all"])
@pytest.mark.parametrize("rows", [300, 700])
def test_feed_forward_part_at_many_rows_under_each_choice_of_products(gpu, rows, policy, monkeypatch):
    """A prompt portion of some hundred rows through the feed-forward with the library's products, with gate and up
    in this package's tiled product (SwiGLU inside), and with every product in it (the way back in shares of the
    inner dimension, float32 results that are added to the residual in order): all against float64, and the last
    one without a library call."""
    from pulse_infer_amd.ops import kernels
    from pulse_infer_amd.parts import linear
    from pulse_infer_amd.parts.base import FEED_FORWARDS
    monkeypatch.setattr(linear, "OWN_MANY_ROWS", policy)
    hidden, inter = 192, 448
    ws = {"m.gate_proj.weight": rnd(inter, hidden, seed=3, scale=hidden ** -0.5),
          "m.up_proj.weight": rnd(inter, hidden, seed=4, scale=hidden ** -0.5),
          "m.down_proj.weight": rnd(hidden, inter, seed=5, scale=inter ** -0.5)}
    build = build_ctx(ws, "bfloat16")
    mlp = FEED_FORWARDS.get("gated_mlp")({"hidden_size": hidden, "intermediate_size": inter, "activation": "silu"}, "m", build)
    x = rnd(rows, hidden, seed=6).to(build.act_dtype).to(DEV)
    ctx = step_ctx(build, list(range(rows)), [0] * rows, [[0]])
    assert mlp.gate_up.takes_tiles(x, swiglu=True) == (policy != "none")
    assert mlp.down.takes_tiles(torch.empty(rows, inter, dtype=torch.bfloat16, device=DEV)) == (policy == "all")
    before = linear.library_calls
    h0 = rnd(rows, hidden, seed=7).float().to(DEV)
    h = h0.clone()
    update = mlp.forward(x, ctx, residual=h)
    assert linear.library_calls - before == {"none": 2, "swiglu": 1, "all": 0}[policy]
    w64 = [ws[f"m.{n}_proj.weight"].to(torch.bfloat16).to(F64) for n in ("gate", "up", "down")]
    want = P.gated_mlp(x.cpu().to(F64), *w64)
    if policy == "all":
        assert update.dim() == 3 and update.dtype == torch.float32       # shares of the inner dimension
    kernels.residual_add(h, update)
    assert torch.allclose(h.cpu().to(F64) - h0.cpu().to(F64), want, **TOL["bfloat16"])


@pytest.mark.parametrize("rows", [1, 7, 16, 20])
def test_a_norm_is_finished_behind_the_product_that_consumes_it(gpu, rows):
    """The protocol that takes the norm kernels out of a decoding step, on real parts of a width the fused products
    take: the product that adds into the residual is told the weight of the norm that reads the residual next and
    leaves, beside the new rows, their sums of squares and a rounded copy with that weight multiplied in; the norm
    recognises its weight in them and hands the feed-forward rows that are only divided by their root mean square
    behind its first product.  The norm's weights are far from 1 and differ by column, so that a weight applied twice,
    not at all or to the wrong operand shows."""
    from pulse_infer_amd.ops import kernels
    from pulse_infer_amd.parts.base import FEED_FORWARDS, NORMS, LazyNorm, ResidualStream, RowStats
    from pulse_infer_amd.parts.linear import Linear
    hidden, inter, inner, eps, mode = 1024, 96, 2048, 1e-5, "bfloat16"
    nw = (torch.linspace(0.25, 4.0, hidden) * torch.tensor([1.0, -1.0]).repeat(hidden // 2)).to(torch.bfloat16)
    ws = {"m.gate_proj.weight": rnd(inter, hidden, seed=3, scale=hidden ** -0.5),
          "m.up_proj.weight": rnd(inter, hidden, seed=4, scale=hidden ** -0.5),
          "m.down_proj.weight": rnd(hidden, inter, seed=5, scale=inter ** -0.5), "n.weight": nw, "other.weight": nw.clone()}
    build = build_ctx(ws, mode)
    mlp = FEED_FORWARDS.get("gated_mlp")({"hidden_size": hidden, "intermediate_size": inter, "activation": "silu"}, "m", build)
    norm = NORMS.get("rmsnorm")({"size": hidden, "eps": eps}, "n", build)
    other = NORMS.get("rmsnorm")({"size": hidden, "eps": eps}, "other", build)
    # the product before: h += a o^T, told who reads h next
    o = Linear(rnd(hidden, inner, seed=7, scale=inner ** -0.5).to(DEV), mode)
    a = rnd(rows, inner, seed=8).to(DEV)
    h = (torch.randn(rows, hidden, generator=torch.Generator().manual_seed(6)) * 3).to(DEV)
    before = h.clone()
    scratch = torch.empty(rows, hidden, dtype=torch.bfloat16, device=DEV)
    left = o.add_into(a, h, scratch, build.workspace, next_scale=norm.column_scale())
    ctx = step_ctx(build, list(range(rows)), [0] * rows, [[0]])
    if rows > kernels.SKINNY_FAST_ROWS:
        assert not isinstance(left, RowStats)          # more rows: an update in parts, which the norm's kernel adds up
        return
    assert isinstance(left, RowStats) and left.scaled_by is norm.weight
    assert torch.allclose(h.double(), before.double() + a.double() @ o.weight.double().T, atol=1e-3, rtol=1e-4)
    assert torch.equal(left.rounded, (h * nw.to(DEV).float()).to(torch.bfloat16))       # the weight is in, rounded once
    want_sums = (h.double() ** 2).view(rows, hidden // 16, 16).sum(-1)
    assert torch.allclose(left.sumsq.double(), want_sums, rtol=1e-5, atol=1e-6)
    want = P.gated_mlp(P.rms_norm(h.cpu().to(F64), nw.to(F64), eps),
                       *(ws[f"m.{n}_proj.weight"].to(F64) for n in ("gate", "up", "down")))
    scale = float(want.abs().max())
    stream = ResidualStream(h)
    stream.push(left)
    assert stream.lazy(other) is None                  # a norm with another weight does not take them for its own
    lazy = stream.lazy(norm)
    assert isinstance(lazy, LazyNorm) and mlp.gate_up.takes_lazy(lazy)
    out = mlp.forward(lazy, ctx)
    assert float((out.cpu().to(F64) - want).abs().max()) <= 3e-2 * scale
    # the ordinary way gives the same within rounding
    x = torch.empty(rows, hidden, dtype=build.act_dtype, device=DEV)
    norm.apply(h, None, x)
    plain_way = mlp.forward(x, ctx)
    assert float((out.float() - plain_way.float()).abs().max()) <= 2e-2 * scale
    # rows left as they are (nobody said who reads next) are nobody's
    left = o.add_into(a, h, scratch, build.workspace)
    assert isinstance(left, RowStats) and left.scaled_by is None
    stream.push(left)
    assert stream.lazy(norm) is None


@pytest.mark.parametrize("mode", ["float32", "bfloat16"])
@pytest.mark.parametrize("variant", ["qwen", "half_partial_window", "no_position_no_norm"])
def test_attention_part(gpu, mode, variant):
    """The mixer alone over a cache it fills in two steps (a portion, then another portion and a single token
    of a second request), against plain attention on the whole sequences."""
    from pulse_infer_amd.parts.base import MIXERS, POSITIONS, PagedCacheView
    hidden, nq, nkv, d, bs = 40, 6, 3, 16, 4
    opts = {"qwen": dict(qk_norm=True, window=None, position="rope", rot=16, pairing="interleaved"),
            "half_partial_window": dict(qk_norm=True, window=5, position="rope", rot=8, pairing="half"),
            "no_position_no_norm": dict(qk_norm=False, window=None, position=None, rot=0, pairing="interleaved")}[variant]
    ws = {"a.q_proj.weight": rnd(nq * d, hidden, seed=7, scale=hidden ** -0.5),
          "a.k_proj.weight": rnd(nkv * d, hidden, seed=8, scale=hidden ** -0.5),
          "a.v_proj.weight": rnd(nkv * d, hidden, seed=9, scale=hidden ** -0.5),
          "a.o_proj.weight": rnd(hidden, nq * d, seed=10, scale=(nq * d) ** -0.5)}
    if opts["qk_norm"]:
        ws["a.q_norm.weight"] = (1 + 0.1 * rnd(d, seed=11).float()).to(torch.bfloat16)
        ws["a.k_norm.weight"] = (1 + 0.1 * rnd(d, seed=12).float()).to(torch.bfloat16)
    build = build_ctx(ws, mode)
    theta, eps, scale = 3e3, 1e-5, 0.29
    if opts["position"]:
        build.positions["rope"] = POSITIONS.get("rope")(
            {"theta": theta, "rotary_dim": opts["rot"], "head_dim": d, "pairing": opts["pairing"]}, build)
    params = {"hidden_size": hidden, "num_heads": nq, "num_kv_heads": nkv, "head_dim": d, "qk_norm": opts["qk_norm"],
              "qk_norm_eps": eps, "scale": scale, "window": opts["window"], "position": opts["position"]}
    attn = MIXERS.get("attention")(params, "a", build)
    spec = attn.cache_spec()
    assert (spec.num_kv_heads, spec.head_dim, spec.window) == (nkv, d, opts["window"])
    cache = PagedCacheView(0, torch.zeros(8, nkv, bs, d, dtype=build.act_dtype, device=DEV),
                           torch.zeros(8, nkv, d, bs, dtype=build.act_dtype, device=DEV), bs)
    xa, xb = rnd(11, hidden, seed=13), rnd(1, hidden, seed=14)
    tables = [[5, 2, 7], [3, -1, -1]]
    dev = lambda t: t.to(build.act_dtype).to(DEV)
    out1 = attn.forward(dev(xa[:6]), step_ctx(build, list(range(6)), [0] * 6, tables[:1]), cache).clone()
    out2 = attn.forward(dev(torch.cat([xa[6:], xb])), step_ctx(build, list(range(6, 11)) + [0], [0] * 5 + [1], tables), cache)
    got = torch.cat([out1, out2]).cpu().to(F64)

    def plain(x):
        t = x.shape[0]
        x = x.to(F64)
        q = P.linear(x, ws["a.q_proj.weight"].to(F64)).view(t, nq, d)
        k = P.linear(x, ws["a.k_proj.weight"].to(F64)).view(t, nkv, d)
        v = P.linear(x, ws["a.v_proj.weight"].to(F64)).view(t, nkv, d)
        if opts["qk_norm"]:
            q, k = P.rms_norm(q, ws["a.q_norm.weight"].to(F64), eps), P.rms_norm(k, ws["a.k_norm.weight"].to(F64), eps)
        if opts["position"]:
            q, k = (P.rope(z, list(range(t)), theta, opts["rot"], opts["pairing"]) for z in (q, k))
        o = P.causal_attention(q, k, v, scale, opts["window"])
        return P.linear(o.reshape(t, nq * d), ws["a.o_proj.weight"].to(F64))

    want = torch.cat([plain(xa), plain(xb)])
    assert torch.allclose(got, want, **TOL[mode])


# ----------------------------------------------------------------- toy parts
TOY = dict(architectures=["ToyForCausalLM"], vocab=211, width=96, depth=4, heads=6, kv_heads=2, head_width=32, inner=160,
           most_positions=256, eps=2e-6, theta=3e4, decay=0.5)


def register_toys():
    """An architecture of its own: a configuration class with keys of its own (it derives from the engine's
    ``ModelConfig`` only), a mixer with state of its own (a decayed running sum per request) in its odd layers,
    whose feed-forward norm is of another kind than the layer's other norm (a toy norm that centres the row first),
    beside ordinary attention layers."""
    from dataclasses import dataclass
    from pulse_infer_amd.cache import StateSpec
    from pulse_infer_amd.config import ConfigError, JsonReader, ModelConfig, register_architecture
    from pulse_infer_amd.models.spec import LayerSpec, ModelSpec, PartSpec, RunSpec
    from pulse_infer_amd.ops import kernels
    from pulse_infer_amd.parts.base import MIXERS, NORMS, Part
    from pulse_infer_amd.weights import TensorSpec

    @MIXERS.register("toy_running_sum", replace=True)
    class RunningSum(Part):
        """state <- decay * state + x_t, output_t = state W^T; the state lives in the request's slot.  A step of single
        tokens reads slots and starts from the step's device arrays only, so it records cleanly."""

        records_cleanly = True

        @classmethod
        def weight_specs(cls, params):
            return {"mix.weight": TensorSpec((params["hidden_size"], params["hidden_size"]), fan_in=params["hidden_size"])}

        def __init__(self, params, prefix, build):
            self.hidden, self.decay = params["hidden_size"], params["decay"]
            self.weight = build.loader.get(f"{prefix}.mix.weight").float()
            self.act = build.act_dtype

        def cache_spec(self):
            return StateSpec((self.hidden,), "float32")

        def forward(self, x, ctx, cache):
            out = torch.empty(x.shape[0], self.hidden, dtype=torch.float32, device=x.device)
            if ctx.max_count == 1:                     # one token a request: no host value decides anything
                slots = ctx.entry_slot.long()
                old = cache.state.index_select(0, slots)
                old = torch.where((ctx.entry_start == 0).unsqueeze(1), torch.zeros_like(old), old)
                new = old * self.decay + x.float()
                cache.state.index_copy_(0, slots, new)
                kernels.gemm_f32(new, self.weight, out)
                return out.to(self.act)
            for e in ctx.entries:
                state = cache.state[e.slot]
                if e.start == 0:
                    state.zero_()                 # a request (re)starts: its slot may hold an older request's state
                for row in range(e.first_row, e.first_row + e.count):
                    state.mul_(self.decay).add_(x[row].float())
                    out[row] = state @ self.weight.t()
            return out.to(self.act)

    @NORMS.register("toy_centered", replace=True)
    class CenteredNorm(Part):
        """y = (x - mean) / sqrt(var + eps) * w over the row, x = h + delta."""

        records_cleanly = True

        @classmethod
        def weight_specs(cls, params):
            return {"weight": TensorSpec((params["size"],), kind="norm")}

        def __init__(self, params, prefix, build):
            self.eps = params["eps"]
            self.weight = build.loader.get(f"{prefix}.weight").float()

        def apply(self, h, delta, out, rows=None):
            if delta is not None and rows is None:
                h.add_(delta.float())
            x = h if delta is None or rows is None else h + delta.float()
            if rows is not None:
                x = x.index_select(0, rows.long())
            x = x - x.mean(dim=-1, keepdim=True)
            out.copy_(x * torch.rsqrt((x * x).mean(dim=-1, keepdim=True) + self.eps) * self.weight)
            return out

    @dataclass
    class ToyConfig(ModelConfig):
        vocab_size: int
        width: int
        depth: int
        heads: int
        kv_heads: int
        head_width: int
        inner: int
        most_positions: int
        eps: float
        theta: float
        decay: float
        odd_norm: str = "toy_centered"      # an option of the engine: which norm stands before an odd layer's feed-forward
        architecture: str = "ToyForCausalLM"

        engine_options = {"odd_norm": {"choices": ["toy_centered", "rmsnorm"], "help": "norm before an odd layer's feed-forward"}}

        @classmethod
        def from_dict(cls, data, origin="<dict>", generation=None, generation_origin="<dict>"):
            r = JsonReader(data, origin)
            cfg = cls(vocab_size=r.integer("vocab"), width=r.integer("width"), depth=r.integer("depth"),
                      heads=r.integer("heads"), kv_heads=r.integer("kv_heads"), head_width=r.integer("head_width"),
                      inner=r.integer("inner"), most_positions=r.integer("most_positions"), eps=r.number("eps"),
                      theta=r.number("theta"), decay=r.number("decay"))
            cfg.read_generation_defaults(generation, generation_origin)
            cfg.validate(origin)
            return cfg

        def validate(self, origin="<config>"):
            if not 0.0 < self.decay < 1.0:
                raise ConfigError(f"'{origin}': decay must lie between 0 and 1, got {self.decay}")
            if self.odd_norm not in ("toy_centered", "rmsnorm"):
                raise ConfigError(f"'{origin}': odd_norm '{self.odd_norm}' is unknown")

        def to_dict(self):
            return dict(architectures=[self.architecture], vocab=self.vocab_size, width=self.width, depth=self.depth,
                        heads=self.heads, kv_heads=self.kv_heads, head_width=self.head_width, inner=self.inner,
                        most_positions=self.most_positions, eps=self.eps, theta=self.theta, decay=self.decay)

        def model_spec(self):
            rms = PartSpec("rmsnorm", {"size": self.width, "eps": self.eps})
            odd = PartSpec(self.odd_norm, {"size": self.width, "eps": self.eps})
            ffn = PartSpec("gated_mlp", {"hidden_size": self.width, "intermediate_size": self.inner, "prefix": "mlp"})
            layers = []
            for i in range(self.depth):
                if i % 2 == 1:
                    mixer = PartSpec("toy_running_sum", {"hidden_size": self.width, "decay": self.decay, "prefix": "toy"})
                    norms = {"mixer_norm": rms, "ffn_norm": odd}
                else:
                    mixer = PartSpec("attention", {
                        "hidden_size": self.width, "num_heads": self.heads, "num_kv_heads": self.kv_heads,
                        "head_dim": self.head_width, "qk_norm": True, "qk_norm_eps": self.eps,
                        "scale": self.head_width ** -0.5, "window": None, "position": "rope", "prefix": "self_attn"})
                    norms = {"mixer_norm": rms, "ffn_norm": rms}
                layers.append(LayerSpec(f"model.layers.{i}", mixer, ffn, norms))
            return ModelSpec(
                architecture=self.architecture, vocab_size=self.vocab_size, hidden_size=self.width,
                max_positions=self.most_positions,
                embedding=PartSpec("embedding", {"vocab_size": self.vocab_size, "hidden_size": self.width,
                                                 "name": "model.embed_tokens.weight"}),
                layers=layers, order=[RunSpec(i) for i in range(self.depth)], final_norm=rms,
                head=PartSpec("lm_head", {"vocab_size": self.vocab_size, "hidden_size": self.width, "name": "lm_head.weight",
                                          "tied": False, "tied_to": "model.embed_tokens.weight"}),
                positions={"rope": PartSpec("rope", {"theta": self.theta, "rotary_dim": self.head_width,
                                                     "head_dim": self.head_width, "pairing": "interleaved"})})

    register_architecture("ToyForCausalLM", ToyConfig, replace=True)
    return ToyConfig


def unregister_toys():
    from pulse_infer_amd.config import unregister_architecture
    from pulse_infer_amd.parts.base import MIXERS, NORMS

    unregister_architecture("ToyForCausalLM")
    MIXERS.unregister("toy_running_sum")
    NORMS.unregister("toy_centered")


def toy_plain(folder):
    """The plain decoder over the toy's tensors (its attention layers are ordinary ones): the toy's keys under the
    names the plain implementation reads."""
    from safetensors.torch import load_file
    c = dict(num_attention_heads=TOY["heads"], num_key_value_heads=TOY["kv_heads"], head_dim=TOY["head_width"],
             hidden_size=TOY["width"], rms_norm_eps=TOY["eps"], rope_theta=TOY["theta"], num_hidden_layers=TOY["depth"],
             vocab_size=TOY["vocab"])
    return P.PlainQwen3(c, load_file(f"{folder}/model.safetensors"))


def plain_toy_logits(plain, ids, odd_norm="toy_centered"):
    """The toy model with plain functions: odd layers use the running sum in place of attention, and centre the row
    in the norm before their feed-forward."""
    c, w = plain.c, plain.w
    h = P.embedding(w["model.embed_tokens.weight"], ids)
    pos = list(range(len(ids)))
    for i in range(c["num_hidden_layers"]):
        if i % 2 == 0:
            h = plain.layer(h, i, pos)
            continue
        p = f"model.layers.{i}."
        a = P.rms_norm(h, w[p + "input_layernorm.weight"], c["rms_norm_eps"])
        state, rows = torch.zeros(h.shape[1], dtype=F64), []
        for t in range(len(ids)):
            state = TOY["decay"] * state + a[t]
            rows.append(state @ w[p + "toy.mix.weight"].T)
        h = h + torch.stack(rows)
        if odd_norm == "toy_centered":
            x = h - h.mean(dim=-1, keepdim=True)
            m = x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + c["rms_norm_eps"]) * w[p + "post_attention_layernorm.weight"]
        else:
            m = P.rms_norm(h, w[p + "post_attention_layernorm.weight"], c["rms_norm_eps"])
        h = h + P.gated_mlp(m, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"], w[p + "mlp.down_proj.weight"])
    return P.linear(P.rms_norm(h, w["model.norm.weight"], c["rms_norm_eps"]), w["lm_head.weight"])


def plain_toy_greedy(plain, prompt, steps, odd_norm="toy_centered"):
    ids, out = list(prompt), []
    for _ in range(steps):
        out.append(int(torch.argmax(plain_toy_logits(plain, ids, odd_norm)[-1])))
        ids.append(out[-1])
    return out


def test_a_toy_mixer_with_state_is_registered_built_and_stepped(gpu, tmp_path):
    from pulse_infer_amd.config import load_config
    from pulse_infer_amd.engine.runner import ModelRunner, StepEntry
    from pulse_infer_amd.models.factory import load_model
    from pulse_infer_amd.weights import write_model_folder
    from test_gpu_model import close

    toy_config = register_toys()
    try:
        folder = write_model_folder(toy_config.from_dict(TOY), str(tmp_path / "toy"), seed=21)
        plain = toy_plain(folder)
        config, model = load_model(folder, mode="float32")
        assert type(config) is toy_config and type(load_config(folder)) is toy_config
        assert type(model.blocks[1].mixer).__name__ == "RunningSum"
        assert type(model.blocks[1].ffn_norm).__name__ == "CenteredNorm" and type(model.blocks[1].mixer_norm).__name__ == "RMSNorm"
        runner = ModelRunner(model, page_size=16, num_pages=16, max_requests=2)
        assert len(runner.cache.groups) == 1 and sorted(runner.cache.state_runs) == [1, 3]
        ids = {k: token_ids(config.vocab_size, n, seed=60 + n) for k, n in (("a", 40), ("b", 23), ("c", 31))}
        got = {k: [] for k in ids}
        # a and b interleaved (portions beside single tokens); c afterwards in b's slot, whose state must not leak
        plan = [[("a", 7), ("b", 2)], [("a", 1), ("b", 9)], [("b", 1)], [("a", 20), ("b", 11)], [("a", 12)],
                [("c", 5)], [("c", 26)]]
        fed = {k: 0 for k in ids}
        for step in plan:
            entries = []
            for k, n in step:
                if not runner.cache.has_request(k):
                    runner.add_request(k)
                runner.reserve(k, fed[k] + n)
                entries.append(StepEntry(k, ids[k][fed[k]:fed[k] + n], list(range(n))))
                fed[k] += n
            logits = runner.step(entries)
            row = 0
            for k, n in step:
                got[k].append(logits[row:row + n])
                row += n
            for k, _ in step:
                if fed[k] == len(ids[k]) and runner.cache.has_request(k):
                    runner.free_request(k)
        for k in ids:
            close(torch.cat(got[k]), plain_toy_logits(plain, ids[k]), "float32", f"toy request {k}")
    finally:
        unregister_toys()


def test_a_toy_architecture_runs_through_the_entry_points(gpu, tmp_path, capsys):
    """The toy's own configuration class (no Qwen3 field in it) through ``LLM.from_pretrained`` / ``generate`` and
    through the command line, including the option its class declares and ``--set``; greedy tokens against the
    plain formulas."""
    import json
    from pulse_infer_amd import LLM, cli
    from pulse_infer_amd.config import ConfigError
    from pulse_infer_amd.weights import write_model_folder

    toy_config = register_toys()
    try:
        folder = write_model_folder(toy_config.from_dict(TOY), str(tmp_path / "toy"), seed=23)
        plain = toy_plain(folder)
        prompts = [token_ids(TOY["vocab"], n, seed=30 + n) for n in (9, 21)]
        llm = LLM.from_pretrained(folder, dtype="float32", max_batch_size=2, chunk_size=8, page_size=16, num_pages=16)
        assert llm.generate(prompts, max_new_tokens=5, ignore_eos=True) == [plain_toy_greedy(plain, p, 5) for p in prompts]
        common = [folder, "--dtype", "f32", "--prompt-ids", ",".join(map(str, prompts[0])), "--max-new-tokens", "4",
                  "--num-pages", "16", "--ignore-eos"]
        assert cli.main(common) == 0
        assert json.loads(capsys.readouterr().out.splitlines()[0])["output_ids"] == plain_toy_greedy(plain, prompts[0], 4)
        for how in (["--odd-norm", "rmsnorm"], ["--set", "odd_norm=rmsnorm"]):
            assert cli.main(common + how) == 0
            assert json.loads(capsys.readouterr().out.splitlines()[0])["output_ids"] == \
                plain_toy_greedy(plain, prompts[0], 4, "rmsnorm")
        with pytest.raises(ConfigError, match="no field 'rope_pairing'"):
            cli.main(common + ["--set", "rope_pairing=half"])
        with pytest.raises(SystemExit):
            cli.main(common + ["--rope-pairing", "half"])            # an option of another architecture
    finally:
        unregister_toys()


def test_a_toy_mixer_that_records_cleanly_is_replayed(gpu, tmp_path):
    """bfloat16: the toy says that its parts record cleanly, so steps of single tokens run as replays of a recording
    although the model has per-request state: every replay against the eager step, with eager prompt portions of
    another request in between, a request that restarts in a used slot, and the plain formulas."""
    from pulse_infer_amd.engine.runner import ModelRunner, StepEntry
    from pulse_infer_amd.models.factory import load_model
    from pulse_infer_amd.weights import write_model_folder
    from test_gpu_model import SPLIT_TOL, close

    toy_config = register_toys()
    try:
        folder = write_model_folder(toy_config.from_dict(TOY), str(tmp_path / "toy"), seed=25)
        plain = toy_plain(folder)
        _, model = load_model(folder, mode="bfloat16")
        ids = {k: token_ids(TOY["vocab"], n, seed=40 + n) for k, n in (("a", 46), ("b", 37), ("c", 25))}
        outs = []
        for graphs in (True, False):
            runner = ModelRunner(model, page_size=16, num_pages=16, max_requests=2, use_graphs=graphs)
            runner.GRAPH_AFTER_STEPS = 1
            assert runner.use_graphs == graphs
            fed, got = {k: 0 for k in ids}, {k: [] for k in ids}

            def feed(pairs):
                entries = []
                for k, n in pairs:
                    if not runner.cache.has_request(k):
                        runner.add_request(k)
                    runner.reserve(k, fed[k] + n)
                    entries.append(StepEntry(k, ids[k][fed[k]:fed[k] + n], list(range(n))))
                    fed[k] += n
                logits = runner.step(entries)
                row = 0
                for k, n in pairs:
                    got[k].append(logits[row:row + n])
                    row += n

            feed([("a", 18), ("b", 5)])
            for _ in range(8):
                feed([("a", 1), ("b", 1)])
            feed([("b", 9)])                               # eager work between the replays
            for _ in range(15):
                feed([("b", 1), ("a", 1)])
            feed([("a", 1)])                               # a step of one request: its shape is recorded here ..
            runner.free_request("b")
            feed([("c", 1)])                               # .. and replayed here, where c starts in the slot b left
            for _ in range(3):
                feed([("a", 1), ("c", 1)])
            feed([("c", 20)])
            assert runner.graph_replays == (7 + 15 + 1 + 3 if graphs else 0) and runner.graph_records == (2 if graphs else 0)
            outs.append({k: torch.cat(v) for k, v in got.items()})
            del runner
        for k in ids:
            want = plain_toy_logits(plain, ids[k])[:outs[0][k].shape[0]]
            close(outs[0][k], want, "bfloat16", f"recorded toy, request {k}")
            close(outs[0][k], outs[1][k], "bfloat16", f"recorded toy against eager, request {k}", SPLIT_TOL)
    finally:
        unregister_toys()


def test_order_may_name_a_layer_twice_and_share_a_cache(gpu, tmp_path):
    """Run order [0, 1, 0(shares nothing), 2 reading run 1's cache]: weights of layer 0 are used twice with a
    cache each; the last run computes only queries and attends to what run 1 wrote."""
    from conftest import TINY_A
    from pulse_infer_amd.config import Qwen3Config
    from pulse_infer_amd.engine.runner import ModelRunner, StepEntry
    from pulse_infer_amd.models.causal_lm import CausalLM
    from pulse_infer_amd.models.spec import RunSpec
    from pulse_infer_amd.weights import SafetensorsSource, write_model_folder
    from test_gpu_model import close

    cfg = Qwen3Config.from_dict(dict(TINY_A, num_hidden_layers=3))
    folder = write_model_folder(cfg, str(tmp_path / "m"), seed=31)
    spec = cfg.model_spec()
    spec.order = [RunSpec(0), RunSpec(1), RunSpec(0), RunSpec(2, cache_of=1)]
    model = CausalLM(spec, SafetensorsSource(folder), mode="float32")
    runner = ModelRunner(model, page_size=4, num_pages=32, max_requests=2)
    assert len(runner.cache.groups[0].runs) == 3          # three runs own pages, the fourth borrows
    ids = token_ids(cfg.vocab_size, 30, seed=9)
    runner.add_request("r")
    outs, fed = [], 0
    for n in (11, 1, 1, 17):
        runner.reserve("r", fed + n)
        outs.append(runner.step([StepEntry("r", ids[fed:fed + n], list(range(n)))]))
        fed += n

    plain = P.PlainQwen3.from_folder(folder)
    c, w = plain.c, plain.w
    pos = list(range(30))
    h = P.embedding(w["model.embed_tokens.weight"], ids)
    h = plain.layer(h, 0, pos)
    # layer 1, keeping its rotated keys and its values for the sharing run
    nq, nkv, d, eps = c["num_attention_heads"], c["num_key_value_heads"], c["head_dim"], c["rms_norm_eps"]
    a = P.rms_norm(h, w["model.layers.1.input_layernorm.weight"], eps)
    k1 = P.rope(P.rms_norm(P.linear(a, w["model.layers.1.self_attn.k_proj.weight"]).view(30, nkv, d),
                           w["model.layers.1.self_attn.k_norm.weight"], eps), pos, c["rope_theta"])
    v1 = P.linear(a, w["model.layers.1.self_attn.v_proj.weight"]).view(30, nkv, d)
    h = plain.layer(h, 1, pos)
    h = plain.layer(h, 0, pos)
    p = "model.layers.2."
    a = P.rms_norm(h, w[p + "input_layernorm.weight"], eps)
    q = P.rope(P.rms_norm(P.linear(a, w[p + "self_attn.q_proj.weight"]).view(30, nq, d), w[p + "self_attn.q_norm.weight"], eps),
               pos, c["rope_theta"])
    o = P.causal_attention(q, k1, v1, d ** -0.5)
    h = h + P.linear(o.reshape(30, nq * d), w[p + "self_attn.o_proj.weight"])
    m = P.rms_norm(h, w[p + "post_attention_layernorm.weight"], eps)
    h = h + P.gated_mlp(m, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"], w[p + "mlp.down_proj.weight"])
    want = P.linear(P.rms_norm(h, w["model.norm.weight"], eps), w["model.embed_tokens.weight"])
    close(torch.cat(outs), want, "float32", "shared order")


# ------------------------------------------- a routed feed-forward and another position encoding, as toys
ROUTED = {"experts": 5, "top_k": 2, "expert_size": 24}
BANDS = {"factor": 4.0, "theta": 500.0}


def register_routed_toys():
    """A feed-forward that routes each token to its best experts, and a rotary encoding whose slow half of the
    frequencies sees positions divided by a factor (pairs (i, i + d/2)); an architecture uses the first in its odd
    layers and the second in its even layers, beside the ordinary parts."""
    from pulse_infer_amd.config import Qwen3Config, register_architecture
    from pulse_infer_amd.models.spec import LayerSpec, PartSpec
    from pulse_infer_amd.parts.base import FEED_FORWARDS, POSITIONS, Part
    from pulse_infer_amd.parts.rope import PAIRINGS, RotationTables
    from pulse_infer_amd.weights import TensorSpec

    @FEED_FORWARDS.register("toy_routed", replace=True)
    class RoutedExperts(Part):
        """y = sum over the top_k experts e of softmax(router logits of those)_e * W2_e relu(W1_e x); router in float32."""

        @classmethod
        def weight_specs(cls, params):
            hidden, size = params["hidden_size"], params["expert_size"]
            specs = {"router.weight": TensorSpec((params["experts"], hidden), fan_in=hidden)}
            for e in range(params["experts"]):
                specs[f"experts.{e}.w1.weight"] = TensorSpec((size, hidden), fan_in=hidden)
                specs[f"experts.{e}.w2.weight"] = TensorSpec((hidden, size), fan_in=size)
            return specs

        def __init__(self, params, prefix, build):
            self.top_k = params["top_k"]
            get = lambda name: build.loader.get(f"{prefix}.{name}").float()
            self.router = get("router.weight")
            self.w1 = torch.stack([get(f"experts.{e}.w1.weight") for e in range(params["experts"])])
            self.w2 = torch.stack([get(f"experts.{e}.w2.weight") for e in range(params["experts"])])
            self.act = build.act_dtype

        def forward(self, x, ctx):
            x = x.float()
            top, chosen = (x @ self.router.t()).topk(self.top_k, dim=-1)
            share = torch.softmax(top, dim=-1)
            out = torch.zeros_like(x)
            for e in range(self.w1.shape[0]):                       # tokens grouped by expert
                rows, slot = (chosen == e).nonzero(as_tuple=True)
                if rows.numel():
                    y = torch.relu(x[rows] @ self.w1[e].t()) @ self.w2[e].t()
                    out.index_add_(0, rows, y * share[rows, slot].unsqueeze(1))
            return out.to(self.act)

    @POSITIONS.register("toy_banded_rope", replace=True)
    class BandedRotary(Part):
        def __init__(self, params, build):
            self.dim, self.factor = params["rotary_dim"], params["factor"]
            half = self.dim // 2
            inv = torch.tensor(params["theta"], dtype=F64) ** (-torch.arange(half, dtype=F64) * 2.0 / self.dim)
            inv[half // 2:] /= self.factor
            self.inv_freq = inv.to(build.device)

        def prepare(self, ctx):
            angle = ctx.positions.to(F64).unsqueeze(1) * self.inv_freq
            return RotationTables(torch.cos(angle).float().contiguous(), torch.sin(angle).float().contiguous(),
                                  self.dim, PAIRINGS["half"])

    class RoutedConfig(Qwen3Config):
        def model_spec(self):
            base = super().model_spec()
            base.positions["bands"] = PartSpec("toy_banded_rope", dict(BANDS, rotary_dim=self.head_dim))
            layers = []
            for i, layer in enumerate(base.layers):
                mixer, ffn = layer.mixer, layer.ffn
                if i % 2 == 0:
                    mixer = PartSpec("attention", dict(mixer.params, position="bands"))
                else:
                    ffn = PartSpec("toy_routed", dict(ROUTED, hidden_size=self.hidden_size, prefix="moe"))
                layers.append(layer.with_parts(mixer=mixer, ffn=ffn))
            base.layers = layers
            base.architecture = "RoutedToyForCausalLM"
            return base

    register_architecture("RoutedToyForCausalLM", RoutedConfig, replace=True)
    return RoutedConfig


def plain_routed_logits(plain, ids):
    c, w = plain.c, plain.w
    nq, nkv, d, eps = c["num_attention_heads"], c["num_key_value_heads"], c["head_dim"], c["rms_norm_eps"]
    t = len(ids)
    pos = list(range(t))
    h = P.embedding(w["model.embed_tokens.weight"], ids)
    margins = []

    def banded(x):  # complex multiplication of (x[i], x[i + d/2]) by e^(i angle)
        half = d // 2
        inv = torch.tensor(BANDS["theta"], dtype=F64) ** (-torch.arange(half, dtype=F64) * 2.0 / d)
        inv[half // 2:] /= BANDS["factor"]
        turn = torch.polar(torch.ones(t, half, dtype=F64), torch.tensor(pos, dtype=F64).unsqueeze(1) * inv).unsqueeze(1)
        z = torch.complex(x[..., :half], x[..., half:]) * turn
        return torch.cat([z.real, z.imag], dim=-1)

    for i in range(c["num_hidden_layers"]):
        p = f"model.layers.{i}."
        a = P.rms_norm(h, w[p + "input_layernorm.weight"], eps)
        q = P.rms_norm(P.linear(a, w[p + "self_attn.q_proj.weight"]).view(t, nq, d), w[p + "self_attn.q_norm.weight"], eps)
        k = P.rms_norm(P.linear(a, w[p + "self_attn.k_proj.weight"]).view(t, nkv, d), w[p + "self_attn.k_norm.weight"], eps)
        v = P.linear(a, w[p + "self_attn.v_proj.weight"]).view(t, nkv, d)
        q, k = (banded(q), banded(k)) if i % 2 == 0 else (P.rope(q, pos, c["rope_theta"]), P.rope(k, pos, c["rope_theta"]))
        o = P.causal_attention(q, k, v, d ** -0.5)
        h = h + P.linear(o.reshape(t, nq * d), w[p + "self_attn.o_proj.weight"])
        m = P.rms_norm(h, w[p + "post_attention_layernorm.weight"], eps)
        if i % 2 == 0:
            h = h + P.gated_mlp(m, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"], w[p + "mlp.down_proj.weight"])
            continue
        rows = []
        for row in m:                                                # token by token, expert by expert
            scores = w[p + "moe.router.weight"] @ row
            order = sorted(range(ROUTED["experts"]), key=lambda e: -scores[e].item())
            margins.append((scores[order[ROUTED["top_k"] - 1]] - scores[order[ROUTED["top_k"]]]).item())
            best = order[:ROUTED["top_k"]]
            share = torch.softmax(torch.stack([scores[e] for e in best]), dim=0)
            rows.append(sum(share[j] * (w[p + f"moe.experts.{e}.w2.weight"] @ torch.relu(w[p + f"moe.experts.{e}.w1.weight"] @ row))
                            for j, e in enumerate(best)))
        h = h + torch.stack(rows)
    return P.linear(P.rms_norm(h, w["model.norm.weight"], eps), w["lm_head.weight"]), min(margins)


def test_a_toy_routed_feed_forward_and_another_position_encoding(gpu, tmp_path):
    from conftest import TINY_B
    from pulse_infer_amd.config import unregister_architecture
    from pulse_infer_amd.engine.runner import ModelRunner, StepEntry
    from pulse_infer_amd.models.factory import load_model
    from pulse_infer_amd.parts.base import FEED_FORWARDS, POSITIONS
    from pulse_infer_amd.weights import write_model_folder
    from test_gpu_model import close

    config = register_routed_toys()
    try:
        cfg = config.from_dict(dict(TINY_B, architectures=["RoutedToyForCausalLM"], num_hidden_layers=4))
        cfg.architecture = "RoutedToyForCausalLM"
        folder = write_model_folder(cfg, str(tmp_path / "routed"), seed=33)
        plain = P.PlainQwen3.from_folder(folder)
        assert f"model.layers.1.moe.experts.{ROUTED['experts'] - 1}.w2.weight" in plain.w
        assert "model.layers.1.mlp.gate_proj.weight" not in plain.w
        _, model = load_model(folder, mode="float32")
        assert type(model.blocks[1].ffn).__name__ == "RoutedExperts" and model.blocks[0].mixer.position == "bands"
        runner = ModelRunner(model, page_size=16, num_pages=12, max_requests=2)
        ids = {k: token_ids(cfg.vocab_size, n, seed=80 + n) for k, n in (("a", 45), ("b", 27))}
        got, fed = {k: [] for k in ids}, {k: 0 for k in ids}
        for step in ([("a", 9), ("b", 2)], [("a", 1), ("b", 14)], [("a", 33), ("b", 1)], [("a", 2), ("b", 10)]):
            entries = []
            for k, n in step:
                if not runner.cache.has_request(k):
                    runner.add_request(k)
                runner.reserve(k, fed[k] + n)
                entries.append(StepEntry(k, ids[k][fed[k]:fed[k] + n], list(range(n))))
                fed[k] += n
            logits = runner.step(entries)
            row = 0
            for k, n in step:
                got[k].append(logits[row:row + n])
                row += n
        for k in ids:
            want, margin = plain_routed_logits(plain, ids[k])
            assert margin > 1e-4, "two experts score alike for a token: choose another seed, the choice is not pinned"
            close(torch.cat(got[k]), want, "float32", f"routed toy request {k}")
    finally:
        unregister_architecture("RoutedToyForCausalLM")
        FEED_FORWARDS.unregister("toy_routed")
        POSITIONS.unregister("toy_banded_rope")
