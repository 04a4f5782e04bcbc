"""Causal attention over a paged cache, with grouped key/value heads, optional
per-head RMSNorm of q and k, an optional window and a pluggable position encoding.

Order of operations per token (reference: src/model/qwen3/model.cpp:784-876):
q, k, v = x Wq^T, x Wk^T, x Wv^T; q, k <- RMSNorm over head_dim (one weight for
all heads); q, k <- rotation at the token's position; k, v written to the
cache; o = softmax(q K^T * scale) V over keys lo..position of the same request;
output = o Wo^T.  Query head h reads kv head h // (num_heads // num_kv_heads).
A window w gives lo = max(0, position - w + 1); without one lo = 0.

The three projections are one product with the row-stacked weight (a layout
choice); norm, rotation and the cache write are one kernel; the attention
kernel is chosen by size and storage type.
"""
from __future__ import annotations

from typing import Any, Dict, Optional

import torch

from ..cache.manager import PagedKVSpec
from ..ops import attention_mfma, kernels
from ..weights.store import TensorSpec
from .base import MIXERS, BuildContext, LazyNorm, PagedCacheView, Part, StepContext, StepCost
from .linear import Linear


@MIXERS.register("attention")
class PagedAttention(Part):
    @classmethod
    def weight_specs(cls, params: Dict[str, Any]) -> Dict[str, TensorSpec]:
        hidden, nq, nkv, d = (params[k] for k in ("hidden_size", "num_heads", "num_kv_heads", "head_dim"))
        specs = {
            "q_proj.weight": TensorSpec((nq * d, hidden), fan_in=hidden),
            "k_proj.weight": TensorSpec((nkv * d, hidden), fan_in=hidden),
            "v_proj.weight": TensorSpec((nkv * d, hidden), fan_in=hidden),
            "o_proj.weight": TensorSpec((hidden, nq * d), fan_in=nq * d),
        }
        if params.get("qk_norm", False):
            specs["q_norm.weight"] = TensorSpec((d,), kind="norm")
            specs["k_norm.weight"] = TensorSpec((d,), kind="norm")
        return specs

    @classmethod
    def step_cost(cls, params: Dict[str, Any], entries, weight_bytes: int, cache_bytes: int) -> StepCost:
        """The projections, plus scores and weighted values over the keys each token sees (2 x 2 x heads x head size
        a key), plus the keys and values of every request's visible context read once."""
        cost = super().step_cost(params, entries, weight_bytes, cache_bytes)
        nq, nkv, d, window = params["num_heads"], params["num_kv_heads"], params["head_dim"], params.get("window")
        for start, count in entries:
            seen = 0
            for p in range(start, start + count):
                seen += min(p + 1, window) if window else p + 1
            cost.flops += 4.0 * nq * d * seen
            context = start + count
            cost.cache_bytes += 2.0 * nkv * d * cache_bytes * (min(context, window + count - 1) if window else context)
        return cost

    def __init__(self, params: Dict[str, Any], prefix: str, build: BuildContext):
        self.hidden = int(params["hidden_size"])
        self.nq = int(params["num_heads"])
        self.nkv = int(params["num_kv_heads"])
        self.d = int(params["head_dim"])
        if self.nq % self.nkv:
            raise ValueError(f"{self.nq} query heads are not a multiple of {self.nkv} key/value heads")
        self.scale = float(params["scale"])
        self.window = params.get("window")
        if self.window is not None and int(self.window) <= 0:
            raise ValueError(f"an attention window must be positive, got {self.window}")
        self.qk_norm = bool(params.get("qk_norm", False))
        self.eps = float(params.get("qk_norm_eps", 0.0))
        self.position = params.get("position")
        self.encodings = build.positions
        if self.position is not None and self.position not in self.encodings:
            raise KeyError(f"attention refers to position encoding '{self.position}', the model defines "
                           f"{sorted(self.encodings)}")
        load = build.loader
        self.qkv = Linear(load.get_concat([f"{prefix}.q_proj.weight", f"{prefix}.k_proj.weight",
                                           f"{prefix}.v_proj.weight"]), build.mode)
        self.o = Linear(load.get(f"{prefix}.o_proj.weight"), build.mode)
        self.q_w = load.get(f"{prefix}.q_norm.weight") if self.qk_norm else None
        self.k_w = load.get(f"{prefix}.k_norm.weight") if self.qk_norm else None
        self.act_dtype = build.act_dtype
        self.options = build.options

    def cache_spec(self) -> PagedKVSpec:
        return PagedKVSpec(self.nkv, self.d, int(self.window) if self.window is not None else None)

    accepts_residual = True
    accepts_lazy_input = True   # the first product may take rows that are not normalised yet and scale its result
    records_cleanly = True      # positions, tables and work lists are read on the device

    def forward(self, x, ctx: StepContext, cache: PagedCacheView, residual: Optional[torch.Tensor] = None,
                next_scale: Optional[torch.Tensor] = None):
        tokens = x.shape[0]
        ws = ctx.workspace
        write = cache.writable
        q_cols = self.nq * self.d
        cols = (self.nq + 2 * self.nkv) * self.d if write else q_cols
        qkv = ws.buffer("attention.qkv", tokens, cols, self.act_dtype)
        if isinstance(x, LazyNorm) and not self.qkv.takes_lazy(x, rows=None if write else q_cols):
            x = x.materialize(ws.buffer("attention.normed", tokens, self.hidden, self.act_dtype))
        self.qkv.forward(x, qkv, rows=None if write else q_cols)
        tables = ctx.position_product(self.position, self.encodings) if self.position is not None else None
        table = ctx.block_tables[cache.group]
        attn = ws.buffer("attention.out", tokens, q_cols, self.act_dtype)
        if self.decodes_from_raw(ctx, cache, qkv, tables):
            # decoded tokens only: the attention kernel prepares q and each token's own key itself
            self.attend(qkv, attn, ctx, cache, table, raw=(tables, write))
        else:
            kernels.qk_rope_kv(
                qkv, self.nq, self.nkv, self.d, self.q_w, self.k_w, self.eps,
                tables.cos if tables is not None else None, tables.sin if tables is not None else None,
                tables.rotary_dim if tables is not None else 0, tables.pairing if tables is not None else 0,
                cache.keys, cache.values, ctx.positions, ctx.token_entry, table, write_kv=write)
            self.attend(qkv, attn, ctx, cache, table)
        out = ws.buffer("attention.proj", tokens, self.hidden, self.act_dtype)
        if residual is not None:
            return self.o.add_into(attn, residual, out, ws, next_scale)
        return self.o.forward(attn, out)

    def uses_matrix_cores(self, q: torch.Tensor, cache: PagedCacheView) -> bool:
        return (self.options.get("attention", "auto") != "generic"
                and attention_mfma.supported(self.d, cache.page_size, q.dtype, cache.keys.dtype))

    def decodes_from_raw(self, ctx: StepContext, cache: PagedCacheView, qkv: torch.Tensor, tables: Any) -> bool:
        """Whether this step's attention can start from the raw projection output: every entry is one decoded
        token, the matrix-core kernel takes the sizes, and norm weights and rotation are of the kinds it prepares."""
        if self.options.get("decode_from_raw", True) is False or not self.uses_matrix_cores(qkv, cache):
            return False
        if "static:attention.single_tokens" not in ctx.extras:
            ctx.extras["static:attention.single_tokens"] = all(e.count == 1 for e in ctx.entries)
        if not ctx.extras["static:attention.single_tokens"]:
            return False
        if any(w is not None and w.dtype != torch.bfloat16 for w in (self.q_w, self.k_w)):
            return False
        if tables is None:
            return True
        return (tables.cos.dtype == torch.float32 and tables.cos.is_contiguous() and tables.sin.is_contiguous()
                and attention_mfma.decode_takes(self.d, tables.rotary_dim, tables.pairing))

    def attend(self, q: torch.Tensor, out: torch.Tensor, ctx: StepContext, cache: PagedCacheView,
               table: torch.Tensor, raw: Optional[tuple] = None) -> None:
        """out = attention of the step's tokens over the cache.  ``raw = (rotation tables, write)``: q is the raw
        projection output of decoded tokens, which the kernel prepares itself (see ``decodes_from_raw``)."""
        window = int(self.window) if self.window is not None else 0
        if not self.uses_matrix_cores(q, cache):
            kernels.attn_generic(q, out, self.nq, self.nkv, self.d, cache.keys, cache.values, ctx.positions,
                                 ctx.token_entry, table, self.scale, window)
            return
        group = self.nq // self.nkv
        per = attention_mfma.tokens_per_item(group)
        portion = attention_mfma.portion_tokens(group, self.d)
        key = f"static:attention.items:{per}:{portion}"
        if key not in ctx.extras:  # depends only on the step's shape; the same lists serve every layer
            short, long = attention_mfma.split_entries(ctx.entries)
            dev = lambda flat: ctx.to_device(flat) if flat else None
            ctx.extras[key] = (
                dev(attention_mfma.build_items(short, per)),
                dev(attention_mfma.build_items(long, portion)),
                max((e.start + e.count for _, e in short), default=0))
        short_items, long_items, short_context = ctx.extras[key]
        if long_items is not None:
            skey = f"static:attention.portion_splits:{portion}:{window}:{self.nkv}:{group}:{self.d}"
            if skey not in ctx.extras:
                ctx.extras[skey] = attention_mfma.choose_prefill_splits(
                    attention_mfma.split_entries(ctx.entries)[1], portion, self.nkv, group, self.d, window)
            split_size, n_splits = ctx.extras[skey]
            part_o = part_ml = None
            if n_splits > 1:
                rows = ctx.num_tokens * self.nq * n_splits
                part_o = ctx.workspace.buffer("attention.portion_part_o", rows, self.d, torch.float32)
                part_ml = ctx.workspace.buffer("attention.portion_part_ml", rows, 2, torch.float32)
            attention_mfma.attn_prefill(q, out, self.nq, self.nkv, self.d, cache.keys, cache.values, ctx.positions,
                                        table, long_items, self.scale, window, split_size, n_splits, part_o, part_ml)
        if short_items is not None:
            # a recorded step passes its context bucket as max_context: its splits must cover that
            max_context = ctx.max_context if long_items is None else short_context
            n_items = short_items.numel() // attention_mfma.ITEM_INTS
            split_size, n_splits = attention_mfma.choose_splits(n_items, self.nkv, group, max_context)
            plan = None
            if ctx.uneven and long_items is None and not window:
                # contexts that differ much: every request's keys cut by its own length, the workgroups in an order
                # that starts the longest walks first (the plan is made on the device, once a step for all layers)
                planned = min(attention_mfma.PLAN_SPLITS, 1024 // n_items)
                if planned > 1 and attention_mfma.plan_fits(n_items, planned):
                    n_splits = planned
                    split_size = max(32, ((max_context + n_splits - 1) // n_splits + 31) // 32 * 32)
                    slots, first = attention_mfma.plan_slots(self.nkv, group)
                    pkey = f"attention.plan:{per}:{n_splits}:{slots}:{first}"
                    if pkey not in ctx.extras:
                        made = ctx.workspace.buffer(f"attention.plan:{n_splits}:{slots}:{first}",
                                                    attention_mfma.plan_ints(n_items, n_splits), 1, torch.int32)
                        attention_mfma.attn_plan(short_items if raw is None else None, ctx.positions, n_splits, slots,
                                                 first, made, self.d)
                        ctx.extras[pkey] = made
                    plan = ctx.extras[pkey]
            part_o = part_ml = None
            if n_splits > 1:
                rows = ctx.num_tokens * self.nq * n_splits
                part_o = ctx.workspace.buffer("attention.part_o", rows, self.d, torch.float32)
                part_ml = ctx.workspace.buffer("attention.part_ml", rows, 2, torch.float32)
            if raw is not None:
                tables, write = raw
                # (no list of items: the step's tokens are its requests' in order, each with its row of the table)
                attention_mfma.attn_decode(
                    q, out, self.nq, self.nkv, self.d, cache.keys, cache.values, ctx.positions, table, None,
                    self.scale, window, split_size, n_splits, max_context, part_o, part_ml, self.q_w, self.k_w,
                    self.eps, tables.cos if tables is not None else None, tables.sin if tables is not None else None,
                    tables.rotary_dim if tables is not None else 0, tables.pairing if tables is not None else 0,
                    new_key=write, live_context=ctx.live_context if plan is None else None, plan=plan)
                return
            attention_mfma.attn_mfma(q, out, self.nq, self.nkv, self.d, cache.keys, cache.values, ctx.positions,
                                     table, short_items, self.scale, window, split_size, n_splits,
                                     max_context, part_o, part_ml,
                                     live_context=ctx.live_context if plan is None else None, plan=plan)
