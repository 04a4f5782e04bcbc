"""The step function.

``ModelRunner.step(entries)`` takes a batch of (request, its next tokens, the
places whose logits are wanted): portions of prompts beside single decoded
tokens, cut anywhere.  It runs only those tokens, as one batch, against the
cache that earlier steps left, and returns float32 logits for the wanted places
in the order of the entries and of ``want``.  Pages must have been reserved
before (``reserve``); the step itself allocates no page.

(reference: Qwen3Model::forward_batched, src/model/qwen3/model.cpp:1179-1374,
which takes flat tokens/positions/seq_ids, grows pages inside the forward and
returns logits for every token.)
"""
from __future__ import annotations

import gc
from dataclasses import dataclass, field
from typing import Any, Hashable, List, Optional, Sequence

import numpy as np
import torch

from .. import log
from ..cache.manager import CacheManager
from ..models.causal_lm import CausalLM
from ..parts.base import EntryMeta, StepContext, contexts_uneven


class StepError(ValueError):
    """The batch handed to ``step`` breaks one of its preconditions."""


@dataclass
class StepEntry:
    request: Hashable
    tokens: Sequence[int]
    want: Sequence[int] = field(default_factory=list)  # indices into ``tokens``


class _Staging:
    """Pinned host buffers for a step's integer metadata, used in turn."""

    def __init__(self, device: torch.device, depth: int = 4):
        self.device = device
        self.host: List[Optional[torch.Tensor]] = [None] * depth
        self.events: List[Optional[torch.cuda.Event]] = [None] * depth
        self.turn = 0

    def upload(self, data: np.ndarray) -> torch.Tensor:
        i = self.turn
        self.turn = (self.turn + 1) % len(self.host)
        if self.events[i] is not None:
            self.events[i].synchronize()
        n = int(data.size)
        if self.host[i] is None or self.host[i].numel() < n:
            self.host[i] = torch.empty(max(n, 4096), dtype=torch.int32, pin_memory=True)
        self.host[i][:n].numpy()[:] = data
        dev = torch.empty(n, dtype=torch.int32, device=self.device)
        dev.copy_(self.host[i][:n], non_blocking=True)
        if self.events[i] is None:
            self.events[i] = torch.cuda.Event()
        self.events[i].record()
        return dev

    def upload_values(self, values) -> torch.Tensor:
        """``upload`` of a list of integers (what a part's work list is)."""
        return self.upload(np.asarray(values, dtype=np.int32))


@dataclass
class _Captured:
    """A recorded decode step: its integer buffers, the graph, and where the logits appear."""

    host: torch.Tensor
    host_np: np.ndarray
    dev: torch.Tensor
    offsets: np.ndarray
    widths: List[int]
    graph: Any = None
    logits: Any = None
    workspace: Any = None
    context: Any = None   # kept alive: the graph reads tensors that the context's parts created (work lists, tables)
    event: Any = None
    row_stamps: Any = None   # per row of the block tables: the stamp of the request's tables when the row was written

    def wait(self) -> None:
        if self.event is not None:
            self.event.synchronize()   # the last copy out of the pinned buffer has finished

    def mark(self) -> None:
        if self.event is None:
            self.event = torch.cuda.Event()
        self.event.record()


class ModelRunner:
    def __init__(self, model: CausalLM, page_size: int, num_pages: int, max_requests: int = 64,
                 use_graphs: bool = True):
        self.model = model
        self.device = model.device
        self.cache = CacheManager(model.run_cache_specs(), page_size, num_pages, max_requests)
        self.cache.allocate_storage(self.device, model.act_dtype)
        # what every run of the order is handed as its cache: a view of its own storage, or of the run's it reads
        self.views: List[Any] = [
            self.cache.view(run.cache_of if run.cache_of is not None else index, writable=run.cache_of is None)
            for index, run in enumerate(model.spec.order)]
        self._staging = _Staging(self.device)
        self.use_graphs = bool(use_graphs) and model.options.get("decode_graph", True)
        self._graphs: dict = {}
        self._graph_seen: dict = {}
        self._graph_refused: set = set()   # shapes whose step holds a library call: no library call is ever recorded
        self.graph_records = 0      # recordings made so far
        self.graph_replays = 0      # steps that ran as a replay of a recording
        self.max_positions = model.spec.max_positions
        self.steps = 0
        self.tokens_run = 0

    # ----------------------------------------------------------------- requests
    def add_request(self, request: Hashable) -> int:
        return self.cache.add_request(request)

    def free_request(self, request: Hashable) -> None:
        self.cache.free_request(request)

    def reserve(self, request: Hashable, length: int) -> None:
        self.cache.reserve(request, length)

    # --------------------------------------------------------------------- step
    def _check(self, entries: Sequence[StepEntry]) -> List[EntryMeta]:
        """Refuses what a step cannot run; returns every entry's share of the step."""
        if not entries:
            raise StepError("a step needs at least one entry")
        seen = set()
        vocab = self.model.vocab_size
        live = self.cache.requests
        metas: List[EntryMeta] = []
        row = 0
        for e in entries:
            if e.request in seen:
                raise StepError(f"request {e.request!r} appears twice in one step")
            seen.add(e.request)
            held = live.get(e.request)
            if held is None:
                raise StepError(f"request {e.request!r} is not live (add_request first)")
            n = len(e.tokens)
            if n == 0:
                raise StepError(f"request {e.request!r} brings no tokens")
            start = held.computed
            if start + n > self.max_positions:
                raise StepError(f"request {e.request!r} would reach position {start + n - 1}, the model allows "
                                f"{self.max_positions} positions")
            if held.reserved < start + n:
                raise StepError(f"request {e.request!r}: pages are reserved for {held.reserved} "
                                f"tokens, the step needs {start + n}")
            if min(e.tokens) < 0 or max(e.tokens) >= vocab:
                bad = next(tok for tok in e.tokens if not 0 <= int(tok) < vocab)
                raise StepError(f"request {e.request!r}: token id {bad} is outside the vocabulary of {vocab}")
            for w in e.want:
                if not 0 <= int(w) < n:
                    raise StepError(f"request {e.request!r}: wanted place {w} is outside its {n} tokens")
            metas.append(EntryMeta(e.request, held.slot, start, n, row))
            row += n
        return metas

    def _layout(self, total: int, batch: int, wanted: int, widths: Sequence[int]) -> np.ndarray:
        """Offsets of the step's integer arrays in one flat buffer:
        [ids | positions | token_entry | start | count | first_row | slot | want | tables... | longest context]"""
        sizes = [total, total, total, batch, batch, batch + 1, batch, wanted] + [batch * w for w in widths] + [1]
        return np.concatenate([[0], np.cumsum(sizes)]).astype(np.int64)

    def _fill(self, flat: np.ndarray, offsets: np.ndarray, entries: Sequence[StepEntry], metas: List[EntryMeta],
              want_rows: List[int], widths: Sequence[int]) -> None:
        cache = self.cache
        total, batch = metas[-1].first_row + metas[-1].count, len(metas)
        ids, pos, tok_entry = (flat[offsets[i]:offsets[i + 1]] for i in range(3))
        for i, (e, m) in enumerate(zip(entries, metas)):
            sl = slice(m.first_row, m.first_row + m.count)
            ids[sl] = np.asarray(e.tokens, dtype=np.int32)
            pos[sl] = np.arange(m.start, m.start + m.count, dtype=np.int32)
            tok_entry[sl] = i
        flat[offsets[3]:offsets[4]] = [m.start for m in metas]
        flat[offsets[4]:offsets[5]] = [m.count for m in metas]
        flat[offsets[5]:offsets[6]] = [m.first_row for m in metas] + [total]
        flat[offsets[6]:offsets[7]] = [m.slot for m in metas]
        flat[offsets[7]:offsets[8]] = want_rows
        for gi, w in enumerate(widths):
            table = np.full((batch, w), -1, dtype=np.int32)
            for i, m in enumerate(metas):
                pages = cache.table(gi, m.request)[:w]
                table[i, :len(pages)] = pages
            flat[offsets[8 + gi]:offsets[9 + gi]] = table.reshape(-1)
        flat[offsets[8 + len(widths)]] = max(m.start + m.count for m in metas)

    def _refill(self, rec: "_Captured", entries: Sequence[StepEntry], metas: List[EntryMeta]) -> None:
        """The integers of a step of single tokens in a recording's buffer: only what changes from one such step to
        the next (ids, positions, slots, the longest context) and the block-table rows of requests whose tables have
        changed since the row was written (a request gets a page every ``page_size`` steps).  Token-to-entry map,
        counts, first rows and wanted rows are the same for every step of the recording's batch size."""
        flat, o, cache = rec.host_np, rec.offsets, self.cache
        starts = [m.start for m in metas]
        flat[o[0]:o[1]] = [e.tokens[0] for e in entries]
        flat[o[1]:o[2]] = starts
        flat[o[3]:o[4]] = starts
        flat[o[6]:o[7]] = [m.slot for m in metas]
        stamps = rec.row_stamps
        for i, m in enumerate(metas):
            stamp = cache.tables_stamp(m.request)
            if stamps[i] != stamp:
                stamps[i] = stamp
                for gi, w in enumerate(rec.widths):
                    pages = cache.table(gi, m.request)[:w]
                    at = int(o[8 + gi]) + i * w
                    flat[at:at + len(pages)] = pages
                    flat[at + len(pages):at + w] = -1
        flat[o[8 + len(rec.widths)]] = max(starts) + 1

    def _context(self, dev: torch.Tensor, offsets: np.ndarray, metas: List[EntryMeta], wanted: int,
                 widths: Sequence[int], workspace, max_context: int, uneven: bool) -> StepContext:
        total, batch = metas[-1].first_row + metas[-1].count, len(metas)
        part = [dev[offsets[i]:offsets[i + 1]] for i in range(len(offsets) - 1)]
        return StepContext(
            num_tokens=total, entries=metas, token_ids=part[0], positions=part[1], token_entry=part[2],
            entry_start=part[3], entry_count=part[4], entry_first_row=part[5], entry_slot=part[6],
            block_tables={gi: part[8 + gi].view(batch, w) for gi, w in enumerate(widths)},
            want_rows=part[7], num_wanted=wanted, workspace=workspace,
            max_count=max(m.count for m in metas), max_context=max_context, live_context=part[8 + len(widths)],
            uneven=uneven,
            upload=self._staging.upload_values)   # (the staging's method, not a closure over the step function: a
                                                   # recording keeps its context, and would keep the step function
                                                   # that holds it alive in a circle that only the collector ends)

    def _feed(self, ids: torch.Tensor, feed) -> None:
        """Token ids that are still on the device (the tokens the step before sampled, which the host has not seen
        yet) go into the step's ids there: ``feed = (source, places, rows)`` puts ``source[rows[i]]`` at
        ``ids[places[i]]``.  The entries hold any valid id at those places."""
        if feed is None:
            return
        source, places, rows = feed
        n = len(places)
        if n == 0:
            return
        if n == ids.numel() == source.numel() and places == rows == list(range(n)):
            ids.copy_(source)      # the same requests in the same order: the usual decoding step
            return
        both = self._staging.upload_values(list(places) + list(rows)).long()
        ids.index_copy_(0, both[:n], source.index_select(0, both[n:]))

    def step(self, entries: Sequence[StepEntry], feed=None) -> torch.Tensor:
        """One step of the model over the entries' tokens, from the cache; the logits at the wanted places.
        ``feed``: see ``_feed``."""
        metas = self._check(entries)
        cache = self.cache
        total = metas[-1].first_row + metas[-1].count
        want_rows = [m.first_row + int(w) for e, m in zip(entries, metas) for w in e.want]
        max_context = max(m.start + m.count for m in metas)
        uneven = contexts_uneven(metas)
        if self._graph_ok(entries, metas) and self._graph_ready(len(metas), max_context, uneven):
            logits = self._step_captured(entries, metas, want_rows, max_context, uneven, feed)
        else:
            widths = [max(1, max(g.pages_for(m.start + m.count) for m in metas)) for g in cache.groups]
            offsets = self._layout(total, len(metas), len(want_rows), widths)
            flat = np.zeros(int(offsets[-1]), dtype=np.int32)
            self._fill(flat, offsets, entries, metas, want_rows, widths)
            dev = self._staging.upload(flat)
            self._feed(dev[offsets[0]:offsets[1]], feed)
            ctx = self._context(dev, offsets, metas, len(want_rows), widths, self.model.workspace, max_context, uneven)
            logits = self.model.forward(ctx, self.views)
        for m in metas:
            cache.advance(m.request, m.start + m.count)
        self.steps += 1
        self.tokens_run += total
        return logits

    # ------------------------------------------------------- captured decoding
    # A step of single tokens (one per request, each wanting its logits) has the same launches every time,
    # so it is recorded once per (batch, context bucket, whether the contexts differ much: parts may share their work
    # out differently then) as a HIP graph over buffers of its own and replayed: the host then only copies the
    # step's integers and starts the graph.
    GRAPH_CONTEXT_BUCKET = 1024
    GRAPH_LIMIT = 64            # recordings kept
    GRAPH_AFTER_STEPS = 4       # a (batch, context bucket) is recorded when it comes for this many-th time

    def _graph_ok(self, entries: Sequence[StepEntry], metas: List[EntryMeta]) -> bool:
        """A step can be replayed if it has the form whose integers ``_refill`` rewrites (a token a request, every one
        wanting its logits) and the model says that such a step records (``recordable``: its parts issue the same
        launches whatever the step's values are, in this run mode, at this many rows)."""
        if not self.use_graphs:
            return False
        if not (all(m.count == 1 for m in metas) and all(list(e.want) == [0] for e in entries)):
            return False
        return self.model.recordable(metas)

    def _graph_key(self, batch: int, max_context: int, uneven: bool):
        bucket = (max_context + self.GRAPH_CONTEXT_BUCKET - 1) // self.GRAPH_CONTEXT_BUCKET * self.GRAPH_CONTEXT_BUCKET
        return batch, min(bucket, max(self.max_positions, max_context)), uneven

    def _graph_ready(self, batch: int, max_context: int, uneven: bool) -> bool:
        """A shape is recorded when it comes for the GRAPH_AFTER_STEPS-th time: recording costs about as much as a
        dozen steps, which a shape that a draining batch passes through once or twice never pays back."""
        key = self._graph_key(batch, max_context, uneven)
        if key in self._graphs:
            return True
        if key in self._graph_refused:
            return False
        seen = self._graph_seen.get(key, 0) + 1
        self._graph_seen[key] = seen
        return seen >= self.GRAPH_AFTER_STEPS

    def _step_captured(self, entries: Sequence[StepEntry], metas: List[EntryMeta], want_rows: List[int],
                       max_context: int, uneven: bool, feed=None) -> torch.Tensor:
        key = self._graph_key(len(metas), max_context, uneven)
        rec = self._graphs.get(key)
        if rec is None:
            # The step that meets a new shape runs eagerly (over the recording's own buffers, which sizes them) and is
            # recorded afterwards without being run again: a part with state of its own must see every step once.
            rec, logits = self._capture(key, entries, metas, want_rows, feed)
            if rec is None:
                self._graph_refused.add(key)
                return logits
            self._graphs[key] = rec
            self.graph_records += 1
            log.debug(f"recorded the step of {key[0]} tokens for contexts up to {key[1]}"
                      f"{' (uneven)' if key[2] else ''}: {self.graph_records} recordings")
            if len(self._graphs) > self.GRAPH_LIMIT:   # oldest recording out: contexts move on to higher buckets
                self._graphs.pop(next(iter(self._graphs)))
            return logits
        rec.wait()
        self._refill(rec, entries, metas)
        rec.dev.copy_(rec.host, non_blocking=True)
        rec.mark()      # (the pinned buffer is free again once this copy has run, whatever the graph still does)
        self._feed(rec.dev[rec.offsets[0]:rec.offsets[1]], feed)
        rec.graph.replay()
        self.graph_replays += 1
        return rec.logits.clone()

    def _capture(self, key, entries, metas, want_rows, feed=None):
        from ..parts.base import Workspace

        batch, bucket, uneven = key
        widths = [max(1, g.pages_for(bucket)) for g in self.cache.groups]
        offsets = self._layout(batch, batch, batch, widths)
        n = int(offsets[-1])
        host = torch.zeros(n, dtype=torch.int32, pin_memory=True)
        dev = torch.zeros(n, dtype=torch.int32, device=self.device)
        rec = _Captured(host=host, host_np=host.numpy(), dev=dev, offsets=offsets, widths=widths)
        workspace = Workspace(self.device)
        ctx = self._context(dev, offsets, metas, batch, widths, workspace, bucket, uneven)
        self._fill(rec.host_np, offsets, entries, metas, want_rows, widths)
        rec.row_stamps = [self.cache.tables_stamp(m.request) for m in metas]
        dev.copy_(host, non_blocking=True)
        self._feed(dev[offsets[0]:offsets[1]], feed)
        # the step itself, eagerly: it sizes the workspace and lets parts build what depends only on the step's shape
        from ..parts import linear

        library_before = linear.library_calls
        logits = self.model.forward(ctx, self.views)
        torch.cuda.synchronize()
        if linear.library_calls != library_before:
            return None, logits   # the step went through the vendor library somewhere: it is not recorded
        ctx.extras = {k: v for k, v in ctx.extras.items() if k.startswith("static:")}
        graph = torch.cuda.CUDAGraph()
        # No graph may be destroyed while a stream records (the runtime refuses it, and an error in a destructor ends
        # the process).  Python's collector runs whenever it likes, also in the middle of the recording, and what it
        # finds may hold graphs (another step function that was dropped, a caller's own): so it rests while the
        # stream records.  (It is not made to run first: a full collection takes 30 ms of a recording's 60.)
        collecting = gc.isenabled()
        gc.disable()
        try:
            with torch.cuda.graph(graph):
                rec.logits = self.model.forward(ctx, self.views)
        finally:
            if collecting:
                gc.enable()
        rec.graph = graph
        rec.workspace = workspace
        rec.context = ctx
        rec.mark()
        return rec, logits
