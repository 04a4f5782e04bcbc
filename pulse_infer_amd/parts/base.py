"""What a part is, and the registries that parts are chosen from.

A model is put together from five kinds of part, each registered under a name
and built from a ``PartSpec`` (its kind and its parameters):

* **mixer** — mixes information along the sequence (attention here).
  ``cache_spec()`` says what it keeps between steps; ``forward(x, ctx, cache)``
  maps the normed input ``[T, H]`` to the update of the residual ``[T, H]``.
* **feed-forward** — ``forward(x, ctx)``, token by token.
* **norm** — ``apply(h, delta, out, rows)``: normalise ``h + delta`` (float32
  residual), optionally only gathered rows.
* **position encoding** — ``prepare(ctx)`` once per step gives whatever its
  mixers consume (rotation tables here).
* **block** — the arrangement of the above around the residual stream.

Two more kinds stand at the model's ends: the **embedding**
(``forward(ids, out)`` fills the float32 residual) and the **output head**
(``forward(x, out)`` gives float32 logits for the normed rows it is handed; it
is built with the embedding at hand, for weights the two share).

Every part states the tensors it loads with ``weight_specs(params)`` (names
relative to its prefix), so the loader can check a checkpoint, and the random
initialiser can create one, before anything is built.  No part knows which
model it is in; sizes and constants arrive as parameters.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Callable, Dict, List, Optional, Tuple

import torch

from ..cache.specs import PagedCacheView, StateView  # noqa: F401  (what a mixer is handed as its cache)
from ..weights.store import TensorSpec, WeightLoader


class Registry:
    """Name -> class, one per kind of part."""

    def __init__(self, what: str):
        self.what = what
        self._items: Dict[str, Any] = {}

    def register(self, name: str, replace: bool = False) -> Callable[[Any], Any]:
        def deco(cls: Any) -> Any:
            if name in self._items and not replace:
                raise ValueError(f"{self.what} '{name}' is already registered")
            self._items[name] = cls
            cls.kind = name
            return cls
        return deco

    def unregister(self, name: str) -> None:
        self._items.pop(name, None)

    def get(self, name: str) -> Any:
        try:
            return self._items[name]
        except KeyError:
            raise KeyError(f"unknown {self.what} '{name}'; registered: {', '.join(sorted(self._items)) or '<none>'}") from None

    def names(self) -> List[str]:
        return sorted(self._items)


MIXERS = Registry("mixer")
FEED_FORWARDS = Registry("feed-forward")
NORMS = Registry("norm")
POSITIONS = Registry("position encoding")
BLOCKS = Registry("block")
EMBEDDINGS = Registry("embedding")
HEADS = Registry("output head")


class Workspace:
    """Named device buffers that grow to the largest size asked for and are reused by every step."""

    def __init__(self, device: torch.device):
        self.device = device
        self._flat: Dict[Tuple[str, torch.dtype], torch.Tensor] = {}
        self._views: Dict[Tuple[str, torch.dtype, int, int], torch.Tensor] = {}   # what buffer() handed out before

    def buffer(self, name: str, rows: int, cols: int, dtype: torch.dtype) -> torch.Tensor:
        view = self._views.get((name, dtype, rows, cols))
        if view is not None:
            return view
        need = max(1, rows * cols)
        key = (name, dtype)
        flat = self._flat.get(key)
        if flat is None or flat.numel() < need:
            flat = torch.empty(need, dtype=dtype, device=self.device)
            self._flat[key] = flat
            for old in [k for k in self._views if k[0] == name and k[1] == dtype]:   # views of the buffer it replaces
                del self._views[old]
        view = flat[: rows * cols].view(rows, cols)
        if len(self._views) >= 4096:   # steps of ever new sizes: start over rather than grow without end
            self._views.clear()
        self._views[(name, dtype, rows, cols)] = view
        return view


@dataclass
class BuildContext:
    """What a part gets when it is built."""

    loader: WeightLoader
    mode: str                    # "bfloat16" or "float32": how the run computes
    device: torch.device
    act_dtype: torch.dtype       # storage type of activations between kernels
    workspace: Workspace
    positions: Dict[str, Any] = field(default_factory=dict)  # name -> position encoding instance
    options: Dict[str, Any] = field(default_factory=dict)


@dataclass
class EntryMeta:
    """One request's share of a step (host side)."""

    request: Any
    slot: int
    start: int      # position of its first token in this step = tokens already in the cache
    count: int      # tokens in this step
    first_row: int  # where they start among the step's tokens


UNEVEN_CONTEXTS = 1.5     # longest context / mean context from which a step counts as uneven
UNEVEN_MIN_ENTRIES = 3


def contexts_uneven(entries: List[EntryMeta]) -> bool:
    """Whether a step's requests hold contexts that differ much (``StepContext.uneven``)."""
    if len(entries) < UNEVEN_MIN_ENTRIES:
        return False
    longest = total = 0
    for e in entries:
        c = e.start + e.count
        total += c
        if c > longest:
            longest = c
    return longest * len(entries) >= UNEVEN_CONTEXTS * total


@dataclass
class StepContext:
    """Everything a part may need to know about the step being run."""

    num_tokens: int
    entries: List[EntryMeta]
    token_ids: torch.Tensor      # int32 [T]
    positions: torch.Tensor      # int32 [T]
    token_entry: torch.Tensor    # int32 [T] index into entries
    entry_start: torch.Tensor    # int32 [B]
    entry_count: torch.Tensor    # int32 [B]
    entry_first_row: torch.Tensor  # int32 [B + 1] (prefix sums of counts)
    entry_slot: torch.Tensor     # int32 [B]
    block_tables: Dict[int, torch.Tensor]  # group -> int32 [B, width]
    want_rows: torch.Tensor      # int32 [R] rows whose logits are wanted
    num_wanted: int
    workspace: Workspace
    max_count: int = 1           # most tokens of one entry
    max_context: int = 1         # longest context (start + count) of an entry that the step's launches must cover
                                 # (of a recorded step: the most its replays may bring)
    live_context: Optional[torch.Tensor] = None   # int32 [1] on the device: the longest context as it is in this
                                                  # step (at most max_context), for kernels that shape their work by it
    uneven: bool = False         # the requests' contexts differ much (the longest at least UNEVEN_CONTEXTS times
                                 # their mean): a part may share its work out differently then; a recorded step is
                                 # recorded for one case or the other
    extras: Dict[str, Any] = field(default_factory=dict)  # per-step products of position encodings etc.
    upload: Optional[Callable[[List[int]], torch.Tensor]] = None   # integers of a part's own to the device, through the
                                                                   # step function's pinned staging (no synchronous copy)

    def to_device(self, values: List[int]) -> torch.Tensor:
        """An int32 device vector of ``values`` (work lists that a part builds from the step's entries)."""
        if self.upload is not None:
            return self.upload(values)
        return torch.tensor(values, dtype=torch.int32, device=self.token_ids.device)

    def position_product(self, name: str, encodings: Dict[str, Any]) -> Any:
        """What position encoding ``name`` prepared for this step (prepared on first use)."""
        key = f"position:{name}"
        if key not in self.extras:
            self.extras[key] = encodings[name].prepare(self)
        return self.extras[key]


@dataclass
class RowStats:
    """What a part that added into the residual itself knows about the new rows: their sums of squares, in parts
    (``sumsq`` [rows, parts] float32), and the rows themselves once more, every column multiplied by ``scaled_by``
    (the weight of the norm that was expected to read them next; None: as they are) and rounded to the activations'
    type (``rounded`` [rows, H]).  What is left of that norm, a division of each row, can then move behind its
    consumer's first product."""

    sumsq: torch.Tensor
    rounded: Optional[torch.Tensor] = None
    scaled_by: Optional[torch.Tensor] = None


@dataclass
class LazyNorm:
    """A normalised input that has not been computed: the rows of ``x`` (the residual ``h`` times the norm's weight,
    rounded) each still to be divided by sqrt(mean of the squares of its row of ``h`` + eps), the mean taken from the
    sums of squares in ``sumsq`` [rows, parts].  A consumer whose first product is linear (``accepts_lazy_input``)
    multiplies the rows of that product's result instead, which is the same and costs nothing.  ``materialize``
    computes the input the ordinary way."""

    x: torch.Tensor
    sumsq: torch.Tensor
    eps: float
    h: torch.Tensor
    norm: Any

    @property
    def shape(self):
        return self.x.shape

    def materialize(self, out: torch.Tensor) -> torch.Tensor:
        return self.norm.apply(self.h, None, out)


class ResidualStream:
    """The float32 residual ``h`` and the update that has not been added to it yet.

    Adding is deferred so that it happens inside the next norm's kernel.  A part that added its result itself may
    hand back ``RowStats`` of the new ``h``; they stay valid until ``h`` changes again.
    """

    def __init__(self, h: torch.Tensor):
        self.h = h
        self.pending: Optional[torch.Tensor] = None
        self.stats: Optional[RowStats] = None
        self.after_block: Any = None   # the norm that reads the residual first once the block in hand is through
                                       # (set by whoever runs the blocks; None: unknown, or no norm)

    def pending_for(self, norm: Any) -> Optional[torch.Tensor]:
        """The update not yet added, in a form ``norm`` takes: an update in parts ([parts, T, H] float32, the shares of
        a product whose inner dimension was split) is added to ``h`` first unless the norm says ``takes_parts``."""
        pending, self.pending = self.pending, None
        if pending is not None and pending.dim() == 3 and not getattr(norm, "takes_parts", False):
            from ..ops import kernels
            kernels.residual_add(self.h, pending)
            return None
        return pending

    def normed(self, norm: Any, out: torch.Tensor) -> torch.Tensor:
        norm.apply(self.h, self.pending_for(norm), out)
        return out

    def lazy(self, norm: Any) -> Optional[LazyNorm]:
        """The norm of the current ``h`` as something a consumer can compute itself, if the norm allows that and the
        rows' statistics are at hand."""
        if self.pending is not None or self.stats is None or not hasattr(norm, "lazy"):
            return None
        return norm.lazy(self.h, self.stats)

    def push(self, delta: Any) -> None:
        """Hand over an update ([T, H], or [parts, T, H] float32 to be added in order); None or RowStats mean the part
        has already added it to ``h``."""
        if isinstance(delta, RowStats):
            self.stats = delta
            return
        self.stats = None
        if delta is None:
            return
        if self.pending is not None:
            from ..ops import kernels
            kernels.residual_add(self.h, self.pending)
        self.pending = delta


@dataclass
class StepCost:
    """What a step costs a part: arithmetic, the weights it has to read (once a step, whatever the rows), and what
    it reads of its cache."""

    flops: float = 0.0
    weight_bytes: float = 0.0
    cache_bytes: float = 0.0

    def __add__(self, other: "StepCost") -> "StepCost":
        return StepCost(self.flops + other.flops, self.weight_bytes + other.weight_bytes,
                        self.cache_bytes + other.cache_bytes)


class Part:
    """Base of all parts: declares the tensors it loads and what a step costs it."""

    kind = "?"
    # A step that runs this part may be recorded as a graph and replayed only if the part says so: its forward
    # must then issue the same launches whatever the step's values are (request slots, positions and tables read
    # on the device from the step's arrays, no host decision on them, no synchronisation, no library call that
    # clears memory).  Parts that do not say so keep a model's steps eager.
    records_cleanly = False

    @classmethod
    def weight_specs(cls, params: Dict[str, Any]) -> Dict[str, TensorSpec]:
        return {}

    @classmethod
    def step_cost(cls, params: Dict[str, Any], entries: List[Tuple[int, int]], weight_bytes: int,
                  cache_bytes: int) -> StepCost:
        """The cost of one step of ``entries`` ((tokens already cached, tokens in this step) per request), with
        ``weight_bytes`` / ``cache_bytes`` a stored element.  Unless a part knows better: every tensor is read once
        and every matrix is multiplied with every row.  Parts with a cache add what they read of it and the
        arithmetic over it; a part that reads only some of its tensors (chosen experts) overrides the whole."""
        rows = sum(count for _, count in entries)
        cost = StepCost()
        for spec in cls.weight_specs(params).values():
            n = 1
            for dim in spec.shape:
                n *= dim
            cost.weight_bytes += n * weight_bytes
            if len(spec.shape) == 2 and spec.kind == "linear":
                cost.flops += 2.0 * rows * n
        return cost


def says(part: Any, name: str) -> bool:
    """A part's yes or no to ``name``, whether it gives it as an attribute or as a method; a part that does not say
    is a no."""
    value = getattr(part, name, False)
    return bool(value() if callable(value) else value)


def joined(prefix: str, name: str) -> str:
    return f"{prefix}.{name}" if prefix else name
