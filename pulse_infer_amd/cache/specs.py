"""What a run of the model keeps between steps, said by its mixer as a cache spec.

A spec is a small hashable object that the cache manager asks, never inspects:

* ``per_token`` — True: the run stores something for every token of a request, in
  pages (a page pool and a block table per request, shared by all runs whose specs
  are equal); False: one array of fixed size per request, addressed by the
  request's slot.
* ``window`` (per-token specs) — None: every token is kept; n: only the last n
  tokens are ever read, so pages wholly below the window go back to the pool
  while the request still runs.
* ``bytes_per_token(element_size)`` (per-token specs) — what one token costs one
  run, for sizing pools and pricing steps.
* ``allocate(runs, units, page_size, device, dtype)`` — the storage of all runs of
  a group (``units`` pages of ``page_size`` tokens each) or of one run's state
  (``units`` slots; ``runs`` is 1).  Whatever it returns is kept as it is.
* ``view(storage, index, group, page_size, writable)`` — what run ``index`` of the
  group is handed as ``cache`` in ``forward``: its slice of the storage and what it
  needs to address it (``group`` is the key into ``StepContext.block_tables``).
* ``tensors(storage)`` — the storage's tensors, for whoever counts or fills them.

Two specs are provided: keys and values of attention heads in pages, and a plain
array per request.  A mixer that pages something else per token (one row of some
width, keys and values of different widths, the tail of a convolution) brings a
spec class of its own with these members; nothing in the cache manager or the
step function changes.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, List, Optional, Tuple


@dataclass
class PagedCacheView:
    """The pages of one run of a group of attention layers."""

    group: int
    keys: Any              # [pages, kv_heads, page_size, head_dim]
    values: Any            # [pages, kv_heads, head_dim, page_size]
    page_size: int
    writable: bool = True  # False: the run reads a cache that another run writes


@dataclass
class StateView:
    """The per-request state of one run: row ``slot`` belongs to the request in that slot."""

    state: Any             # [slots, *shape]


@dataclass(frozen=True)
class PagedKVSpec:
    """Keys and values of ``num_kv_heads`` heads of ``head_dim`` channels for every token.

    Storage: K ``[runs, pages, kv_heads, page, head_dim]`` and V ``[runs, pages, kv_heads, head_dim, page]``: values
    lie transposed inside a page, so that both matrix-core operands of attention are direct 16-/8-byte loads."""

    num_kv_heads: int
    head_dim: int
    window: Optional[int] = None  # None: all keys

    per_token = True

    def bytes_per_token(self, element_size: int) -> int:
        return 2 * self.num_kv_heads * self.head_dim * element_size

    def allocate(self, runs: int, units: int, page_size: int, device: Any, dtype: Any) -> Tuple[Any, Any]:
        import torch

        keys = torch.zeros((runs, units, self.num_kv_heads, page_size, self.head_dim), dtype=dtype, device=device)
        values = torch.zeros((runs, units, self.num_kv_heads, self.head_dim, page_size), dtype=dtype, device=device)
        return keys, values

    def view(self, storage: Tuple[Any, Any], index: int, group: int, page_size: int, writable: bool) -> PagedCacheView:
        keys, values = storage
        return PagedCacheView(group=group, keys=keys[index], values=values[index], page_size=page_size,
                              writable=writable)

    def tensors(self, storage: Tuple[Any, Any]) -> List[Any]:
        return list(storage)


@dataclass(frozen=True)
class StateSpec:
    """One array of ``shape`` per request, of a storage type of its own (the run mode does not change it)."""

    shape: Tuple[int, ...]
    dtype: str = "float32"

    per_token = False

    def allocate(self, runs: int, units: int, page_size: int, device: Any, dtype: Any) -> Any:
        import torch

        return torch.zeros((units, *self.shape), dtype=getattr(torch, self.dtype), device=device)

    def view(self, storage: Any, index: int, group: int, page_size: int, writable: bool) -> StateView:
        return StateView(storage)

    def tensors(self, storage: Any) -> List[Any]:
        return [storage]


def check_spec(spec: Any, run: int) -> None:
    """A clear error for something that is no cache spec."""
    if not isinstance(getattr(spec, "per_token", None), bool) or not all(
            callable(getattr(spec, name, None)) for name in ("allocate", "view", "tensors")):
        raise TypeError(f"run {run}: {spec!r} is no cache spec (it needs per_token, allocate, view and tensors; "
                        "per-token specs also window and bytes_per_token)")
    if spec.per_token and not callable(getattr(spec, "bytes_per_token", None)):
        raise TypeError(f"run {run}: the per-token cache spec {spec!r} does not say bytes_per_token")
    try:
        hash(spec)
    except TypeError:
        raise TypeError(f"run {run}: the cache spec {spec!r} is not hashable (runs with equal specs share a pool)") from None
