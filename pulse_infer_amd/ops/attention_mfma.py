"""The matrix-core attention kernel (bfloat16), one compiled library per head size."""
from __future__ import annotations

import ctypes
from typing import List, Optional, Sequence, Tuple

import torch

from .device import compute_units
from .kernels import _check_cache, _f32, _gpu, _i32, _i64, _int_vec, _need, _ptr, _stream
from .library import call_in, load_variant

MAX_HEAD_DIM = 224
BLOCK_KEYS = 32


def supported(head_dim: int, page_size: int, dtype: torch.dtype, cache_dtype: torch.dtype) -> bool:
    """Sizes the kernel takes; anything else goes to the generic kernel."""
    return (dtype == torch.bfloat16 and cache_dtype == torch.bfloat16 and head_dim % 16 == 0
            and 16 <= head_dim <= MAX_HEAD_DIM and page_size % 16 == 0)


def tokens_per_item(group: int) -> int:
    """How many consecutive tokens of a request share one work item (16 columns / heads per kv head)."""
    gp = 1
    while gp < group and gp < 16:
        gp *= 2
    return 16 // gp


PORTION_MIN_TOKENS = 16   # entries with at least this many tokens go to the kernel that shares keys through LDS
PORTION_WAVES = 4         # wavefronts of its workgroup


def portion_tokens(group: int, head_dim: int) -> int:
    """Tokens of one work item of the prompt-portion kernel: its four wavefronts take one or two column tiles of
    ``tokens_per_item`` tokens each (two for the head sizes its wide variant takes)."""
    return tokens_per_item(group) * PORTION_WAVES * (2 if head_dim in (32, 64, 128) else 1)


ITEM_INTS = 4


def build_items(entries: Sequence, tokens_per: int) -> List[int]:
    """Flat [first row, token count, row of the block table, 0] quadruples covering the given entries of a step.

    ``entries`` are (index of the entry in the step, entry) pairs: the index is the entry's row of the block table
    (what ``token_entry`` holds for its tokens), so that a kernel finds the table with the item alone."""
    flat: List[int] = []
    for index, e in entries:
        for b in range(0, e.count, tokens_per):
            flat.extend((e.first_row + b, min(tokens_per, e.count - b), index, 0))
    return flat


def split_entries(entries: Sequence):
    """(single tokens and short portions, long portions), each as (index in the step, entry) pairs"""
    numbered = list(enumerate(entries))
    short = [(i, e) for i, e in numbered if e.count < PORTION_MIN_TOKENS]
    long = [(i, e) for i, e in numbered if e.count >= PORTION_MIN_TOKENS]
    return short, long


SPLIT_OVERHEAD_KEYS = 256      # what a workgroup costs beside its walk (start-up, merge inside it), in keys walked
MERGE_OVERHEAD_KEYS = 350      # what splitting at all costs (partial results through memory, the second kernel)
MIN_SPLIT_KEYS = 64            # no split is shorter
MAX_CHOSEN_SPLITS = 64


def choose_splits(num_items: int, nkv: int, group: int, max_context: int) -> Tuple[int, int]:
    """(split_size, n_splits) for the kernel of decoded tokens and short portions.

    The kernel's time is that of the compute unit with the longest walk: the workgroups that land on it times the
    keys of a split plus a fixed cost each, and splitting at all costs the partial results' trip through memory and
    the second kernel.  The number of splits with the least such cost is taken.  Measured at 8 kv heads of 4 query
    heads, contexts of 4,096: one request is fastest in 32 splits, two in 16, four in 8, eight in 4 (256 workgroups
    each time; 6 splits at batch 8, which leave half the units two workgroups, are 15% slower); 20 to 32 requests in
    one (160 to 256 workgroups; two splits are 10 to 25% slower), 40 in 4 and 48 in 2 (a multiple of the units
    again), 64 in one.  Walks of 4,096 keys and more stream better with two workgroups a unit (16 requests at 8,192:
    4 splits 95.9 us, 2 splits 97.6; at 4,096, walks of 2,048 keys, 2 splits 51.9 us and 4 splits 53.8), so a choice
    that gives every unit one such walk is cut in two once more.  Short contexts (the merge's cost as it was measured
    there, 5 to 6 us, about 350 keys' worth of a walk): 8 requests of 512 keys 15.0 us whole and 13.1 in four splits,
    16 of 1,024 25.0 whole and 21.8 in two, one of 1,024 11.6 in 8 splits and 10.3 in 16."""
    units = compute_units()        # the split kernel's workgroups are counted against them
    groups = num_items * nkv * ((group + 15) // 16)
    whole = (max_context + BLOCK_KEYS - 1) // BLOCK_KEYS * BLOCK_KEYS
    if groups <= 0 or max_context <= 0:
        return max(whole, BLOCK_KEYS), 1

    def split_size(n: int) -> int:
        return ((max_context + n - 1) // n + BLOCK_KEYS - 1) // BLOCK_KEYS * BLOCK_KEYS

    best = None
    for n in range(1, MAX_CHOSEN_SPLITS + 1):
        size = split_size(n)
        if n > 1 and (size < MIN_SPLIT_KEYS or (n - 1) * size >= max_context):
            continue
        on_a_unit = (groups * n + units - 1) // units
        # (more workgroups than the units hold at a time, two each, wait for one another: 24 requests of 4,096 keys
        # take 79 us whole and 85 in four splits, which this rule's sums alone would prefer)
        merge = 0 if n == 1 else MERGE_OVERHEAD_KEYS * (2 if groups * n > 2 * units else 1)
        cost = on_a_unit * (size + SPLIT_OVERHEAD_KEYS) + merge
        if best is None or cost < best[0]:
            best = (cost, n)
    n = best[1]
    if n > 1 and split_size(n) >= 4096 and groups * n * 2 in (units, 2 * units):
        n *= 2
    if n == 1:
        return whole, 1
    size = split_size(n)
    return size, (max_context + size - 1) // size


def attn_mfma(q: torch.Tensor, out: torch.Tensor, nq: int, nkv: int, d: int, kcache: torch.Tensor,
              vcache: torch.Tensor, positions: torch.Tensor, block_table: torch.Tensor,
              items: torch.Tensor, scale: float, window: int, split_size: int, n_splits: int, max_context: int,
              part_o: Optional[torch.Tensor], part_ml: Optional[torch.Tensor],
              live_context: Optional[torch.Tensor] = None, plan: Optional[torch.Tensor] = None) -> None:
    """Attention of decoded tokens and short portions.  ``split_size`` x ``n_splits`` is what the launch is made for
    (contexts up to ``max_context``); ``live_context`` (one int32 on the device: the longest context among the step's
    entries as it is now) lets the kernel cut the keys that are there evenly into the same number of splits;
    ``plan`` (what ``attn_plan`` made of these items for this ``n_splits``) takes the place of that even cut."""
    _gpu("attn_mfma", q, out, kcache, vcache, positions, block_table, items, part_o, part_ml, live_context, plan)
    _live(live_context)
    _planned(plan, items.numel() // ITEM_INTS, n_splits)
    tokens = q.shape[0]
    _need(q.dtype == torch.bfloat16 and out.dtype == torch.bfloat16 and q.stride(1) == 1 and out.stride(1) == 1,
          "attn_mfma: q and out must be bfloat16 matrices with contiguous rows")
    _need(q.shape[1] >= nq * d and out.shape[1] >= nq * d and out.shape[0] == tokens, "attn_mfma: q/out too narrow")
    pages, page_size = _check_cache("attn_mfma", kcache, vcache, nkv, d)
    _need(supported(d, page_size, q.dtype, kcache.dtype), f"attn_mfma: head size {d} / page size {page_size} / "
          f"{kcache.dtype} is not supported by the matrix-core kernel")
    _int_vec("attn_mfma: positions", positions, tokens)
    _need(block_table.dim() == 2 and block_table.dtype == torch.int32 and block_table.is_contiguous(),
          "attn_mfma: block_table must be contiguous int32 [entries, width]")
    _need(items.dtype == torch.int32 and items.is_contiguous() and items.numel() % ITEM_INTS == 0,
          "attn_mfma: items must be int32 quadruples")
    n_items = items.numel() // ITEM_INTS
    if n_splits > 1:
        need = tokens * nq * n_splits
        _need(part_o is not None and part_ml is not None and part_o.dtype == torch.float32
              and part_ml.dtype == torch.float32 and part_o.numel() >= need * d and part_ml.numel() >= need * 2,
              "attn_mfma: scratch for the split results is too small")
    lib = load_variant("attn_mfma", {"PULSE_HEAD_DIM": d})
    call_in(lib, "pulse_attn_mfma", _ptr(q), _i64(q.stride(0)), _ptr(out), _i64(out.stride(0)), _ptr(kcache),
            _ptr(vcache), _ptr(positions), _ptr(block_table), _i32(block_table.shape[1]),
            _ptr(items), _i32(n_items), _i32(tokens), _i32(nq), _i32(nkv), _i32(page_size), _i32(pages), _f32(scale),
            _i32(window), _i32(split_size), _i32(n_splits), _i32(max_context), _ptr(part_o), _ptr(part_ml),
            _ptr(live_context), _ptr(plan), _stream())


PLAN_MIN_KEYS = 256      # no split of a plan is shorter (what a workgroup costs beside its walk, in keys walked)
PLAN_SPLITS = 8          # most splits of an item in a planned step


def plan_ints(n_items: int, n_splits: int) -> int:
    """int32 values of a plan for ``n_items`` items in up to ``n_splits`` splits."""
    return 1 + n_items * n_splits + n_items


def plan_slots(nkv: int, group: int) -> Tuple[int, int]:
    """(slots, first_wave) for ``attn_plan``: the workgroups of one kv head (and chunk of 16 heads) that the compute
    units hold at a time, two a unit, and how many of them land on a unit of their own."""
    heads = nkv * ((group + 15) // 16)
    first = max(1, compute_units() // heads)
    return 2 * first, first


def plan_fits(n_items: int, n_splits: int) -> bool:
    return 1 <= n_items and n_items * n_splits <= 1024     # PLAN_MAX_PAIRS of attn_mfma.hip


def attn_plan(items: Optional[torch.Tensor], positions: torch.Tensor, n_splits: int, slots: int, first_wave: int,
              plan: torch.Tensor, d: int, min_keys: int = PLAN_MIN_KEYS) -> None:
    """The plan of a step whose contexts differ much (on the device, from ``positions`` as they are now): every
    item's keys are cut into min(n_splits, ceil(context / T)) even splits, T the smallest length with at most
    ``slots`` (item, split) pairs in all, and the pairs are put in the order the workgroups take them, longest first.
    ``plan``: int32 [plan_ints(items, n_splits)], to be passed to ``attn_mfma`` / ``attn_decode`` with the same items,
    positions and n_splits."""
    _gpu("attn_plan", items, positions, plan)
    if items is None:        # every token an item of its own, in order (decoded tokens)
        n_items = positions.numel()
    else:
        n_items = items.numel() // ITEM_INTS
        _need(items.dtype == torch.int32 and items.is_contiguous() and items.numel() % ITEM_INTS == 0,
              "attn_plan: items must be int32 quadruples")
    _need(positions.dtype == torch.int32 and positions.is_contiguous(), "attn_plan: positions must be contiguous int32")
    _need(plan_fits(n_items, n_splits), f"attn_plan: {n_items} items in up to {n_splits} splits do not fit a plan")
    _planned(plan, n_items, n_splits)
    lib = load_variant("attn_mfma", {"PULSE_HEAD_DIM": d})
    call_in(lib, "pulse_attn_plan", _ptr(items), _ptr(positions), _i32(n_items), _i32(n_splits), _i32(slots),
            _i32(first_wave), _i32(min_keys), _ptr(plan), _stream())


def _planned(plan: Optional[torch.Tensor], n_items: int, n_splits: int) -> None:
    _need(plan is None or (plan.dtype == torch.int32 and plan.is_contiguous()
                           and plan.numel() >= plan_ints(n_items, n_splits)),
          f"attention: a plan must hold {plan_ints(n_items, n_splits)} contiguous int32 values")


def _live(live_context: Optional[torch.Tensor]) -> None:
    _need(live_context is None or (live_context.dtype == torch.int32 and live_context.numel() >= 1
                                   and live_context.is_contiguous()),
          "the live context must be an int32 value on the device")


PREFILL_SPLIT_KEYS = 64        # a split of the prompt-portion kernel is a whole number of its 64-key blocks
PREFILL_SPLIT_HEAD_DIMS = (32, 64, 128)
PREFILL_MAX_SPLITS = 64
PREFILL_SCRATCH_BYTES = 1 << 30
TAIL_SPLIT_MIN_BLOCKS = 64     # walks from here on (4,096 keys) are worth a cut at three quarters on a full chip


def choose_prefill_splits(entries: Sequence, portion: int, nkv: int, group: int, d: int, window: int,
                          target_groups: Optional[int] = None, min_blocks: int = 8) -> Tuple[int, int]:
    """(split_size, n_splits) for the prompt-portion kernel over these (index, entry) pairs.

    A workgroup walks its item's keys block by block, so the longest item sets the kernel's time while the chip
    waits.  Cutting the keys into splits with workgroups of their own pays when there are fewer workgroups than the
    chip runs at a time (``target_groups``, two a compute unit unless given; a short portion over a long context):
    they get as many splits as fill it.  Splits never hold fewer than ``min_blocks`` blocks, and nothing is cut
    otherwise, but for the tail of a long whole prompt (below): the partial results cost a trip through memory and a
    second launch (2,048 tokens: 64.7 us whole, 67.4 cut at 1,664 keys, 88 at 1,024)."""
    if d not in PREFILL_SPLIT_HEAD_DIMS or window > 0:   # (a window keeps every walk short)
        return 0, 1
    if target_groups is None:
        target_groups = 2 * compute_units()
    longest = tokens = items = 0
    walks = []
    for _, e in entries:
        tokens += e.count
        for b in range(0, e.count, portion):
            blocks = (e.start + min(b + portion, e.count) - 1) // PREFILL_SPLIT_KEYS + 1
            longest = max(longest, blocks)
            walks.append(blocks)
            items += 1
    if items == 0:
        return 0, 1
    per_item = nkv * ((group + 15) // 16)
    groups = items * per_item
    budget = PREFILL_SCRATCH_BYTES // max(1, tokens * nkv * group * d * 4)
    if groups >= target_groups:
        # A full chip.  What is left to gain is the end of the kernel, when the few items with the longest walks run
        # on while most units are idle: a whole prompt, whose walks grow from one block to all of them.  From 4,096
        # keys on, cutting at three quarters of the longest walk gives that last quarter of the items a short
        # second split (measured, one prompt: 4,096 tokens 228 -> 207 us, 8,192 677 -> 636, 16,384 2,439 -> 2,328;
        # cuts at 5/8 to 7/8 are within 2% of each other; at 2,048 tokens nothing is gained).  Items that all walk
        # about as far (portions deep inside a context) would all pay for the detour and are left whole.
        cut = 3 * longest // 4
        late = sum(1 for w in walks if w > cut)
        if longest >= TAIL_SPLIT_MIN_BLOCKS and budget >= 2 and 10 * late <= 3 * items:
            return cut * PREFILL_SPLIT_KEYS, 2
        return 0, 1
    size = max(min_blocks, (longest * groups + target_groups - 1) // target_groups)
    n_splits = (longest + size - 1) // size
    n_splits = min(n_splits, PREFILL_MAX_SPLITS, max(1, budget))
    if n_splits <= 1:
        return 0, 1
    size = (longest + n_splits - 1) // n_splits   # splits of equal length
    return size * PREFILL_SPLIT_KEYS, (longest + size - 1) // size


def attn_prefill(q: torch.Tensor, out: torch.Tensor, nq: int, nkv: int, d: int, kcache: torch.Tensor,
                 vcache: torch.Tensor, positions: torch.Tensor, block_table: torch.Tensor,
                 items: torch.Tensor, scale: float, window: int, split_size: int = 0, n_splits: int = 1,
                 part_o: Optional[torch.Tensor] = None, part_ml: Optional[torch.Tensor] = None) -> None:
    """Attention for prompt portions: items of up to portion_tokens(group, d) tokens, keys shared through LDS.
    With ``n_splits > 1`` the keys are walked in splits of ``split_size`` (a multiple of 64) by workgroups of their
    own and merged by a second kernel; ``part_o`` / ``part_ml`` are float32 scratch of tokens * nq * n_splits * d
    and * 2 elements."""
    _gpu("attn_prefill", q, out, kcache, vcache, positions, block_table, items, part_o, part_ml)
    tokens = q.shape[0]
    if n_splits > 1:
        _need(d in PREFILL_SPLIT_HEAD_DIMS, f"attn_prefill: head size {d} has no split variant")
        _need(split_size > 0 and split_size % PREFILL_SPLIT_KEYS == 0,
              f"attn_prefill: split size {split_size} must be a positive multiple of {PREFILL_SPLIT_KEYS}")
        need = tokens * nq * n_splits
        _need(part_o is not None and part_ml is not None and part_o.dtype == torch.float32
              and part_ml.dtype == torch.float32 and part_o.numel() >= need * d and part_ml.numel() >= need * 2,
              "attn_prefill: scratch for the split results is too small")
    _need(q.dtype == torch.bfloat16 and out.dtype == torch.bfloat16 and q.stride(1) == 1 and out.stride(1) == 1,
          "attn_prefill: q and out must be bfloat16 matrices with contiguous rows")
    _need(q.shape[1] >= nq * d and out.shape[1] >= nq * d and out.shape[0] == tokens, "attn_prefill: q/out too narrow")
    pages, page_size = _check_cache("attn_prefill", kcache, vcache, nkv, d)
    _need(supported(d, page_size, q.dtype, kcache.dtype), f"attn_prefill: head size {d} / page size {page_size} / "
          f"{kcache.dtype} is not supported by the matrix-core kernel")
    _int_vec("attn_prefill: positions", positions, tokens)
    _need(block_table.dim() == 2 and block_table.dtype == torch.int32 and block_table.is_contiguous(),
          "attn_prefill: block_table must be contiguous int32 [entries, width]")
    _need(items.dtype == torch.int32 and items.is_contiguous() and items.numel() % ITEM_INTS == 0,
          "attn_prefill: items must be int32 quadruples")
    lib = load_variant("attn_mfma", {"PULSE_HEAD_DIM": d})
    call_in(lib, "pulse_attn_prefill", _ptr(q), _i64(q.stride(0)), _ptr(out), _i64(out.stride(0)), _ptr(kcache),
            _ptr(vcache), _ptr(positions), _ptr(block_table), _i32(block_table.shape[1]),
            _ptr(items), _i32(items.numel() // ITEM_INTS), _i32(tokens), _i32(nq), _i32(nkv), _i32(page_size), _i32(pages),
            _f32(scale), _i32(window), _i32(split_size if n_splits > 1 else 0), _i32(n_splits),
            _ptr(part_o if n_splits > 1 else None), _ptr(part_ml if n_splits > 1 else None), _stream())


def decode_takes(d: int, rotary_dim: int, pairing: int) -> bool:
    """Whether ``attn_decode`` can rotate ``rotary_dim`` channels with this pairing for head size ``d``."""
    lib = load_variant("attn_mfma", {"PULSE_HEAD_DIM": d})
    return bool(lib.pulse_attn_decode_takes(int(rotary_dim), int(pairing)))


def attn_decode(qkv: torch.Tensor, out: torch.Tensor, nq: int, nkv: int, d: int, kcache: torch.Tensor,
                vcache: torch.Tensor, positions: torch.Tensor, block_table: torch.Tensor,
                items: Optional[torch.Tensor],
                scale: float, window: int, split_size: int, n_splits: int, max_context: int,
                part_o: Optional[torch.Tensor], part_ml: Optional[torch.Tensor], q_w: Optional[torch.Tensor],
                k_w: Optional[torch.Tensor], eps: float, cos: Optional[torch.Tensor], sin: Optional[torch.Tensor],
                rotary_dim: int, pairing: int, new_key: bool, live_context: Optional[torch.Tensor] = None,
                plan: Optional[torch.Tensor] = None) -> None:
    """Attention for decoded tokens from the raw projection output ``qkv`` [tokens, (nq + 2 nkv) d]: per-head norm
    and rotation of q and of the token's own key happen inside the kernel; with ``new_key`` key and value are also
    written to the token's page.  Every item must hold one token; ``items`` None says that item i is token i with row
    i of the block table (a step of decoded tokens in the order of its requests), which spares every workgroup the
    trip to memory for its item.  ``live_context``, ``plan``: as for ``attn_mfma``."""
    _gpu("attn_decode", qkv, out, kcache, vcache, positions, block_table, items, part_o, part_ml, q_w, k_w, cos, sin,
         live_context, plan)
    _live(live_context)
    tokens = qkv.shape[0]
    _planned(plan, tokens, n_splits)
    _need(qkv.dtype == torch.bfloat16 and out.dtype == torch.bfloat16 and qkv.stride(1) == 1 and out.stride(1) == 1,
          "attn_decode: qkv and out must be bfloat16 matrices with contiguous rows")
    _need(qkv.shape[1] >= (nq + (2 * nkv if new_key else 0)) * d and out.shape[1] >= nq * d and out.shape[0] == tokens,
          "attn_decode: qkv/out too narrow")
    pages, page_size = _check_cache("attn_decode", kcache, vcache, nkv, d)
    _need(supported(d, page_size, qkv.dtype, kcache.dtype), f"attn_decode: head size {d} / page size {page_size} / "
          f"{kcache.dtype} is not supported by the matrix-core kernel")
    _int_vec("attn_decode: positions", positions, tokens)
    _need(block_table.dim() == 2 and block_table.dtype == torch.int32 and block_table.is_contiguous(),
          "attn_decode: block_table must be contiguous int32 [entries, width]")
    _need(items is None or (items.dtype == torch.int32 and items.is_contiguous() and items.numel() == ITEM_INTS * tokens),
          "attn_decode: one int32 quadruple for every token")
    _need(items is not None or block_table.shape[0] >= tokens, "attn_decode: without items every token needs its row "
          "of the block table")
    for name, w in (("q_w", q_w), ("k_w", k_w)):
        _need(w is None or (w.dtype == torch.bfloat16 and w.numel() == d and w.is_contiguous()),
              f"attn_decode: {name} must hold {d} bfloat16 values")
    _need((cos is None) == (sin is None), "attn_decode: cos and sin come together")
    if cos is not None:
        half = rotary_dim // 2
        for name, t in (("cos", cos), ("sin", sin)):
            _need(t.dtype == torch.float32 and t.is_contiguous() and t.dim() == 2 and t.shape[0] >= tokens
                  and t.shape[1] == half, f"attn_decode: {name} must be float32 [tokens, {half}]")
    if n_splits > 1:
        need = tokens * nq * n_splits
        _need(part_o is not None and part_ml is not None and part_o.dtype == torch.float32
              and part_ml.dtype == torch.float32 and part_o.numel() >= need * d and part_ml.numel() >= need * 2,
              "attn_decode: scratch for the split results is too small")
    lib = load_variant("attn_mfma", {"PULSE_HEAD_DIM": d})
    call_in(lib, "pulse_attn_decode", _ptr(qkv), _i64(qkv.stride(0)), _ptr(out), _i64(out.stride(0)), _ptr(kcache),
            _ptr(vcache), _ptr(positions), _ptr(block_table), _i32(block_table.shape[1]), _ptr(items), _i32(tokens),
            _i32(tokens), _i32(nq), _i32(nkv), _i32(page_size), _i32(pages), _f32(scale), _i32(window),
            _i32(split_size), _i32(n_splits), _i32(max_context), _ptr(part_o), _ptr(part_ml), _ptr(q_w), _ptr(k_w),
            _f32(eps), _ptr(cos), _ptr(sin), _i32(rotary_dim if cos is not None else 0), _i32(pairing),
            _i32(1 if new_key else 0), _ptr(live_context), _ptr(plan), _stream())
