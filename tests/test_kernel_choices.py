"""Decisions the host takes for the kernels (no GPU needed): what must hold of every choice, whatever the
numbers the cost rules currently prefer, and for another count of compute units than the MI355X's."""
import itertools

import pytest


class E:
    def __init__(self, start, count):
        self.start, self.count = start, count


@pytest.fixture(params=[256, 304, 64])
def units(request, monkeypatch):
    from pulse_infer_amd.ops import device

    monkeypatch.setattr(device, "_units", request.param)
    assert device.compute_units() == request.param
    return request.param


def test_decode_splits_cover_the_context_in_whole_blocks(units):
    from pulse_infer_amd.ops import attention_mfma as M

    for items, nkv, group, context in itertools.product((1, 2, 8, 24, 64, 200), (1, 8), (1, 4, 20),
                                                        (1, 31, 500, 1024, 4096, 40000)):
        size, n = M.choose_splits(items, nkv, group, context)
        assert n >= 1 and size % M.BLOCK_KEYS == 0 and size > 0
        assert size * n >= context and size * (n - 1) < max(context, 1)          # every key once, no empty last split
        assert n <= 2 * M.MAX_CHOSEN_SPLITS
        if n > 1:
            assert size >= M.MIN_SPLIT_KEYS                                      # a split is worth its workgroup
    # more work than the chip has units is never cut finer than one split a unit would need
    size, n = M.choose_splits(4 * units, 8, 4, 2048)
    assert n == 1


def test_a_plan_for_uneven_contexts_has_room_for_every_pair(units):
    from pulse_infer_amd.ops import attention_mfma as M

    for nkv, group in ((8, 4), (1, 6), (2, 20), (16, 1)):
        slots, first = M.plan_slots(nkv, group)
        heads = nkv * ((group + 15) // 16)
        assert first >= 1 and slots == 2 * first and first * heads <= max(units, heads)   # one round fills the units once
    for items, splits in ((1, 8), (64, 8), (128, 8), (200, 5), (1024, 1)):
        assert M.plan_fits(items, splits)
        assert M.plan_ints(items, splits) == 1 + items * splits + items                    # count, pairs, split sizes
    assert not M.plan_fits(129, 8) and not M.plan_fits(0, 8)


def test_a_step_counts_as_uneven_by_its_longest_context_over_the_mean():
    from pulse_infer_amd.parts.base import UNEVEN_CONTEXTS, EntryMeta, contexts_uneven

    def metas(contexts):
        return [EntryMeta(i, i, c - 1, 1, i) for i, c in enumerate(contexts)]

    assert not contexts_uneven(metas([4096] * 8))
    assert not contexts_uneven(metas([9000, 10]))                     # two requests: nothing to order
    assert contexts_uneven(metas([4096, 200, 200, 200]))
    assert contexts_uneven(metas([1500, 1000, 500]))                  # exactly 1.5 times the mean
    assert not contexts_uneven(metas([1499, 1000, 500]))
    assert UNEVEN_CONTEXTS == 1.5
    # portions count with what they bring: a context is start + count
    assert contexts_uneven([EntryMeta(0, 0, 0, 900, 0), EntryMeta(1, 1, 99, 1, 900), EntryMeta(2, 2, 49, 1, 901)])


def test_prefill_splits_are_chosen_for_long_walks(units):
    from pulse_infer_amd.ops import attention_mfma as M

    choose = lambda entries, **kw: M.choose_prefill_splits(list(enumerate(entries)), 32, 8, 4, 128, kw.get("window", 0))
    assert choose([E(0, 128)]) == (0, 1)                      # short walks: nothing to gain
    assert choose([E(0, 2048)], window=256) == (0, 1)         # a window keeps them short
    assert M.choose_prefill_splits([(0, E(0, 4096))], 16, 8, 4, 96, 0) == (0, 1)     # no split variant for this head size
    for entries in ([E(16384 - 512, 512)], [E(4032, 64)], [E(0, 2048)], [E(0, 8192)], [E(100, 700), E(3000, 40)],
                    [E(39000, 1000)]):
        size, n = choose(entries)
        longest = max(e.start + e.count for e in entries)
        tokens = sum(e.count for e in entries)
        if n == 1:
            assert size == 0
            continue
        assert size % M.PREFILL_SPLIT_KEYS == 0 and size >= 8 * M.PREFILL_SPLIT_KEYS
        assert size * n >= longest and size * (n - 1) < longest + M.PREFILL_SPLIT_KEYS
        assert n <= M.PREFILL_MAX_SPLITS and tokens * 8 * 4 * 128 * 4 * n <= M.PREFILL_SCRATCH_BYTES
    assert choose([E(16384 - 64, 64)])[1] > 1                 # few items over a long context are cut
    # a full chip: only the tail of a long whole prompt is cut, at three quarters of its longest walk
    if 2048 // 32 * 8 >= 2 * units:
        assert choose([E(0, 2048)]) == (0, 1)
        assert choose([E(0, 8192)]) == (6144, 2)
        assert choose([E(0, 4096), E(0, 8192)]) == (6144, 2)
        assert choose([E(8192 - 512, 512)] * 8) == (0, 1)     # every item walks as far: nothing to gain


def test_library_products_share_out_a_wide_inner_dimension(units):
    import torch
    from pulse_infer_amd.parts.linear import Linear

    rows = lambda m, k: torch.empty(m, k, dtype=torch.bfloat16)
    for n, k in ((5120, 17408), (4096, 12288), (5120, 25600), (5120, 5120), (96, 8192)):
        lin = Linear(torch.empty(n, k, dtype=torch.bfloat16), "bfloat16")
        for m in (100, 192, 272, 544, 2048):
            shares = lin.library_shares_for(rows(m, k))
            assert shares in (0, 2, 4)
            if shares:
                assert m > Linear.SHARES_ROWS[1] and k >= Linear.LIBRARY_SHARES_MIN_K
                assert k % shares == 0 and (k // shares) % 64 == 0
    down = Linear(torch.empty(5120, 17408, dtype=torch.bfloat16), "bfloat16")
    assert down.library_shares_for(rows(272, 17408)) >= down.library_shares_for(rows(2048, 17408))   # fewer tiles, more shares
    assert Linear(torch.empty(64, 8192), "float32").library_shares_for(torch.empty(300, 8192)) == 0


def test_own_products_share_out_their_inner_dimension_evenly(units):
    import torch
    from pulse_infer_amd.parts.linear import Linear

    shape = lambda n, k: Linear(torch.empty(n, k, dtype=torch.bfloat16, device="meta"), "bfloat16")
    for n, k in ((4096, 12288), (4096, 4096), (5120, 17408), (5120, 25600), (96, 224), (1000, 384)):
        lin = shape(n, k)
        for m in (1, 12, 13, 64, 192, 193):
            x = torch.empty(m, k, dtype=torch.bfloat16)
            shares, waves = lin.shares_and_waves_for(x)
            if not Linear.SHARES_ROWS[0] <= m <= Linear.SHARES_ROWS[1] or n % 4:
                assert (shares, waves) == (0, 0)
            elif shares:
                assert k % shares == 0 and (k // shares) % 128 == 0 and waves in (4, 6) and 1 <= shares <= 16
    for n, k in ((24576, 4096), (34816, 5120), (51200, 5120), (448, 96), (12288, 2048)):
        lin = shape(n, k)
        for m in (17, 32, 64):
            waves = lin.swiglu_waves_for(m)
            assert waves in (0, 2, 4, 6, 10)
            if waves and n > 64 * units:
                # chosen only where no compute unit gets much more than its share of the weight rows
                groups = -(-n // (16 * waves))
                fullest = -(-groups // units) * 16 * waves
                assert fullest * units < 1.5 * n + 1.5 * units * (m // 2)
