"""Decisions the host takes for the kernels (no GPU needed)."""
import pytest


def test_prefill_splits_are_chosen_for_long_walks():
    from pulse_infer_amd.ops import attention_mfma as M

    class E:
        def __init__(self, start, count):
            self.start, self.count = start, count
    choose = lambda entries, **kw: M.choose_prefill_splits(list(enumerate(entries)), 32, 8, 4, 128, kw.get("window", 0))
    assert choose([E(0, 512)]) == (0, 1)                      # short walks: nothing to gain
    assert choose([E(0, 2048)], window=256) == (0, 1)         # a window keeps them short
    size, n = choose([E(16384 - 512, 512)])                   # few items over a long context
    assert n > 1 and size % 64 == 0 and size * n >= 16384 and size * (n - 1) < 16384
    size, n = choose([E(4032, 64)])
    assert n >= 4 and size >= 8 * 64
    size, n = choose([E(0, 2048)])                            # a whole prompt: its late items walk twice their share
    assert n == 2 and size > 1024 and size * n >= 2048        # cut beyond the middle: most items finish in one split
    assert M.choose_prefill_splits([(0, E(0, 4096))], 16, 8, 4, 96, 0) == (0, 1)     # no split variant for this head size


def test_library_products_share_out_a_wide_inner_dimension():
    import torch
    from pulse_infer_amd.parts.linear import Linear

    down = Linear(torch.empty(5120, 17408, dtype=torch.bfloat16), "bfloat16")        # 14B shape
    rows = lambda m, k=17408: torch.empty(m, k, dtype=torch.bfloat16)
    assert down.library_shares_for(rows(100)) == 0          # up to 192 rows the package's own product takes it
    assert down.library_shares_for(rows(272)) == 4
    assert down.library_shares_for(rows(544)) == 2
    assert down.library_shares_for(rows(2048)) == 0         # enough output tiles to fill the chip
    o = Linear(torch.empty(5120, 5120, dtype=torch.bfloat16), "bfloat16")
    assert o.library_shares_for(rows(544, 5120)) == 0       # a narrow inner dimension: nothing to gain
    f32 = Linear(torch.empty(64, 8192), "float32")
    assert f32.library_shares_for(torch.empty(300, 8192)) == 0


def test_gate_up_takes_the_workgroup_shape_that_shares_its_rows_out_evenly():
    import torch
    from pulse_infer_amd.parts.linear import Linear

    shape = lambda n, k: Linear(torch.empty(n, k, dtype=torch.bfloat16, device="meta"), "bfloat16")
    assert shape(24576, 4096).swiglu_waves_for(32) == 6       # 8B: 256 workgroups of 96 rows
    assert shape(34816, 5120).swiglu_waves_for(32) == 10      # 14B: 218 workgroups of 160 rows
    assert shape(51200, 5120).swiglu_waves_for(32) == 0       # 32B: no even share; the library's product
    assert shape(448, 96).swiglu_waves_for(20) == 2           # few rows: the most workgroups
