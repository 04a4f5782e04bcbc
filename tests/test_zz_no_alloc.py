"""The entry point that allocates nothing (``pulse_argmax_static``), called through ctypes as a caller
that cannot allocate would call it, against ``pulse_argmax`` with a workspace: two calls in a row on the
same GPU, the second with a smaller input, so that what the first call left in the built-in array must
not show in the second; and the refusal of an input beyond the array's size."""
from __future__ import annotations

import ctypes

import pytest
import torch

from conftest import require_gpu

pytestmark = pytest.mark.gpu


def _static_argmax(lib, logits: torch.Tensor, out: torch.Tensor) -> int:
    fn = lib.pulse_argmax_static
    fn.restype = ctypes.c_int
    fn.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_int64, ctypes.c_void_p, ctypes.c_void_p]
    rows, vocab = logits.shape
    return fn(logits.data_ptr(), rows, vocab, logits.stride(0), out.data_ptr(),
              torch.cuda.current_stream().cuda_stream)


def test_static_argmax_matches_the_workspace_one_twice_in_a_row():
    require_gpu()
    from pulse_infer_amd.ops import kernels, library

    lib = library.load()
    dev = torch.device("cuda:0")
    gen = torch.Generator().manual_seed(5)
    # the second input is smaller in both directions: fewer rows and fewer chunks of the vocabulary
    for rows, vocab in ((37, 151936), (5, 4099)):
        logits = torch.randn(rows, vocab, generator=gen).to(dev)
        logits[1, 7] = logits[1, vocab - 3] = 50.0          # equal maxima: the lowest index wins
        logits[2].fill_(float("nan"))                       # nothing is a number: -1
        logits[3, vocab - 1] = 60.0                         # the winner sits in the last, partly filled chunk
        chunks = kernels.argmax_chunks(vocab)
        want = torch.full((rows,), -7, dtype=torch.int32, device=dev)
        kernels.argmax(logits, want, torch.empty(rows * chunks, device=dev),
                       torch.empty(rows * chunks, dtype=torch.int32, device=dev))
        got = torch.full((rows,), -9, dtype=torch.int32, device=dev)
        code = _static_argmax(lib, logits, got)
        assert code == 0, lib.pulse_last_error().decode()
        torch.cuda.synchronize()
        assert got.tolist() == want.tolist()
        assert got[1].item() == 7 and got[2].item() == -1 and got[3].item() == vocab - 1
        reference = torch.argmax(torch.nan_to_num(logits.cpu(), nan=-1e30), dim=1)
        keep = [r for r in range(rows) if r != 2]
        assert got.cpu()[keep].tolist() == reference[keep].tolist()


def test_static_argmax_refuses_what_does_not_fit():
    require_gpu()
    from pulse_infer_amd.ops import kernels, library

    lib = library.load()
    dev = torch.device("cuda:0")
    vocab = 2048 * 40 + 1                                    # 41 chunks
    rows = 65536 // kernels.argmax_chunks(vocab) + 1         # one row more than the array holds
    logits = torch.zeros(rows, vocab, device=dev)
    out = torch.full((rows,), -9, dtype=torch.int32, device=dev)
    assert _static_argmax(lib, logits, out) != 0
    assert "exceed" in lib.pulse_last_error().decode()
    torch.cuda.synchronize()
    assert set(out.tolist()) == {-9}                         # nothing was launched
    logits = logits[:rows - 1]
    assert _static_argmax(lib, logits, out) == 0             # what just fits is taken
    torch.cuda.synchronize()
    assert out[:rows - 1].tolist() == [0] * (rows - 1)
