"""The sampling entry point that allocates nothing (``tl_sample_chunks_static``: csrc/no_alloc.h),
called through ``ctypes`` and compared with ``tl_sample_chunks``, which takes its workspace from
the caller."""

import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def _both(lib, logits, temps, seeds, steps, chunks):
    """(tokens of the entry point with a workspace, tokens of the one without), same inputs."""
    n, vocab = logits.shape
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    out_ws = torch.full((n,), -1, dtype=torch.int32, device=DEV)
    out_static = torch.full((n,), -2, dtype=torch.int32, device=DEV)
    candidates = torch.empty((n, chunks, 2), dtype=torch.int32, device=DEV)
    torch.cuda.synchronize()
    rc = lib.tl_sample_chunks(
        logits.data_ptr(), logits.stride(0), n, vocab, temps.data_ptr(), seeds.data_ptr(), steps.data_ptr(), chunks,
        candidates.data_ptr(), out_ws.data_ptr(), stream,
    )
    assert rc == 0, lib.tl_last_error()
    before = torch.cuda.memory_allocated(DEV)
    rc = lib.tl_sample_chunks_static(
        logits.data_ptr(), logits.stride(0), n, vocab, temps.data_ptr(), seeds.data_ptr(), steps.data_ptr(), chunks,
        out_static.data_ptr(), stream,
    )
    assert rc == 0, lib.tl_last_error()
    assert torch.cuda.memory_allocated(DEV) == before
    torch.cuda.synchronize()
    return out_ws.cpu(), out_static.cpu()


def _inputs(rows, vocab, seed):
    g = torch.Generator().manual_seed(seed)
    logits = (torch.randn(rows, vocab, generator=g) * 3).to(DEV)
    temps = torch.tensor([0.7, 0.0, 1.3] + [0.9] * (rows - 3), dtype=torch.float32, device=DEV)[:rows].contiguous()
    seeds = torch.arange(11, 11 + rows, dtype=torch.int64, device=DEV)
    steps = torch.arange(rows, dtype=torch.int64, device=DEV)
    return logits, temps, seeds, steps


def test_static_candidates_give_the_tokens_of_the_workspace_entry_point_twice_in_a_row():
    """Two calls in a row, the second with fewer rows, fewer pieces and a smaller vocabulary: the
    array keeps the first call's candidates, and none of them may reach the second call's result."""
    from torchllms_amd.kernels.lib import core

    lib = core()
    logits, temps, seeds, steps = _inputs(8, 128256, 3)
    logits[1, 128255] = logits[1, 9000] = 40.0  # a greedy row with a tie across pieces: the lower index
    ws, static = _both(lib, logits, temps, seeds, steps, 16)
    assert ws.tolist() == static.tolist() and static[1] == 9000
    assert all(0 <= t < 128256 for t in static.tolist())

    logits2, temps2, seeds2, steps2 = _inputs(3, 40000, 4)
    ws2, static2 = _both(lib, logits2, temps2, seeds2, steps2, 4)
    assert ws2.tolist() == static2.tolist()
    assert static2[1] == int(logits2[1].argmax())
    assert all(0 <= t < 40000 for t in static2.tolist())


def test_static_candidates_refuse_what_the_array_cannot_hold():
    from torchllms_amd.kernels.lib import core

    lib = core()
    rows, vocab, chunks = 1025, 4096, 8  # 1025 * 8 candidates > 8192
    logits = torch.zeros((rows, vocab), dtype=torch.float32, device=DEV)
    temps = torch.zeros(rows, dtype=torch.float32, device=DEV)
    seeds = torch.zeros(rows, dtype=torch.int64, device=DEV)
    out = torch.full((rows,), -5, dtype=torch.int32, device=DEV)
    rc = lib.tl_sample_chunks_static(
        logits.data_ptr(), logits.stride(0), rows, vocab, temps.data_ptr(), seeds.data_ptr(), seeds.data_ptr(), chunks,
        out.data_ptr(), ctypes.c_void_p(torch.cuda.current_stream().cuda_stream),
    )
    assert rc != 0 and b"fixed array holds 8192" in lib.tl_last_error()
    torch.cuda.synchronize()
    assert (out == -5).all()  # nothing was launched
    # exactly at the limit it runs
    rows = 1024
    rc = lib.tl_sample_chunks_static(
        logits.data_ptr(), logits.stride(0), rows, vocab, temps.data_ptr(), seeds.data_ptr(), seeds.data_ptr(), chunks,
        out.data_ptr(), ctypes.c_void_p(torch.cuda.current_stream().cuda_stream),
    )
    assert rc == 0, lib.tl_last_error()
    torch.cuda.synchronize()
    assert (out[:rows] == 0).all() and out[rows] == -5  # all logits equal: the lowest index
