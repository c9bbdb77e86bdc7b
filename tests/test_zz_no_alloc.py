"""The argmax entry point that allocates nothing, called through ctypes as a caller without torch's
allocator would: its output must equal that of the entry point whose scratch buffers the caller
brings, on two calls in a row, the second smaller than the first (the fixed buffer keeps the first
call's contents)."""

from __future__ import annotations

import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu

MAX_ROWS = 1024  # LLMSERVE_ARGMAX_STATIC_MAX_ROWS
TOO_LARGE = 1002  # LLMSERVE_ERR_TOO_LARGE


def _library() -> ctypes.CDLL:
    from llmserve_amd.kernels.build import build_module

    library = ctypes.CDLL(str(build_module("sampling")))
    pointer, integer = ctypes.c_void_p, ctypes.c_int
    library.llmserve_argmax_static.argtypes = [pointer, pointer, integer, integer, pointer]
    library.llmserve_argmax_static.restype = integer
    library.llmserve_argmax.argtypes = [pointer, pointer, pointer, pointer, integer, integer, pointer]
    library.llmserve_argmax.restype = integer
    return library


def _with_buffers(library, logits: torch.Tensor) -> torch.Tensor:
    rows, vocab = logits.shape
    values = torch.empty(rows * 64, dtype=torch.float32, device="cuda")
    indices = torch.empty(rows * 64, dtype=torch.int32, device="cuda")
    out = torch.full((rows,), -1, dtype=torch.int32, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    assert library.llmserve_argmax(logits.data_ptr(), values.data_ptr(), indices.data_ptr(), out.data_ptr(), rows, vocab, stream) == 0
    torch.cuda.synchronize()
    return out.cpu()


def test_argmax_without_allocation_equals_argmax_with_buffers():
    library = _library()
    generator = torch.Generator().manual_seed(5)
    stream = torch.cuda.current_stream().cuda_stream
    for rows, vocab in [(37, 151936), (5, 1031)]:  # the second call is smaller: stale pieces must not be read
        logits = torch.randn(rows, vocab, generator=generator)
        logits[:, vocab // 3] = logits.max(dim=1).values  # a tie: the first maximum wins
        logits = logits.cuda()
        out = torch.full((rows,), -1, dtype=torch.int32, device="cuda")
        torch.cuda.synchronize()
        before = torch.cuda.memory_stats()["allocation.all.allocated"]
        status = library.llmserve_argmax_static(logits.data_ptr(), out.data_ptr(), rows, vocab, stream)
        assert status == 0
        assert torch.cuda.memory_stats()["allocation.all.allocated"] == before
        torch.cuda.synchronize()
        expected = _with_buffers(library, logits)
        assert torch.equal(out.cpu(), expected)
        assert torch.equal(out.cpu().long(), logits.cpu().argmax(dim=1))


def test_argmax_without_allocation_refuses_more_rows_than_its_buffer_holds():
    library = _library()
    logits = torch.zeros(2, 8, device="cuda")
    out = torch.full((2,), -7, dtype=torch.int32, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    assert library.llmserve_argmax_static(logits.data_ptr(), out.data_ptr(), MAX_ROWS + 1, 8, stream) == TOO_LARGE
    assert library.llmserve_argmax_static(logits.data_ptr(), out.data_ptr(), 2, 0, stream) == 1001
    torch.cuda.synchronize()
    assert out.tolist() == [-7, -7]  # nothing ran
    full = torch.randn(MAX_ROWS, 40, device="cuda")
    most = torch.empty(MAX_ROWS, dtype=torch.int32, device="cuda")
    assert library.llmserve_argmax_static(full.data_ptr(), most.data_ptr(), MAX_ROWS, 40, stream) == 0
    torch.cuda.synchronize()
    assert torch.equal(most.cpu().long(), full.cpu().argmax(dim=1))
