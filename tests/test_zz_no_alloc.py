"""The greedy choice that allocates nothing (``ms_argmax_rows_static``), called
through ctypes as a caller outside the package would, against the entry point
whose partial results the caller allocates (``ms_argmax_rows``)."""

from __future__ import annotations

import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


def _library() -> ctypes.CDLL:
    from miniserve_amd.ops import build

    path = build.find_built_library()
    assert path is not None, "the HIP library is not built"
    lib = ctypes.CDLL(str(path))
    pointer, integer = ctypes.c_void_p, ctypes.c_int
    lib.ms_last_error.restype = ctypes.c_char_p
    lib.ms_argmax_rows.restype = integer
    lib.ms_argmax_rows.argtypes = [pointer, pointer, pointer, pointer, integer, integer, integer, pointer]
    lib.ms_argmax_rows_static.restype = integer
    lib.ms_argmax_rows_static.argtypes = [pointer, pointer, integer, integer, pointer]
    return lib


def _both(lib: ctypes.CDLL, logits: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """Tokens of the existing entry point and of the one without allocations."""

    rows, vocab = logits.shape
    stream = torch.cuda.current_stream().cuda_stream
    chunks = min(64, vocab)
    chunk_max = torch.empty((rows, chunks), dtype=torch.float32, device=logits.device)
    chunk_index = torch.empty((rows, chunks), dtype=torch.int32, device=logits.device)
    want = torch.full((rows,), -7, dtype=torch.int32, device=logits.device)
    got = torch.full((rows,), -9, dtype=torch.int32, device=logits.device)
    status = lib.ms_argmax_rows(logits.data_ptr(), chunk_max.data_ptr(), chunk_index.data_ptr(), want.data_ptr(),
                                rows, vocab, chunks, stream)
    assert status == 0, lib.ms_last_error()
    status = lib.ms_argmax_rows_static(logits.data_ptr(), got.data_ptr(), rows, vocab, stream)
    assert status == 0, lib.ms_last_error()
    torch.cuda.synchronize()
    return want.cpu(), got.cpu()


def test_two_calls_in_a_row_the_second_smaller_agree_with_the_allocating_entry_point():
    lib = _library()
    generator = torch.Generator().manual_seed(5)
    large = torch.randn((200, 151_936), generator=generator).cuda()
    large[3, 77] = float("inf")               # a row with a non-finite value gives -1
    large[9, 150_000] = 50.0
    large[10, 0] = 50.0
    want, got = _both(lib, large)
    assert torch.equal(want, got)
    assert got[3] == -1 and got[9] == 150_000 and got[10] == 0
    assert torch.equal(got[[0, 1, 2]].long(), large[:3].argmax(dim=1).cpu())
    # the array still holds the first call's partial results: a smaller call must not see them
    small = torch.randn((5, 1000), generator=generator).cuda()
    small[4, 999] = 9.0
    want, got = _both(lib, small)
    assert torch.equal(want, got)
    assert torch.equal(got.long(), small.argmax(dim=1).cpu())
    # fewer tokens than chunks
    tiny = torch.randn((3, 37), generator=generator).cuda()
    want, got = _both(lib, tiny)
    assert torch.equal(want, got) and torch.equal(got.long(), tiny.argmax(dim=1).cpu())


def test_sizes_beyond_the_static_scratch_are_refused():
    lib = _library()
    logits = torch.zeros((1025, 64), dtype=torch.float32, device="cuda")
    out = torch.full((1025,), -9, dtype=torch.int32, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    assert lib.ms_argmax_rows_static(logits.data_ptr(), out.data_ptr(), 1025, 64, stream) != 0
    assert b"1..1024" in lib.ms_last_error()
    assert lib.ms_argmax_rows_static(logits.data_ptr(), out.data_ptr(), 0, 64, stream) != 0
    assert lib.ms_argmax_rows_static(None, out.data_ptr(), 4, 64, stream) != 0
    torch.cuda.synchronize()
    assert bool((out == -9).all())           # nothing ran
    assert lib.ms_argmax_rows_static(logits.data_ptr(), out.data_ptr(), 1024, 64, stream) == 0
    torch.cuda.synchronize()
    assert bool((out[:1024] == 0).all())     # equal values: the lowest index
