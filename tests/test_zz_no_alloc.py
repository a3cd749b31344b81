"""The entry point that allocates nothing (`ta_argmax_static`, csrc/no_alloc.h), called through ctypes as a
caller outside Python would, against the existing `ta_argmax` with a workspace of the caller's."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


def _library():
    from tokenizer_amd.kernels import build
    path = build.find_library()
    assert path is not None, "the kernel library is not built"
    lib = ctypes.CDLL(path)
    lib.ta_argmax.restype = ctypes.c_int
    lib.ta_argmax.argtypes = [ctypes.c_void_p] * 4 + [ctypes.c_int] * 3 + [ctypes.c_void_p]
    lib.ta_argmax_static.restype = ctypes.c_int
    lib.ta_argmax_static.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_void_p]
    return lib


def _with_workspace(lib, logits, stream):
    n_rows, vocab = logits.shape
    chunks = max(1, min(256, vocab // 2048, 2048 // max(1, n_rows)))
    partial_v = torch.empty((n_rows, chunks), dtype=torch.float32, device=logits.device)
    partial_i = torch.empty((n_rows, chunks), dtype=torch.int32, device=logits.device)
    out = torch.full((n_rows,), -7, dtype=torch.int32, device=logits.device)
    assert lib.ta_argmax(logits.data_ptr(), out.data_ptr(), partial_v.data_ptr(), partial_i.data_ptr(), n_rows, vocab,
                         chunks, stream) == 0
    return out


def test_the_pick_that_allocates_nothing_equals_the_one_with_a_workspace():
    lib = _library()
    device = torch.device("cuda:0")
    stream = torch.cuda.current_stream(device).cuda_stream
    gen = torch.Generator(device="cpu").manual_seed(5)
    # Two calls in a row on the same array, the second smaller in both sizes (fewer and shorter pieces: what
    # the first call left behind lies beyond and between them); then a third with other sizes again.
    for n_rows, vocab in ((64, 151936), (5, 9001), (1, 1000), (300, 4097)):
        logits = torch.randn((n_rows, vocab), generator=gen, dtype=torch.float32).to(device)
        logits[0, vocab // 3] = logits[0, vocab - 1] = 50.0          # two equal maxima: the first one wins
        if n_rows > 2:
            logits[2] = 0.0                                          # all equal: index 0
        want = _with_workspace(lib, logits, stream)
        got = torch.full((n_rows,), -9, dtype=torch.int32, device=device)
        held = torch.cuda.memory_allocated(device)
        assert lib.ta_argmax_static(logits.data_ptr(), got.data_ptr(), n_rows, vocab, stream) == 0
        assert torch.cuda.memory_allocated(device) == held
        torch.cuda.synchronize(device)
        assert torch.equal(got, want), (n_rows, vocab)
        # Independently of the other entry point: every row against the library routine, but for the row of all
        # ties (the first index) and the row with two planted maxima (the first of them).
        expected = logits.cpu().argmax(dim=1)
        expected[0] = vocab // 3
        if n_rows > 2:
            expected[2] = 0
        assert torch.equal(got.cpu().long(), expected), (n_rows, vocab)
    # Sizes beyond the array are refused before anything is launched.
    too_many = 4097
    logits = torch.zeros((too_many, 8), dtype=torch.float32, device=device)
    got = torch.full((too_many,), -9, dtype=torch.int32, device=device)
    assert lib.ta_argmax_static(logits.data_ptr(), got.data_ptr(), too_many, 8, stream) == -2
    assert lib.ta_argmax_static(logits.data_ptr(), got.data_ptr(), 4, 0, stream) == -1
    torch.cuda.synchronize(device)
    assert int(got.min()) == -9 and int(got.max()) == -9
    assert lib.ta_argmax_static(logits.data_ptr(), got.data_ptr(), 4096, 8, stream) == 0
    torch.cuda.synchronize(device)
    assert int(got[:4096].abs().max()) == 0 and int(got[4096]) == -9
