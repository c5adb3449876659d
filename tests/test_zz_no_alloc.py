"""The entry point of the kernel library that allocates nothing (csrc/no_alloc.h), called through
ctypes as a C caller would, against the entry point it is a variant of."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


def _lib():
    from libllm_amd.hip import build
    lib = build.load()
    vp, i = ctypes.c_void_p, ctypes.c_int
    lib.llm_argmax.argtypes = [vp, vp, vp, vp, i, i, vp]
    lib.llm_argmax_static.argtypes = [vp, vp, i, i, vp]
    lib.llm_argmax_static_max_rows.argtypes = [i]
    lib.llm_argmax_parts.argtypes = [i]
    lib.llm_argmax_static_init.argtypes = []
    for fn in (lib.llm_argmax, lib.llm_argmax_static, lib.llm_argmax_static_max_rows, lib.llm_argmax_parts,
               lib.llm_argmax_static_init):
        fn.restype = i
    return lib


def _both(lib, logits):
    """(tokens by the entry point whose caller brings the scratch arrays, tokens by the static one)."""
    rows, vocab = logits.shape
    stream = torch.cuda.current_stream().cuda_stream
    parts = lib.llm_argmax_parts(vocab)
    pv = torch.empty(rows * parts, dtype=torch.float32, device="cuda")
    pi = torch.empty(rows * parts, dtype=torch.int32, device="cuda")
    want = torch.full((rows,), -1, dtype=torch.int32, device="cuda")
    got = torch.full((rows,), -2, dtype=torch.int32, device="cuda")
    assert lib.llm_argmax(logits.data_ptr(), want.data_ptr(), pv.data_ptr(), pi.data_ptr(), rows, vocab, stream) == 0
    assert lib.llm_argmax_static(logits.data_ptr(), got.data_ptr(), rows, vocab, stream) == 0
    torch.cuda.synchronize()
    return want.cpu(), got.cpu()


def test_argmax_without_allocation_matches_the_entry_point_with_scratch_arrays():
    """Two calls in a row on one stream, the second with fewer rows and a smaller vocabulary (the
    array still holds the first call's partial results, which must not leak into the second); a
    row whose maximum lies in the last slice, ties, and the limit on the size."""
    lib = _lib()
    assert lib.llm_argmax_static_init() == 0
    g = torch.Generator().manual_seed(3)
    big = torch.randn((48, 128256), generator=g).cuda()
    big[5, 128255] = 50.0                                # the last element of the last slice
    big[6, :] = 1.0                                      # all equal: the lowest index wins
    want, got = _both(lib, big)
    assert torch.equal(want, got)
    keep = [r for r in range(48) if r != 6]
    assert torch.equal(got.long()[keep], big.cpu().argmax(dim=-1)[keep])
    assert got[5] == 128255 and got[6] == 0
    small = torch.randn((7, 5003), generator=g).cuda() - 100.0      # all below what the array holds from before
    want, got = _both(lib, small)
    assert torch.equal(want, got)
    assert torch.equal(got.long(), small.cpu().argmax(dim=-1))
    # no allocation happened inside the static call
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    out = torch.empty((48,), dtype=torch.int32, device="cuda")
    held = torch.cuda.memory_allocated()
    assert lib.llm_argmax_static(big.data_ptr(), out.data_ptr(), 48, 128256, torch.cuda.current_stream().cuda_stream) == 0
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == held and held >= before
    # beyond the array: refused with its own code, nothing launched, the output untouched
    limit = lib.llm_argmax_static_max_rows(128256)
    assert limit == 32768 // lib.llm_argmax_parts(128256)
    out.fill_(-7)
    assert lib.llm_argmax_static(big.data_ptr(), out.data_ptr(), limit + 1, 128256, torch.cuda.current_stream().cuda_stream) == 3
    torch.cuda.synchronize()
    assert (out == -7).all()
    assert lib.llm_argmax_static_max_rows(0) == 0
