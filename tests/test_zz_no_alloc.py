"""The arg max that allocates nothing (`ia_argmax_static`), called through ctypes as a caller without torch's
allocator would call it, against the entry point that takes a workspace: two calls in a row on the library's one
scratch array, the second smaller than the first, and the sizes it refuses."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


def test_argmax_static_equals_argmax_with_a_workspace():
    from inferrs_amd import ops
    lib = ops.library()
    lib.ia_argmax_static_capacity.restype = ctypes.c_longlong
    capacity = lib.ia_argmax_static_capacity()
    assert capacity == 16384
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    gen = torch.Generator().manual_seed(5)

    def both(rows, vocab, plant):
        logits = torch.randn(rows, vocab, generator=gen).to("cuda:0")
        for r, c in plant:                                   # equal maxima in different stretches: the lowest index wins
            logits[r, c] = 50.0
        want = ops.argmax(logits)                            # the existing entry point, workspace from torch
        got = torch.full((rows,), -7, dtype=torch.int32, device="cuda:0")
        torch.cuda.synchronize()
        before = torch.cuda.memory_allocated()
        rc = lib.ia_argmax_static(ctypes.c_void_p(got.data_ptr()), ctypes.c_void_p(logits.data_ptr()), rows, vocab, stream)
        assert rc == 0, lib.ia_last_error().decode()
        torch.cuda.synchronize()
        assert torch.cuda.memory_allocated() == before
        assert torch.equal(got, want), (rows, vocab)
        # the lowest index among a row's maxima, written out (torch's own arg max names any of them)
        top = logits.max(dim=-1, keepdim=True).values
        index = torch.arange(vocab, device=logits.device).expand(rows, vocab)
        lowest = torch.where(logits == top, index, torch.full_like(index, vocab)).min(dim=-1).values
        assert torch.equal(got.cpu().long(), lowest.cpu())
        return got

    first = both(40, 151936, [(3, 150000), (3, 9000), (7, 151935), (39, 0), (39, 100000)])
    assert first[3] == 9000 and first[7] == 151935 and first[39] == 0
    both(5, 40000, [(0, 39999), (4, 17000), (4, 33000)])     # a smaller call on the array the first one left
    both(9, 1000, [])                                        # short rows need no scratch
    # sizes beyond the array are refused, with a message, and nothing runs
    out = torch.zeros(500, dtype=torch.int32, device="cuda:0")
    big = torch.zeros(500, 151936, device="cuda:0")
    assert ops.library().ia_argmax_workspace(500, 151936) > capacity
    rc = lib.ia_argmax_static(ctypes.c_void_p(out.data_ptr()), ctypes.c_void_p(big.data_ptr()), 500, 151936, stream)
    assert rc != 0 and "words of scratch" in lib.ia_last_error().decode()
