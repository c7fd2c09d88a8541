"""The entry point that allocates nothing (`tm_argmax_rows_static`), called the way a foreign caller
would: through ctypes, with device pointers and a stream, against the entry point it is a variant of."""
from __future__ import annotations

import ctypes
from ctypes import c_int, c_void_p

import pytest
import torch

pytestmark = pytest.mark.gpu


def _lib():
    from tokenmill_amd.hip.library import library
    lib = library()
    lib.tm_argmax_rows_static.restype = c_int
    lib.tm_argmax_rows.restype = c_int
    return lib


def _both(lib, logits):
    """(static entry point's result, allocating entry point's result) for one [R, V] tensor."""
    R, V = logits.shape
    stream = c_void_p(torch.cuda.current_stream().cuda_stream)
    nb = lib.tm_argmax_work_chunks(c_int(V))
    got = torch.full((R,), -7, dtype=torch.int32, device=logits.device)
    want = torch.full((R,), -9, dtype=torch.int32, device=logits.device)
    work_v = torch.empty(R * nb, dtype=torch.float32, device=logits.device)
    work_i = torch.empty(R * nb, dtype=torch.int32, device=logits.device)
    rc = lib.tm_argmax_rows_static(c_void_p(logits.data_ptr()), c_int(R), c_int(V), c_void_p(got.data_ptr()), stream)
    assert rc == 0, f"tm_argmax_rows_static returned {rc}"
    rc = lib.tm_argmax_rows(c_void_p(logits.data_ptr()), c_int(R), c_int(V), c_void_p(want.data_ptr()),
                            c_void_p(work_v.data_ptr()), c_void_p(work_i.data_ptr()), stream)
    assert rc == 0
    torch.cuda.synchronize()
    return got.cpu(), want.cpu()


def test_static_argmax_matches_the_allocating_one_on_two_calls_in_a_row():
    lib = _lib()
    torch.manual_seed(11)
    dev = torch.device("cuda:0")
    V = 151936
    big = torch.randn(24, V, device=dev)
    nb = lib.tm_argmax_work_chunks(c_int(V))
    chunk = -(-V // nb)                                    # entries of a chunk: 3,999 here, no power of two
    assert nb > 1 and chunk * (nb - 1) < V <= chunk * nb and chunk % 64
    big[3, V - 1] = 40.0                                   # a maximum in the last, shorter chunk
    big[5, 5 * chunk] = 41.0                               # ... at a chunk's first entry
    big[6, 9 * chunk - 1] = 41.0                           # ... at a chunk's last entry
    big[7, 100] = big[7, 90000] = 42.0                     # a tie across chunks: the lower index wins
    big[8, 3 * chunk - 1] = big[8, 3 * chunk] = 43.0       # a tie across a chunk's edge
    got, want = _both(lib, big)
    assert torch.equal(got, want) and torch.equal(got.long(), big.argmax(dim=1).cpu())
    assert got[3] == V - 1 and got[5] == 5 * chunk and got[6] == 9 * chunk - 1 and got[7] == 100
    assert got[8] == 3 * chunk - 1
    # a second call with a smaller input: fewer rows and fewer chunks; what the first call left in the
    # array beyond them must not be read
    small = torch.randn(5, 20000, device=dev)
    small[2, 19999] = 30.0
    got, want = _both(lib, small)
    assert torch.equal(got, want) and torch.equal(got.long(), small.argmax(dim=1).cpu())
    # one chunk: no scratch at all
    narrow = torch.randn(9, 307, device=dev)
    got, want = _both(lib, narrow)
    assert torch.equal(got, want) and torch.equal(got.long(), narrow.argmax(dim=1).cpu())


def test_static_argmax_refuses_more_than_the_array_holds_and_allocates_nothing():
    lib = _lib()
    dev = torch.device("cuda:0")
    most = lib.tm_argmax_rows_static_max_pairs()
    V = 151936
    nb = lib.tm_argmax_work_chunks(c_int(V))
    rows = most // nb + 1
    logits = torch.zeros((rows, V), device=dev)
    out = torch.full((rows,), -7, dtype=torch.int32, device=dev)
    stream = c_void_p(torch.cuda.current_stream().cuda_stream)
    rc = lib.tm_argmax_rows_static(c_void_p(logits.data_ptr()), c_int(rows), c_int(V), c_void_p(out.data_ptr()), stream)
    torch.cuda.synchronize()
    assert rc == 1 and bool((out == -7).all())             # refused before anything ran
    # the largest size that fits runs, and the driver's count of free memory does not move across calls
    rows -= 1
    logits = logits[:rows]
    logits[rows - 1, V - 1] = 1.0
    torch.cuda.synchronize()
    free_before, _ = torch.cuda.mem_get_info(dev)
    for _ in range(3):
        rc = lib.tm_argmax_rows_static(c_void_p(logits.data_ptr()), c_int(rows), c_int(V), c_void_p(out.data_ptr()), stream)
        assert rc == 0
    torch.cuda.synchronize()
    free_after, _ = torch.cuda.mem_get_info(dev)
    assert free_after == free_before
    assert int(out[rows - 1]) == V - 1 and int(out[0]) == 0
    from tokenmill_amd.hip import ops
    with pytest.raises(ops.KernelArgumentError, match="fixed array"):
        ops.argmax_rows_static(torch.zeros((rows + 1, V), device=dev), torch.empty(rows + 1, dtype=torch.int32, device=dev))
