"""The entry point that allocates nothing (csrc/no_alloc.h), called through ctypes and
held against the existing greedy choice, twice in a row on one stream, the second time
with a smaller input: what the first call left in the library's own array must not
reach the second call's result."""

import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu

MAX_PARTIALS = 65536


def entry():
    from zig_ai_amd.kernels import build
    lib = build.load("sampling")
    fn = lib.za_argmax_no_alloc
    fn.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_int,
                   ctypes.c_void_p]
    fn.restype = ctypes.c_int
    why = lib.za_no_alloc_last_error
    why.argtypes = []
    why.restype = ctypes.c_char_p
    return fn, why


def logits_for(rows, vocab, seed):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn((rows, vocab), generator=g)
    # the maximum sits in another chunk for every row, once tied with a later entry
    for r in range(rows):
        at = (r * 7919 + 13) % vocab
        x[r, at] = 9.0
        if r % 3 == 0 and at + 5 < vocab:
            x[r, at + 5] = 9.0
    return x


def test_two_calls_in_a_row_the_second_smaller():
    from zig_ai_amd.kernels import ops
    fn, why = entry()
    dev = torch.device("cuda", 0)
    stream = torch.cuda.current_stream().cuda_stream
    # the set-up (the array's address on this device, asked of the runtime once) is not
    # part of what is measured below: whatever the runtime does for it happens here
    warm = torch.zeros((2, 128), device=dev)
    warm_out = torch.empty((2,), dtype=torch.int32, device=dev)
    assert fn(warm.data_ptr(), 2, 128, warm_out.data_ptr(), 2, stream) == 0, why()
    torch.cuda.synchronize()
    for (rows, vocab, chunks), (rows2, vocab2, chunks2) in (
            ((8, 65536, 16), (3, 10001, 4)), ((64, 4099, 8), (1, 301, 2)), ((5, 70000, 64), (5, 640, 1))):
        first = logits_for(rows, vocab, 1).to(dev)
        second = logits_for(rows2, vocab2, 2).to(dev)
        out1 = torch.full((rows,), -7, dtype=torch.int32, device=dev)
        out2 = torch.full((rows2,), -7, dtype=torch.int32, device=dev)
        want1, want2 = ops.argmax(first), ops.argmax(second)
        torch.cuda.synchronize()
        before = torch.cuda.memory_stats(dev)["allocation.all.allocated"]
        free_before = torch.cuda.mem_get_info(dev)[0]
        rc1 = fn(first.data_ptr(), rows, vocab, out1.data_ptr(), chunks, stream)
        rc2 = fn(second.data_ptr(), rows2, vocab2, out2.data_ptr(), chunks2, stream)
        after = torch.cuda.memory_stats(dev)["allocation.all.allocated"]
        free_after = torch.cuda.mem_get_info(dev)[0]
        assert rc1 == 0 and rc2 == 0, why()
        assert before == after                   # (the tensor library was not asked either)
        # and the device's free memory is what it was: no hipMalloc or hipFree of the
        # entry point's own (the array is part of the library's image)
        assert free_before == free_after
        torch.cuda.synchronize()
        assert torch.equal(out1, want1) and torch.equal(out2, want2)
        assert torch.equal(out1.cpu().long(), first.cpu().argmax(dim=1))
        assert torch.equal(out2.cpu().long(), second.cpu().argmax(dim=1))


def test_sizes_beyond_the_array_are_refused():
    fn, why = entry()
    dev = torch.device("cuda", 0)
    x = torch.zeros((4, 64), device=dev)
    out = torch.full((4,), -7, dtype=torch.int32, device=dev)
    stream = torch.cuda.current_stream().cuda_stream
    assert fn(x.data_ptr(), MAX_PARTIALS // 16 + 1, 64, out.data_ptr(), 16, stream) == -2
    assert b"partial results" in why()
    assert fn(x.data_ptr(), 4, 64, out.data_ptr(), 0, stream) == -1 and b"bad argument" in why()
    assert fn(None, 4, 64, out.data_ptr(), 2, stream) == -1
    torch.cuda.synchronize()
    assert torch.equal(out.cpu(), torch.full((4,), -7, dtype=torch.int32))   # nothing ran
    # exactly the maximum is taken
    rows = MAX_PARTIALS // 64
    big = logits_for(rows, 2048, 3).to(dev)
    got = torch.empty((rows,), dtype=torch.int32, device=dev)
    assert fn(big.data_ptr(), rows, 2048, got.data_ptr(), 64, stream) == 0, why()
    torch.cuda.synchronize()
    assert torch.equal(got.cpu().long(), big.cpu().argmax(dim=1))
