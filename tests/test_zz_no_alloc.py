"""The entry point that allocates nothing (``pylon_argmax_static``, declared in
``pylon_amd/csrc/no_alloc.h``) against the ordinary ``pylon_argmax``, called through ctypes
as a caller without torch would: two calls in a row, the second with a smaller input, which
must not see what the first left in the library's scratch array."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


def test_argmax_without_allocation_matches_the_ordinary_entry_point():
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    from pylon_amd.kernels import library

    lib = library.load()
    static = lib.pylon_argmax_static
    static.restype = ctypes.c_int
    static.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_longlong,
                       ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p]
    ordinary = lib.pylon_argmax
    scratch_bytes = lib.pylon_argmax_scratch_bytes
    scratch_bytes.restype = ctypes.c_longlong
    scratch_bytes.argtypes = [ctypes.c_int]
    lib.pylon_argmax_static_init.restype = ctypes.c_int
    assert lib.pylon_argmax_static_init() == 0, lib.pylon_last_error()
    stream = torch.cuda.current_stream().cuda_stream
    gen = torch.Generator(device="cuda").manual_seed(11)

    def both(rows, vocab, with_table):
        logits = torch.randn((rows, vocab), generator=gen, device="cuda", dtype=torch.float32)
        logits[0, vocab - 1] = 50.0  # the last column of the last chunk
        if rows > 1:
            logits[1, 5] = logits[1, 77] = 60.0  # equal maxima: the lower index
        place = torch.randperm(rows, device="cuda").to(torch.int32)
        outs, tables = [], []
        for fn in ("static", "ordinary"):
            out = torch.full((rows,), -1, dtype=torch.int32, device="cuda")
            table = torch.full((rows,), -1, dtype=torch.int32, device="cuda")
            chosen = table.data_ptr() if with_table else None
            where = place.data_ptr() if with_table else None
            if fn == "static":
                status = static(out.data_ptr(), logits.data_ptr(), rows, vocab, logits.stride(0), chosen, where, stream)
            else:
                n = scratch_bytes(rows)
                scratch = torch.empty(n, dtype=torch.uint8, device="cuda")
                status = ordinary(out.data_ptr(), logits.data_ptr(), rows, vocab, logits.stride(0), chosen, where,
                                  scratch.data_ptr(), n, stream)
            assert status == 0, lib.pylon_last_error()
            torch.cuda.synchronize()
            outs.append(out.cpu())
            tables.append(table.cpu())
        assert torch.equal(outs[0], outs[1]) and torch.equal(tables[0], tables[1])
        assert torch.equal(outs[0].long(), logits.argmax(dim=1).cpu()) or rows > 1  # row 1 holds a tie
        assert int(outs[0][0]) == vocab - 1 and (rows == 1 or int(outs[0][1]) == 5)
        if with_table:
            assert torch.equal(tables[0][place.cpu().long()], outs[0])

    both(200, 151936, True)  # the first call fills most of the scratch array
    both(7, 3001, False)  # a smaller input right after: fewer rows, fewer chunks per row
    both(256, 1024, True)  # the most rows it takes
    # beyond the array it refuses, and says so
    logits = torch.zeros((257, 64), device="cuda")
    out = torch.zeros(257, dtype=torch.int32, device="cuda")
    assert static(out.data_ptr(), logits.data_ptr(), 257, 64, 64, None, None, stream) != 0
    assert b"at most 256 rows" in lib.pylon_last_error()
