"""The argmax entry point that allocates nothing (``pyre_argmax_static``), called through
ctypes as a caller outside Python would: two calls in a row, the second with fewer rows and
a narrower vocabulary, each against ``pyre_argmax`` with scratch of the caller's own."""

from __future__ import annotations

import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu

MAX_ROWS = 256


def _library():
    from pyre_amd.hip import build

    lib = ctypes.CDLL(str(build.ensure_built()))
    P, I, L = ctypes.c_void_p, ctypes.c_int, ctypes.c_long
    lib.pyre_argmax_static.argtypes = [P, L, P, I, I, P]
    lib.pyre_argmax_static.restype = I
    lib.pyre_argmax_static_init.argtypes = []
    lib.pyre_argmax_static_init.restype = I
    lib.pyre_argmax.argtypes = [P, L, P, P, I, I, P]
    lib.pyre_argmax.restype = I
    lib.pyre_last_error.restype = ctypes.c_char_p
    return lib


def _both(lib, logits):
    m, vocab = logits.shape
    stream = torch.cuda.current_stream().cuda_stream
    got = torch.full((m,), -7, dtype=torch.int32, device=logits.device)
    want = torch.full((m,), -9, dtype=torch.int32, device=logits.device)
    own = torch.empty(m * 128, dtype=torch.int32, device=logits.device)
    rc = lib.pyre_argmax_static(logits.data_ptr(), logits.stride(0), got.data_ptr(), m, vocab, stream)
    assert rc == 0, lib.pyre_last_error().decode()
    rc = lib.pyre_argmax(logits.data_ptr(), logits.stride(0), want.data_ptr(), own.data_ptr(), m, vocab, stream)
    assert rc == 0, lib.pyre_last_error().decode()
    torch.cuda.synchronize()
    return got.cpu(), want.cpu()


def test_argmax_static_twice_then_too_many_rows():
    lib = _library()
    with torch.cuda.device(0):
        gen = torch.Generator(device="cuda:0").manual_seed(11)
        first = torch.randn(37, 15013, device="cuda:0", generator=gen)
        first[5, 15012] = 9.0     # the last element of the last slice
        first[6, 0] = 9.0
        first[7, 4000] = first[7, 9000] = 9.5   # equal values: the lower index
        second = torch.randn(3, 1000, device="cuda:0", generator=gen)   # smaller: stale slices stay behind it
        for logits in (first, second):
            got, want = _both(lib, logits)
            assert torch.equal(got, want)
            assert torch.equal(got.long(), logits.argmax(dim=1).cpu())
        assert int(got[0]) == int(second[0].argmax())
        # beyond the built-in scratch: refused with a message, nothing launched
        big = torch.zeros(MAX_ROWS + 1, 8, device="cuda:0")
        out = torch.zeros(MAX_ROWS + 1, dtype=torch.int32, device="cuda:0")
        rc = lib.pyre_argmax_static(big.data_ptr(), big.stride(0), out.data_ptr(), MAX_ROWS + 1, 8,
                                    torch.cuda.current_stream().cuda_stream)
        assert rc != 0 and b"256" in lib.pyre_last_error()
        full = torch.randn(MAX_ROWS, 515, device="cuda:0", generator=gen)
        got, want = _both(lib, full)
        assert torch.equal(got, want)


def test_argmax_static_in_a_captured_graph():
    """The caller that cannot allocate: the entry point under HIP graph capture. The scratch's
    address is looked up beforehand (``pyre_argmax_static_init``; a lookup during capture is not
    allowed); the graph is replayed several times on new logits, with eager work and
    synchronisations of the program's own in between, every replay against torch's argmax."""
    lib = _library()
    with torch.cuda.device(0):
        assert lib.pyre_argmax_static_init() == 0, lib.pyre_last_error().decode()
        assert lib.pyre_argmax_static_init() == 0                  # any number of times
        gen = torch.Generator(device="cuda:0").manual_seed(12)
        logits = torch.randn(9, 4099, device="cuda:0", generator=gen)
        out = torch.full((9,), -1, dtype=torch.int32, device="cuda:0")
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            rc = lib.pyre_argmax_static(logits.data_ptr(), logits.stride(0), out.data_ptr(), 9, 4099,
                                        torch.cuda.current_stream().cuda_stream)
        assert rc == 0, lib.pyre_last_error().decode()
        for k in range(4):
            logits.copy_(torch.randn(9, 4099, device="cuda:0", generator=gen))
            logits[k, 4098 - k] = 11.0
            want = logits.argmax(dim=1).cpu()                       # eager work and a synchronisation between replays
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(out.cpu().long(), want), k
            assert int(out[k]) == 4098 - k
