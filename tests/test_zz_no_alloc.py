"""rocml_argmax_static, the entry point that allocates nothing, called through ctypes as a caller
without this package would: two calls in a row on one stream, the second with a smaller input,
each checked against rocml_argmax with a workspace of the caller's."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


def _library():
    from rocml_amd.csrc import build
    lib = ctypes.CDLL(build.ensure("sampling"))
    lib.rocml_argmax_static.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p]
    lib.rocml_argmax_static.restype = ctypes.c_int
    lib.rocml_argmax.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p]
    lib.rocml_argmax.restype = ctypes.c_int
    lib.sampling_last_error.restype = ctypes.c_char_p
    return lib


def test_argmax_without_allocation_matches_argmax_with_a_workspace():
    lib = _library()
    torch.cuda.set_device(0)
    stream = torch.cuda.current_stream().cuda_stream
    g = torch.Generator(device="cuda:0")
    g.manual_seed(7)
    for batch, vocab in ((64, 151936), (5, 5000)):            # the second call is smaller: stale partial results lie behind it
        logits = torch.randn(batch, vocab, generator=g, device="cuda:0")
        logits[batch // 2, vocab - 1] = 50.0                   # a maximum in the last chunk
        logits[0, 3] = logits[0, 3000] = 60.0                  # a tie: the first index wins
        work = torch.empty(batch * 64, dtype=torch.int32, device="cuda:0")
        want = torch.full((batch,), -1, dtype=torch.int32, device="cuda:0")
        got = torch.full((batch,), -2, dtype=torch.int32, device="cuda:0")
        assert lib.rocml_argmax(logits.data_ptr(), batch, vocab, want.data_ptr(), work.data_ptr(), stream) == 0
        before = torch.cuda.memory_allocated(0)
        rc = lib.rocml_argmax_static(logits.data_ptr(), batch, vocab, got.data_ptr(), stream)
        assert rc == 0, lib.sampling_last_error().decode()
        assert torch.cuda.memory_allocated(0) == before
        torch.cuda.synchronize()
        assert torch.equal(got, want)
        assert torch.equal(got.long().cpu(), logits.argmax(dim=-1).cpu())
        assert int(got[0]) == 3 and int(got[batch // 2]) == vocab - 1
    # more rows than the library's array holds: refused with a message, nothing launched
    too_many = 1025
    logits = torch.zeros(too_many, 8, device="cuda:0")
    out = torch.full((too_many,), -7, dtype=torch.int32, device="cuda:0")
    assert lib.rocml_argmax_static(logits.data_ptr(), too_many, 8, out.data_ptr(), stream) != 0
    assert b"1024" in lib.sampling_last_error()
    torch.cuda.synchronize()
    assert bool((out == -7).all())
