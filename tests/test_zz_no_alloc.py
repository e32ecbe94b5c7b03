"""The greedy choice through the entry point that allocates nothing, called through ctypes,
against the entry point whose partial results go through buffers of the caller."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


def _library():
    from sonicboom_amd.csrc import build
    lib = ctypes.CDLL(build.ensure_core())
    P, I = ctypes.c_void_p, ctypes.c_int
    lib.sb_argmax.argtypes = [P, P, I, I, P, P, P]
    lib.sb_argmax_noalloc.argtypes = [P, P, I, I, P]
    lib.sb_argmax_parts.argtypes = [I]
    for fn in (lib.sb_argmax, lib.sb_argmax_noalloc, lib.sb_argmax_parts, lib.sb_argmax_noalloc_max_entries):
        fn.restype = I
    lib.sb_last_error.restype = ctypes.c_char_p
    return lib


def _both(lib, logits):
    n, vocab = logits.shape
    parts = lib.sb_argmax_parts(vocab)
    stream = torch.cuda.current_stream().cuda_stream
    want = torch.full((n,), -7, dtype=torch.int32, device=logits.device)
    pv = torch.empty((n * parts,), dtype=torch.float32, device=logits.device)
    pi = torch.empty((n * parts,), dtype=torch.int32, device=logits.device)
    assert lib.sb_argmax(want.data_ptr(), logits.data_ptr(), n, vocab, pv.data_ptr(), pi.data_ptr(), stream) == 0
    got = torch.full((n,), -9, dtype=torch.int32, device=logits.device)
    rc = lib.sb_argmax_noalloc(got.data_ptr(), logits.data_ptr(), n, vocab, stream)
    assert rc == 0, lib.sb_last_error().decode()
    torch.cuda.synchronize()
    return want.cpu(), got.cpu()


def test_two_calls_in_a_row_the_second_smaller():
    lib = _library()
    dev = torch.device("cuda:0")
    g = torch.Generator(device="cpu").manual_seed(5)
    big = torch.randn((37, 152064), generator=g).to(dev)
    big[3, 151000] = 50.0                      # a maximum in the last part
    big[4, 9000] = big[4, 70000] = 60.0        # a tie across parts: the lower id wins
    small = torch.randn((5, 20001), generator=g).to(dev)
    small[2, 20000] = 40.0
    for logits in (big, small):
        want, got = _both(lib, logits)
        assert torch.equal(got, want)
        assert torch.equal(got.long(), torch.argmax(logits.cpu(), dim=1))
    assert int(got[2]) == 20000
    # one part: the fixed buffer is not used at all
    tiny = torch.randn((3, 300), generator=g).to(dev)
    want, got = _both(lib, tiny)
    assert torch.equal(got, want)


def test_sizes_beyond_the_fixed_buffer_are_refused():
    lib = _library()
    dev = torch.device("cuda:0")
    most = lib.sb_argmax_noalloc_max_entries()
    vocab = 152064
    parts = lib.sb_argmax_parts(vocab)
    rows = most // parts + 1
    out = torch.zeros((rows,), dtype=torch.int32, device=dev)
    one_row = torch.zeros((1, vocab), dtype=torch.float32, device=dev)
    # refused on the host before anything is launched or read
    rc = lib.sb_argmax_noalloc(out.data_ptr(), one_row.data_ptr(), rows, vocab, None)
    assert rc == 2
    assert b"fixed buffer" in lib.sb_last_error()
