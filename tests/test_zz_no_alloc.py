"""The entry point that allocates nothing (csrc/no_alloc.h), called through ctypes: its result equals
li_argmax's on two calls in a row, the second with a smaller input, and sizes beyond its array are
refused."""
from ctypes import c_int, c_void_p

import pytest
import torch

pytestmark = pytest.mark.gpu


def _lib():
    from llm_infer_amd.kernels import build
    lib = build.core_library()
    lib.li_argmax_static.restype = c_int
    lib.li_argmax_static.argtypes = [c_void_p, c_int, c_int, c_void_p, c_void_p]
    lib.li_argmax_static_capacity.restype = c_int
    lib.li_argmax_static_capacity.argtypes = [c_int]
    lib.li_argmax_static_init.restype = c_int
    lib.li_argmax_static_init.argtypes = []
    lib.li_argmax_chunks.restype = c_int
    lib.li_argmax_chunks.argtypes = [c_int]
    lib.li_argmax.restype = c_int
    lib.li_argmax.argtypes = [c_void_p, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p]
    return lib


def _both(lib, logits):
    """(li_argmax_static's tokens, li_argmax's tokens) for float32 logits [rows, V] on the GPU."""
    rows, vocab = logits.shape
    stream = c_void_p(torch.cuda.current_stream().cuda_stream)
    got = torch.full((rows,), -1, dtype=torch.int32, device="cuda")
    want = torch.full((rows,), -2, dtype=torch.int32, device="cuda")
    chunks = lib.li_argmax_chunks(vocab)
    part_v = torch.empty((rows * chunks,), dtype=torch.float32, device="cuda")
    part_i = torch.empty((rows * chunks,), dtype=torch.int32, device="cuda")
    torch.cuda.synchronize()
    assert lib.li_argmax_static(logits.data_ptr(), rows, vocab, got.data_ptr(), stream) == 0
    assert lib.li_argmax(logits.data_ptr(), rows, vocab, part_v.data_ptr(), part_i.data_ptr(), want.data_ptr(),
                         stream) == 0
    torch.cuda.synchronize()
    return got.cpu(), want.cpu()


def test_argmax_static_equals_argmax_on_two_calls_in_a_row():
    lib = _lib()
    torch.cuda.set_device(0)
    assert lib.li_argmax_static_init() == 0
    g = torch.Generator(device="cuda").manual_seed(11)
    # first call: many rows and chunks, so that the array holds a lot that the second call must not read
    big = torch.randn((48, 50_021), generator=g, device="cuda", dtype=torch.float32)
    big[5, 4095] = big[5, 4096] = big[5, 40_000] = 9.0          # a tie across chunks: the first one wins
    got, want = _both(lib, big)
    assert torch.equal(got, want)
    ref = big.argmax(dim=1).cpu()
    assert all(got[r].item() == ref[r].item() for r in range(48) if r != 5)
    assert got[5].item() == 4095
    # second call, smaller in rows and in chunks: what the first left in the array changes nothing
    small = torch.randn((3, 9_001), generator=g, device="cuda", dtype=torch.float32)
    small[1, 9_000] = 7.5
    got, want = _both(lib, small)
    assert torch.equal(got, want)
    assert got.tolist() == small.argmax(dim=1).cpu().tolist() and got[1].item() == 9_000
    # one chunk only
    tiny = torch.randn((2, 100), generator=g, device="cuda", dtype=torch.float32)
    got, want = _both(lib, tiny)
    assert torch.equal(got, want) and got.tolist() == tiny.argmax(dim=1).cpu().tolist()


def test_argmax_static_refuses_what_does_not_fit():
    lib = _lib()
    vocab = 128_256
    cap = lib.li_argmax_static_capacity(vocab)
    assert cap == 8192 // lib.li_argmax_chunks(vocab) and cap >= 64
    assert lib.li_argmax_static_capacity(0) == 0
    stream = c_void_p(torch.cuda.current_stream().cuda_stream)
    out = torch.zeros((cap + 1,), dtype=torch.int32, device="cuda")
    logits = torch.zeros((1, vocab), dtype=torch.float32, device="cuda")
    # refused before anything is launched: the row count alone decides, so one row of logits is enough
    assert lib.li_argmax_static(logits.data_ptr(), cap + 1, vocab, out.data_ptr(), stream) == 2
    assert lib.li_argmax_static(None, 1, vocab, out.data_ptr(), stream) == 1
    assert lib.li_argmax_static(logits.data_ptr(), 1, vocab, out.data_ptr(), stream) == 0
    torch.cuda.synchronize()
    assert out[0].item() == 0
