"""The argmax entry point that allocates nothing (``pa_argmax_static``), called through ctypes as a caller
without an allocator would, against ``pa_argmax`` with a workspace of the caller's."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


def _lib():
    from prelude_amd import _native
    return _native.kernels()


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _with_workspace(lib, logits: torch.Tensor) -> torch.Tensor:
    rows, vocab = logits.shape
    out = torch.full((rows,), -1, dtype=torch.int32, device=logits.device)
    words = lib.pa_argmax_scratch(rows, vocab)
    ws = torch.empty(max(words, 1), dtype=torch.float32, device=logits.device)
    assert lib.pa_argmax(_stream(), logits.data_ptr(), out.data_ptr(), ws.data_ptr(), rows, vocab) == 0
    return out


def _static(lib, logits: torch.Tensor, out: torch.Tensor) -> int:
    rows, vocab = logits.shape
    return lib.pa_argmax_static(ctypes.c_void_p(_stream()), ctypes.c_void_p(logits.data_ptr()),
                                ctypes.c_void_p(out.data_ptr()), ctypes.c_int(rows), ctypes.c_int(vocab))


def test_two_calls_in_a_row_the_second_smaller():
    lib = _lib()
    dev = torch.device("cuda:0")
    g = torch.Generator(device="cpu").manual_seed(11)
    # wide rows (candidates go through the built-in array), then fewer and shorter rows that leave most of
    # what the first call wrote in place, then narrow rows that use no scratch at all
    shapes = [(7, 151936), (3, 40000), (5, 509)]
    inputs = [torch.randn(s, generator=g, dtype=torch.float32).to(dev) for s in shapes]
    # an exact tie must go to the lower index in both
    inputs[0][2, 150001] = inputs[0][2, 777] = 50.0
    inputs[1][1, 39999] = 60.0
    outs = [torch.full((s[0],), -1, dtype=torch.int32, device=dev) for s in shapes]
    for x, o in zip(inputs, outs):          # back to back on one stream, nothing in between
        assert _static(lib, x, o) == 0, lib.pa_last_error().decode()
    torch.cuda.synchronize()
    for x, o in zip(inputs, outs):
        want = _with_workspace(lib, x)
        torch.cuda.synchronize()
        assert o.tolist() == want.tolist()
    for x, o in zip(inputs[1:], outs[1:]):   # no ties there: the library's answer is the only one
        assert o.tolist() == torch.argmax(x, dim=1).tolist()
    assert outs[0][2].item() == 777
    assert outs[1][1].item() == 39999


def test_sizes_beyond_the_array_are_refused():
    lib = _lib()
    dev = torch.device("cuda:0")
    cap = lib.pa_argmax_static_capacity()
    assert cap == 65536
    rows, vocab = 64, 2048 * 600          # 64 * 600 * 2 words > 65,536
    out = torch.zeros(rows, dtype=torch.int32, device=dev)
    # refused before anything is read: the pointer only has to be non-null
    rc = lib.pa_argmax_static(ctypes.c_void_p(_stream()), ctypes.c_void_p(out.data_ptr()),
                              ctypes.c_void_p(out.data_ptr()), rows, vocab)
    assert rc != 0
    msg = lib.pa_last_error().decode()
    assert "built-in array holds 65536" in msg and "76800" in msg
    # the largest that fits runs
    x = torch.randn((16, 2048 * 1024), device=dev)       # 16 * 1024 * 2 = 32,768 words
    o = torch.full((16,), -1, dtype=torch.int32, device=dev)
    assert _static(lib, x, o) == 0
    torch.cuda.synchronize()
    assert o.tolist() == torch.argmax(x, dim=1).tolist()
