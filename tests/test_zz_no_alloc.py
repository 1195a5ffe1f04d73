"""The arg-max entry point that allocates nothing (``tl_argmax_static``), called through ctypes:
its answers equal those of ``tl_argmax`` with caller-allocated buffers, on two calls in a row of
which the second is smaller (so it runs over what the first left in the static buffer)."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _lib():
    from tensorline_amd.ops import kernels
    lib = kernels.library()
    lib.tl_argmax_static.restype = ctypes.c_int
    lib.tl_argmax_static.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_void_p,
                                     ctypes.c_void_p]
    lib.tl_argmax_static_setup.restype = ctypes.c_int
    lib.tl_argmax_static_setup.argtypes = []
    return lib, kernels


def _static(lib, logits, out):
    R, V = logits.shape
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    return lib.tl_argmax_static(ctypes.c_void_p(logits.data_ptr()), logits.stride(0), R, V,
                                ctypes.c_void_p(out.data_ptr()), stream)


def test_static_argmax_matches_the_allocating_one_on_two_calls_in_a_row():
    lib, kernels = _lib()
    torch.cuda.set_device(0)
    assert lib.tl_argmax_static_setup() == 0, lib.tl_last_error()
    g = torch.Generator(device=DEV).manual_seed(7)
    # wide rows (above 8,192 columns partial results go through the buffer); the second call has
    # fewer rows and narrower ones, the third is narrow enough to need no buffer at all
    shapes = [(37, 152064), (5, 20011), (3, 1000)]
    inputs = [torch.randn(R, V, device=DEV, generator=g) for R, V in shapes]
    for x in inputs:                                   # make ties and a far-away winner part of the test
        x[0, -1] = 50.0
        x[-1, 3] = x[-1, x.shape[1] // 2] = 60.0
    want = [kernels.argmax(x) for x in inputs]
    outs = [torch.full((x.shape[0],), -1, dtype=torch.int32, device=DEV) for x in inputs]
    torch.cuda.synchronize()
    free0 = allocated0 = None
    for i, (x, out) in enumerate(zip(inputs, outs)):
        if i == 1:                                     # the first call may load the code object; later ones must not allocate
            free0, allocated0 = torch.cuda.mem_get_info()[0], torch.cuda.memory_allocated()
        assert _static(lib, x, out) == 0, lib.tl_last_error()
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free0 and torch.cuda.memory_allocated() == allocated0
    for x, out, w in zip(inputs, outs, want):
        assert torch.equal(out, w)
        assert torch.equal(out.long(), x.argmax(-1))
    assert outs[0][0].item() == shapes[0][1] - 1 and outs[0][-1].item() == 3


def test_static_argmax_refuses_more_rows_than_its_buffer_holds():
    lib, kernels = _lib()
    g = torch.Generator(device=DEV).manual_seed(11)
    x = torch.randn(1025, 16, device=DEV, generator=g)
    winners = torch.arange(1025, device=DEV) % 16
    x[torch.arange(1025, device=DEV), winners] = 9.0                     # a known winner in every row
    out = torch.full((1025,), -1, dtype=torch.int32, device=DEV)
    assert _static(lib, x, out) != 0
    assert b"1024" in lib.tl_last_error()
    torch.cuda.synchronize()
    assert bool((out == -1).all()), "a refused call wrote its output"
    assert _static(lib, x[:1024], out) == 0
    torch.cuda.synchronize()
    assert torch.equal(out[:1024].long(), winners[:1024]) and int(out[1024]) == -1


def test_static_argmax_at_its_row_limit_with_wide_rows():
    """1,024 rows of more than 8,192 columns: the static buffer is written and read to its last
    entry (best value and index per row and chunk), against the allocating entry point."""
    lib, kernels = _lib()
    g = torch.Generator(device=DEV).manual_seed(13)
    x = torch.randn(1024, 8200, device=DEV, generator=g)
    x[1023, 8199] = 40.0                                                 # the last row's winner in its last chunk
    x[0, 0] = x[0, 8199] = 41.0                                          # a tie across the first and the last chunk
    out = torch.full((1024,), -1, dtype=torch.int32, device=DEV)
    assert _static(lib, x, out) == 0, lib.tl_last_error()
    torch.cuda.synchronize()
    assert torch.equal(out, kernels.argmax(x)) and torch.equal(out.long(), x.argmax(-1))
    assert int(out[1023]) == 8199 and int(out[0]) == 0
