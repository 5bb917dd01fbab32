"""`dpk_linear_ghost_norm_static`: the ghost-norm entry point that takes no workspace and
allocates nothing. It runs the same kernels as `dpk_linear_ghost_norm`, with the partial
sums in a buffer that is part of the library's device image, so its results must be those
of the workspace entry point bit for bit (well inside the fp32 bar of rel 1e-5), also on a
second call with a smaller input that leaves most of the buffer holding the first call's
partial sums. Both entry points are called through the C ABI with ctypes."""

import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu

FP32_REL = 1e-5

# (n, T, out, in, dtype, route): Gram route with whole-tile blocks and tail pieces, the direct
# route (which also keeps the column sums of b in the buffer), fp32 and bf16, T == 1
FIRST_THEN_SMALLER = [
    ((16, 1000, 64, 128, torch.bfloat16, 0), (3, 150, 64, 64, torch.bfloat16, 0)),
    ((6, 300, 160, 288, torch.float32, 1), (2, 70, 40, 24, torch.float32, 1)),
    ((4, 512, 1024, 16, torch.bfloat16, 2), (2, 130, 520, 8, torch.bfloat16, 2)),
    ((5, 200, 96, 64, torch.float32, 0), (5, 1, 96, 64, torch.float32, 0)),
]


def _ptr(t):
    return None if t is None else ctypes.c_void_p(t.data_ptr())


def _both(lib, shape):
    from opacus_amd._lib import DPK_BF16, DPK_F32

    n, T, out_f, in_f, dtype, route = shape
    g = torch.Generator().manual_seed(n * 1000 + T)
    a = torch.randn(n, T, in_f, generator=g).to(dtype).cuda()
    b = (torch.randn(n, T, out_f, generator=g) * 0.1).to(dtype).cuda()
    code = DPK_BF16 if dtype == torch.bfloat16 else DPK_F32
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    want_w, want_b = torch.empty(n, device="cuda"), torch.empty(n, device="cuda")
    nbytes = lib.dpk_linear_ghost_norm_workspace_bytes(n, T, out_f, in_f)
    ws = torch.empty(max(nbytes, 1), dtype=torch.uint8, device="cuda")
    rc = lib.dpk_linear_ghost_norm(
        _ptr(b), _ptr(a), code, _ptr(want_w), _ptr(want_b), n, T, out_f, in_f, 1.0, route, _ptr(ws), nbytes, stream
    )
    assert rc == 0, lib.dpk_last_error()
    got_w = torch.full((n,), float("nan"), device="cuda")
    got_b = torch.full((n,), float("nan"), device="cuda")
    rc = lib.dpk_linear_ghost_norm_static(
        _ptr(b), _ptr(a), code, _ptr(got_w), _ptr(got_b), n, T, out_f, in_f, 1.0, route, stream
    )
    assert rc == 0, lib.dpk_last_error()
    torch.cuda.synchronize()
    return (got_w.cpu(), got_b.cpu()), (want_w.cpu(), want_b.cpu()), (a, b)


@pytest.mark.parametrize("first,second", FIRST_THEN_SMALLER)
def test_static_entry_point_matches_the_workspace_one_twice_in_a_row(first, second):
    from opacus_amd import _lib
    from oracle import dp_oracle as O

    lib = _lib.lib()
    for shape in (first, second):
        (got_w, got_b), (want_w, want_b), (a, b) = _both(lib, shape)
        assert torch.isfinite(got_w).all() and torch.isfinite(got_b).all()
        # same kernels, same order of summation: the same bits
        assert torch.equal(got_w, want_w), shape
        assert torch.equal(got_b, want_b), shape
        # and both agree with the float64 oracle to the fp32 bar (the inputs are exact in either dtype)
        ow, ob = O.linear_norm_sample(a.cpu().double(), b.cpu().double())
        bar = 1e-4 if a.dtype == torch.bfloat16 else FP32_REL  # the bars of the workspace entry point's tests
        assert ((got_w.double() - ow).abs() / ow).max() < bar, shape
        assert ((got_b.double() - ob).abs() / ob).max() < bar, shape


def test_static_entry_point_refuses_what_does_not_fit_and_takes_empty_batches():
    from opacus_amd import _lib

    lib = _lib.lib()
    # 2048 samples of 4096 positions: the partial sums alone exceed the built-in buffer
    n, T, out_f, in_f = 2048, 4096, 64, 64
    assert lib.dpk_linear_ghost_norm_workspace_bytes(n, T, out_f, in_f) > _lib.DPK_STATIC_SCRATCH_BYTES
    dummy = torch.zeros(8, device="cuda")
    rc = lib.dpk_linear_ghost_norm_static(
        _ptr(dummy), _ptr(dummy), 0, _ptr(dummy), None, n, T, out_f, in_f, 1.0, 0, None
    )
    assert rc == -1 and b"built-in buffer" in lib.dpk_last_error()
    assert lib.dpk_linear_ghost_norm_static(None, None, 0, None, None, 0, 5, 8, 8, 1.0, 0, None) == 0
