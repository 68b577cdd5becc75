"""The entry point that allocates nothing: ``bnb_rmsnorm_bwd_static`` against ``bnb_rmsnorm_bwd``.

Both run the same kernels; the static one keeps the per-work-group partial weight gradients in a
buffer built into the library instead of a workspace of the caller's.  Integer-free float work, so
the bar is the existing entry point's own: identical bits (same kernels, same order of every sum).
Two calls in a row, the second with a smaller input, so anything the first call left in the buffer
would show in the second call's weight gradient.
"""

import ctypes

import pytest
import torch

from helpers import max_rel

import boost_and_broadside_amd as bnb
from boost_and_broadside_amd import _native, ops

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def _case(R, D, seed, dy_dtype):
    g = torch.Generator().manual_seed(seed)
    x = (torch.randn(R, D, generator=g) * (0.2 + 3.0 * torch.rand(R, 1, generator=g))).to(DEV)
    dy = torch.randn(R, D, generator=g).to(dy_dtype).to(DEV)
    gs = torch.randn(R, D, generator=g).to(DEV)
    w = (1.0 + 0.3 * torch.randn(D, generator=g)).to(DEV)
    return x, dy, gs, w


def _static_call(x, dy, gs, w, eps):
    """Straight through the C ABI with preallocated outputs (ctypes, no wrapper logic in between)."""
    R, D = x.shape
    dx = torch.full((R, D), float("nan"), device=DEV)
    dw = torch.full((D,), float("nan"), device=DEV)
    dx_lp = torch.zeros((R, D), dtype=torch.bfloat16, device=DEV)
    lib = _native.load()
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    rc = lib.bnb_rmsnorm_bwd_static(
        x.data_ptr(), D, dy.data_ptr(), _native.BF16 if dy.dtype == torch.bfloat16 else _native.F32, D, w.data_ptr(),
        ctypes.c_float(eps), gs.data_ptr(), dx.data_ptr(), dx_lp.data_ptr(), dw.data_ptr(), R, D,
        torch.cuda.current_stream().cuda_stream)
    _native.check(rc, "bnb_rmsnorm_bwd_static")
    torch.cuda.synchronize()
    # the call took no device memory from the driver: its workspace is part of the loaded library
    assert torch.cuda.mem_get_info()[0] == free_before
    return dx, dw, dx_lp


def test_static_workspace_entry_point_matches_the_workspace_one_on_two_calls_in_a_row():
    eps = 1e-5
    # first a large input (every work-group's partial row is written), then a small one that uses
    # fewer rows of the shared buffer and a different width
    for R, D, seed, dy_dtype in ((70001, 128, 1, torch.bfloat16), (37, 256, 2, torch.float32), (3001, 128, 3, torch.bfloat16)):
        x, dy, gs, w = _case(R, D, seed, dy_dtype)
        want_dx, want_dw, want_lp = ops.rmsnorm_bwd(x, dy, w, eps=eps, grad_sum=gs, also_bf16=True)
        got_dx, got_dw, got_lp = _static_call(x, dy, gs, w, eps)
        assert torch.equal(got_dx, want_dx), (R, D)
        assert torch.equal(got_dw, want_dw), (R, D)
        assert torch.equal(got_lp, want_lp), (R, D)
        # and against the definition, so both cannot be wrong together
        xr, wr = x.cpu().double().requires_grad_(), w.cpu().double().requires_grad_()
        n = xr * torch.rsqrt(xr.pow(2).mean(-1, keepdim=True) + eps) * wr
        (n * dy.cpu().double()).sum().backward()
        assert max_rel(got_dx.cpu().double(), xr.grad + gs.cpu().double()) <= 1e-5
        assert max_rel(got_dw.cpu().double(), wr.grad) <= 1e-5


def test_static_workspace_wrapper_and_limits():
    x, dy, gs, w = _case(513, 128, 5, torch.bfloat16)
    dx, dw = torch.empty_like(x), torch.empty_like(w)
    ops.rmsnorm_bwd_static(x, dy, w, dx, dw, eps=1e-5)
    want_dx, want_dw = ops.rmsnorm_bwd(x, dy, w, eps=1e-5)
    assert torch.equal(dx, want_dx) and torch.equal(dw, want_dw)
    # no rows: the weight gradient is zero, nothing else is touched
    empty = torch.empty(0, 128, device=DEV)
    ops.rmsnorm_bwd_static(empty, empty.bfloat16(), w, torch.empty_like(empty), dw, eps=1e-5)
    assert not dw.any()
    lib = _native.load()
    assert lib.bnb_rmsnorm_bwd_static_limit() == 1280 * 512 * 4
    # beyond the built-in buffer: a clear error code, nothing launched
    wide = torch.zeros(4, 1024, device=DEV)
    rc = lib.bnb_rmsnorm_bwd_static(wide.data_ptr(), 1024, wide.data_ptr(), _native.F32, 1024, wide.data_ptr(),
                                    ctypes.c_float(1e-5), None, wide.data_ptr(), None, wide.data_ptr(), 4, 1024, None)
    assert rc == _native.ERR_SCRATCH_LIMIT
    assert b"built-in buffer" in lib.bnb_error_string(rc)
    assert bnb is not None
