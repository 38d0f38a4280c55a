"""pico_rmsnorm_bwd_static -- the entry point that allocates nothing -- against pico_rmsnorm_bwd, through the C ABI.

Both run the same kernels; the only difference is where the per-block partial sums of dweight live (a static device
array inside the library instead of the caller's workspace), so dx and dweight must agree bit for bit.  Two calls
in a row, the second with a smaller input: the array keeps the first call's contents and nothing of it may leak
into the second result.
"""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else None


def _both(lib, check, rows, hidden, dtype, with_residual, dw_dtype, seed):
    from picotron_amd._lib import PICO_BF16, PICO_F32
    code = {torch.bfloat16: PICO_BF16, torch.float32: PICO_F32}
    dev = torch.device("cuda", 0)
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(rows, hidden, generator=g).to(dtype).to(dev)
    dy = torch.randn(rows, hidden, generator=g).to(dtype).to(dev)
    w = (1 + 0.1 * torch.randn(hidden, generator=g)).to(dtype).to(dev)
    dres = torch.randn(rows, hidden, generator=g).to(dtype).to(dev) if with_residual else None
    rstd = torch.rsqrt(x.float().pow(2).mean(-1) + 1e-5)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)

    # the existing entry point, with a workspace from torch
    ws_bytes = lib.pico_rmsnorm_bwd_workspace_bytes(rows, hidden)
    ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=dev)
    dx_a = torch.empty_like(x)
    dw_a = torch.empty(hidden, dtype=dw_dtype, device=dev)
    check(lib.pico_rmsnorm_bwd(_ptr(dy), _ptr(x), _ptr(w), _ptr(rstd), _ptr(dres), _ptr(dx_a), _ptr(dw_a), code[dw_dtype],
                               _ptr(ws), ws_bytes, rows, hidden, code[dtype], stream))
    # the entry point under test: outputs allocated BEFORE the call, nothing else handed over
    dx_b = torch.full_like(x, float("nan"))
    dw_b = torch.full((hidden,), float("nan"), dtype=dw_dtype, device=dev)
    # one call first: the first call on a device looks up the array's address (and, for long rows, raises the
    # kernel's LDS limit); what is measured is a call after that
    check(lib.pico_rmsnorm_bwd_static(_ptr(dy), _ptr(x), _ptr(w), _ptr(rstd), _ptr(dres), _ptr(dx_b), _ptr(dw_b),
                                      code[dw_dtype], rows, hidden, code[dtype], stream))
    dx_b.fill_(float("nan"))
    dw_b.fill_(float("nan"))
    torch.cuda.synchronize()
    # the driver's own count of free device memory: an allocation inside the library (which torch's allocator would
    # not see) would lower it
    free_before = torch.cuda.mem_get_info()[0]
    check(lib.pico_rmsnorm_bwd_static(_ptr(dy), _ptr(x), _ptr(w), _ptr(rstd), _ptr(dres), _ptr(dx_b), _ptr(dw_b),
                                      code[dw_dtype], rows, hidden, code[dtype], stream))
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before
    assert torch.equal(dx_a, dx_b), (rows, hidden)
    assert torch.equal(dw_a, dw_b), (rows, hidden)
    # and the result is right, not merely equal: fp32 closed form on the GPU
    xh = x.float() * rstd[:, None]
    gg = dy.float() * w.float()
    want_dx = rstd[:, None] * (gg - xh * (gg * xh).mean(-1, keepdim=True))
    if dres is not None:
        want_dx = want_dx + dres.float()
    want_dw = (dy.float() * xh).sum(0)
    tol = 2e-2 if dtype == torch.bfloat16 else 1e-5
    assert ((dx_b.float() - want_dx).norm() / want_dx.norm()).item() <= tol
    assert ((dw_b.float() - want_dw).norm() / want_dw.norm()).item() <= tol


def test_static_scratch_entry_matches_workspace_entry():
    from picotron_amd import _lib
    lib = _lib.lib()
    assert lib.pico_rmsnorm_bwd_static_max_bytes() == 4 << 20
    # two calls in a row on one GPU, the second smaller (fewer blocks, shorter rows): stale partial sums of the first
    # call lie behind and between the ones the second call writes
    _both(lib, _lib.check, 4096, 2048, torch.bfloat16, True, torch.bfloat16, seed=1)
    _both(lib, _lib.check, 37, 576, torch.bfloat16, False, torch.float32, seed=2)
    # the other kernel families: one row per 256-thread block (long rows), fp32, a single row
    _both(lib, _lib.check, 300, 8192, torch.bfloat16, True, torch.float32, seed=3)
    _both(lib, _lib.check, 5, 64, torch.float32, False, torch.float32, seed=4)
    _both(lib, _lib.check, 1, 4096, torch.bfloat16, False, torch.bfloat16, seed=5)


def test_static_scratch_entry_rejects_what_the_workspace_entry_rejects():
    from picotron_amd import _lib
    lib = _lib.lib()
    from picotron_amd._lib import PICO_BF16
    rc = lib.pico_rmsnorm_bwd_static(None, None, None, None, None, None, ctypes.c_void_p(16), PICO_BF16, 8, 20000,
                                     PICO_BF16, None)
    assert rc < 0 and b"hidden" in lib.pico_last_error()
    rc = lib.pico_rmsnorm_bwd_static(None, None, None, None, None, None, ctypes.c_void_p(16), PICO_BF16, 8, 2048,
                                     PICO_BF16, None)
    assert rc < 0 and b"required" in lib.pico_last_error()
