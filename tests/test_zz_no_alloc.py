"""gmc_eval_bwd_static (the backward entry point that allocates nothing: its per-Gaussian sums live in a static
device array inside the library) against gmc_eval_bwd / gmc_eval_cov_bwd with a caller's workspace, through the raw
C ABI.  Two calls in a row on the shared array, the second with a smaller input, in both precisions, with several
point chunks per mixture (zero fill + atomics + epilogue launch) and with one chunk per mixture (plain stores,
epilogue inside the pair kernel).  Tolerances as everywhere: relative L2 <= 1e-5 (float32) / 1e-12 (float64); the
two entry points run the same kernels, only the order of the atomic additions differs."""
import ctypes

import numpy as np
import pytest
import torch

from conftest import rel_l2
from gmc import _native, synthetic

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
TOL = {torch.float32: 1e-5, torch.float64: 1e-12}


def _inputs(B, L, M, N, D, dtype, seed, broadcast=False):
    g = torch.Generator().manual_seed(seed)
    mix = synthetic.random_inversed_mixture(B, L, M, D, g, dtype=torch.float64).to(dtype).to(DEV)
    shape = (1, 1, N, D) if broadcast else (B, L, N, D)
    xes = (torch.rand(shape, generator=g, dtype=torch.float64) * 20 - 10).to(dtype).to(DEV)
    gout = torch.randn((B, L, N), generator=g, dtype=torch.float64).to(dtype).to(DEV)
    return mix.contiguous(), xes.contiguous(), gout.contiguous()


def _both(mix, xes, gout, need_m, need_x, cov):
    lib = _native.lib()
    shape = _native.check_input(mix, xes)
    stream = _native._stream(mix.device)
    # existing entry point, workspace from the caller
    gm_ref, gx_ref = torch.full_like(mix, 7.0), torch.full_like(xes, 7.0)
    ws_bytes = lib.gmc_eval_bwd_workspace_bytes(ctypes.byref(shape))
    ws = torch.empty((max(ws_bytes, 8) // 8,), dtype=torch.float64, device=mix.device)
    fn = lib.gmc_eval_cov_bwd if cov else lib.gmc_eval_bwd
    _native.check(fn(gout.data_ptr(), mix.data_ptr(), xes.data_ptr(), gm_ref.data_ptr(), gx_ref.data_ptr(),
                     ws.data_ptr(), ws_bytes, ctypes.byref(shape), int(need_m), int(need_x), stream))
    # the entry point under test: outputs allocated here, nothing allocated inside
    gm_new, gx_new = torch.full_like(mix, 7.0), torch.full_like(xes, 7.0)
    call = lambda: _native.check(lib.gmc_eval_bwd_static(gout.data_ptr(), mix.data_ptr(), xes.data_ptr(), gm_new.data_ptr(),
                                                         gx_new.data_ptr(), ctypes.byref(shape), int(need_m), int(need_x),
                                                         int(cov), stream))
    call()                   # (the first call on a device looks up the array's address; code objects are loaded by now)
    torch.cuda.synchronize()
    # free device memory as the driver reports it (hipMemGetInfo): an allocation inside the library, which torch's
    # own counters would not see, lowers it
    free_before, _ = torch.cuda.mem_get_info()
    reserved_before = torch.cuda.memory_reserved()
    call()
    torch.cuda.synchronize()
    free_after, _ = torch.cuda.mem_get_info()
    assert torch.cuda.memory_reserved() == reserved_before and free_after == free_before
    return (gm_ref.cpu().numpy(), gx_ref.cpu().numpy()), (gm_new.cpu().numpy(), gx_new.cpu().numpy())


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
def test_static_scratch_backward_two_calls_in_a_row(dtype):
    tol = TOL[dtype]
    # first call: large (several chunks per mixture); second: smaller and in the one-chunk-per-mixture mode, so stale
    # sums of the first call lie behind and inside the part of the array the second call uses; then a third, again
    # with atomics, on the part the second call has written
    cases = [(3, 4, 300, 2500, 3, False, False), (16, 16, 40, 100, 2, False, True), (2, 3, 200, 1500, 3, True, False),
             (2, 2, 17, 700, 2, False, False)]
    for k, (B, L, M, N, D, broadcast, cov) in enumerate(cases):
        mix, xes, gout = _inputs(B, L, M, N, D, dtype, 4100 + k, broadcast)
        if cov:
            c = torch.linalg.inv(mix[..., 1 + D:].reshape(B, L, M, D, D).double())
            c = 0.5 * (c + c.transpose(-1, -2))
            mix = torch.cat([mix[..., :1 + D], c.reshape(B, L, M, D * D).to(dtype)], -1).contiguous()
        (gm_ref, gx_ref), (gm_new, gx_new) = _both(mix, xes, gout, True, True, cov)
        assert np.isfinite(gm_new).all() and np.isfinite(gx_new).all()
        assert rel_l2(gm_new, gm_ref) <= tol, f"grad mixture, call {k}"
        assert rel_l2(gx_new, gx_ref) <= tol, f"grad xes, call {k}"
    # need flags: an output that is not asked for is not touched
    mix, xes, gout = _inputs(2, 2, 50, 300, 3, dtype, 4200)
    (gm_ref, gx_ref), (gm_new, gx_new) = _both(mix, xes, gout, True, False, False)
    assert rel_l2(gm_new, gm_ref) <= tol and (gx_new == 7.0).all()
    (gm_ref, gx_ref), (gm_new, gx_new) = _both(mix, xes, gout, False, True, False)
    assert rel_l2(gx_new, gx_ref) <= tol and (gm_new == 7.0).all()


def test_static_scratch_backward_rejects_oversized_shapes():
    lib = _native.lib()
    null = ctypes.c_void_p(0)
    # 64 MiB / (10 floats) = 1 677 721 Gaussians in 3-D float32.  Real buffers of the shape's sizes are passed: the call
    # must return before any launch, but a regression of that check should give a wrong code, not a fault.
    big = _native.Shape(64, 64, 512, 16, 3, 64, 64, 0)
    assert lib.gmc_eval_bwd_workspace_bytes(ctypes.byref(big)) > _native.STATIC_SCRATCH_BYTES
    mix = torch.zeros(64, 64, 512, 13, device=DEV)
    mix[..., [4, 8, 12]] = 1.0
    xes = torch.zeros(64, 64, 16, 3, device=DEV)
    gout = torch.zeros(64, 64, 16, device=DEV)
    gmix, gxes = torch.empty_like(mix), torch.empty_like(xes)
    rc = lib.gmc_eval_bwd_static(gout.data_ptr(), mix.data_ptr(), xes.data_ptr(), gmix.data_ptr(), gxes.data_ptr(),
                                 ctypes.byref(big), 1, 1, 0, _native._stream(mix.device))
    torch.cuda.synchronize()
    assert rc == -8 and b"static scratch" in lib.gmc_error_string(rc)
    assert lib.gmc_eval_bwd_static(null, null, null, null, null, ctypes.byref(_native.Shape(2, 2, 4, 5, 3, 2, 2, 0)),
                                   1, 1, 0, null) == -4


def test_static_scratch_backward_in_a_captured_graph():
    """After one eager call on the device (which looks up the address of the static array) the entry point only
    enqueues kernels: it is captured into a HIP graph with outputs allocated beforehand, and every replay, with eager
    work of the same entry point in between, gives what gmc_eval_bwd gives."""
    lib = _native.lib()
    mix, xes, gout = _inputs(3, 4, 300, 2500, 3, torch.float32, 4300)
    shape = _native.check_input(mix, xes)
    gm_ref, gx_ref = _native.eval_bwd(gout, mix, xes, True, True)
    gm_new, gx_new = torch.empty_like(mix), torch.empty_like(xes)
    small = _inputs(2, 2, 40, 300, 3, torch.float32, 4301)
    small_shape = _native.check_input(small[0], small[1])
    gm_small, gx_small = torch.empty_like(small[0]), torch.empty_like(small[1])

    def call(stream):
        _native.check(lib.gmc_eval_bwd_static(gout.data_ptr(), mix.data_ptr(), xes.data_ptr(), gm_new.data_ptr(),
                                              gx_new.data_ptr(), ctypes.byref(shape), 1, 1, 0, stream))

    call(_native._stream(mix.device))                       # the eager call that must precede a capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call(_native._stream(mix.device))
    torch.cuda.synchronize()
    for _ in range(3):
        gm_new.fill_(7.0)
        gx_new.fill_(7.0)
        graph.replay()
        torch.cuda.synchronize()
        assert rel_l2(gm_new.cpu().numpy(), gm_ref.cpu().numpy()) <= 1e-5
        assert rel_l2(gx_new.cpu().numpy(), gx_ref.cpu().numpy()) <= 1e-5
        # eager work on the shared array between the replays
        _native.check(lib.gmc_eval_bwd_static(small[2].data_ptr(), small[0].data_ptr(), small[1].data_ptr(), gm_small.data_ptr(),
                                              gx_small.data_ptr(), ctypes.byref(small_shape), 1, 1, 0,
                                              _native._stream(mix.device)))
        torch.cuda.synchronize()
