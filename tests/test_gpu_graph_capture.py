"""The compute entry points only enqueue kernels (no allocation, no synchronisation, no stream creation), so a caller may
record them into a HIP graph, as Makani records its whole step (makani/utils/trainer.py:84-152).  Captured here through
the C ABI: forward transform -> dhconv -> inverse transform on caller-preallocated buffers, replayed several times with
new inputs and eager work in between; every replay must equal the eager result bit for bit."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr())


@pytest.mark.parametrize("shape", [dict(nlat=33, nlon=64, lmax=16, mmax=17, grid="equiangular", B=2, C=6),
                                   dict(nlat=240, nlon=480, lmax=240, mmax=241, grid="legendre-gauss", B=1, C=16)])
def test_spectral_chain_replays_from_a_graph(lib_built, shape):
    from makani_amd import _lib
    from makani_amd._lib import lib, check

    print(f"case graph capture {shape}", flush=True)
    dev = torch.device("cuda:0")
    nlat, nlon, lmax, mmax, B, C = (shape[k] for k in ("nlat", "nlon", "lmax", "mmax", "B", "C"))
    rows = B * C
    plan = ctypes.c_void_p()
    wts = ctypes.c_void_p()
    with torch.cuda.device(dev):
        check(lib.sfno_sht_plan_create(nlat, nlon, lmax, mmax, _lib.GRID[shape["grid"]], 0, 1, _lib.DIR_FORWARD | _lib.DIR_INVERSE,
                                       _lib.COMPUTE_FP32, ctypes.byref(plan)), "plan")
        check(lib.sfno_dhconv_weights_create(C, C, lmax, _lib.COMPUTE_FP32, ctypes.byref(wts)), "weights")
    try:
        g = torch.Generator().manual_seed(31)
        w = (torch.complex(torch.randn(C, C, lmax, generator=g), torch.randn(C, C, lmax, generator=g)) / (2 * C) ** 0.5).to(dev)
        nbytes = lib.sfno_sht_workspace_bytes(plan, rows)
        ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)
        nspec = lib.sfno_spectral_elems(plan, rows)
        spec_a = torch.zeros(nspec, dtype=torch.float32, device=dev)
        spec_b = torch.zeros(nspec, dtype=torch.float32, device=dev)
        x = torch.zeros(B, C, nlat, nlon, device=dev)
        y = torch.zeros(B, C, nlat, nlon, device=dev)
        coeffs = torch.zeros(B, C, lmax, mmax, dtype=torch.complex64, device=dev)

        def chain():
            s = ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
            check(lib.sfno_sht_analysis(plan, _ptr(x), _lib.DTYPE_F32, _ptr(spec_a), rows, _ptr(ws), nbytes, s), "analysis")
            check(lib.sfno_dhconv_spectral(wts, _ptr(spec_a), _ptr(spec_b), B, mmax, 1, s), "dhconv")
            check(lib.sfno_sht_synthesis(plan, _ptr(spec_b), _ptr(y), _lib.DTYPE_F32, rows, _ptr(ws), nbytes, s), "synthesis")
            # the entry point whose scratch lives inside the library is meant for exactly this use
            check(lib.sfno_sht_forward_static(plan, _ptr(x), _ptr(coeffs), rows, s), "forward_static")

        check(lib.sfno_dhconv_weights_update(wts, _ptr(w), ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)), "pack")
        inputs = [torch.randn(B, C, nlat, nlon, generator=g).to(dev) for _ in range(4)]
        eager = []
        for xi in inputs:
            x.copy_(xi)
            chain()
            torch.cuda.synchronize()
            eager.append((y.clone(), coeffs.clone()))
        assert torch.isfinite(eager[0][0]).all() and eager[0][0].abs().max() > 0
        y.zero_()
        coeffs.zero_()
        graph = torch.cuda.CUDAGraph()
        side = torch.cuda.Stream(dev)
        side.wait_stream(torch.cuda.current_stream(dev))
        with torch.cuda.stream(side):
            x.copy_(inputs[0])
            chain()                                 # warm-up on the capture stream
        torch.cuda.current_stream(dev).wait_stream(side)
        torch.cuda.synchronize()
        with torch.cuda.graph(graph, stream=side):
            chain()
        torch.cuda.synchronize()
        for rep in range(2):
            for i, xi in enumerate(inputs):
                x.copy_(xi)
                graph.replay()
                torch.cuda.synchronize()
                assert torch.equal(y, eager[i][0]), f"replay {rep}.{i}: field differs from the eager result"
                assert torch.equal(torch.view_as_real(coeffs), torch.view_as_real(eager[i][1])), f"replay {rep}.{i}: coefficients differ"
                # eager work of the program between replays, on the same buffers' neighbours
                _ = (torch.randn(1 << 16, device=dev) * 2).sum().item()
        del graph
    finally:
        torch.cuda.synchronize()
        lib.sfno_dhconv_weights_destroy(wts)
        lib.sfno_sht_plan_destroy(plan)
