"""sfno_sht_forward_static, the entry point that allocates nothing (its scratch is a file-scope device array of the library),
called through the C ABI and compared with sfno_sht_forward, the entry point it is a variant of: bit for bit, on two calls
in a row, the second with a smaller input (the array then still holds the first call's contents); a request beyond the
array is refused with SFNO_EWORKSPACE."""
import ctypes

import numpy as np
import pytest
import torch

from oracle.sht import ShtTables, sht_forward

pytestmark = pytest.mark.gpu

STATIC_BYTES = 64 << 20


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr())


def test_static_scratch_forward_matches_workspace_forward(lib_built):
    from makani_amd import _lib
    from makani_amd._lib import lib

    print("case sfno_sht_forward_static: 33x64 equiangular, 24 rows then 5 rows", flush=True)
    dev = torch.device("cuda:0")
    nlat, nlon, lmax, mmax = 33, 64, 20, 21
    plan = ctypes.c_void_p()
    with torch.cuda.device(dev):
        rc = lib.sfno_sht_plan_create(nlat, nlon, lmax, mmax, _lib.GRID["equiangular"], _lib.NORM["ortho"], 1, _lib.DIR_FORWARD, _lib.COMPUTE_FP32,
                                      ctypes.byref(plan))
    assert rc == 0
    stream = ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
    t = ShtTables(nlat, nlon, lmax, mmax, "equiangular")
    try:
        g = torch.Generator().manual_seed(21)
        for rows in (24, 5):                      # second call: smaller input over the leftovers of the first
            x = torch.randn(rows, nlat, nlon, generator=g).to(dev)
            want = torch.full((rows, lmax, mmax), float("nan"), dtype=torch.complex64, device=dev)
            got = torch.full((rows, lmax, mmax), float("nan"), dtype=torch.complex64, device=dev)
            nbytes = lib.sfno_sht_workspace_bytes(plan, rows)
            assert 0 < nbytes <= STATIC_BYTES
            ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)
            assert lib.sfno_sht_forward(plan, _ptr(x), _ptr(want), rows, _ptr(ws), nbytes, stream) == 0
            assert lib.sfno_sht_forward_static(plan, _ptr(x), _ptr(got), rows, stream) == 0
            torch.cuda.synchronize()
            assert torch.equal(torch.view_as_real(got), torch.view_as_real(want)), f"rows={rows}"
            ref = sht_forward(x.double().cpu().numpy(), t)
            err = np.linalg.norm(got.cpu().numpy() - ref) / np.linalg.norm(ref)
            assert err < 1e-5, err
        # a transform whose buffers exceed the array is refused, and nothing is written
        rows_big = 1 << 16
        assert lib.sfno_sht_workspace_bytes(plan, rows_big) > STATIC_BYTES
        x = torch.zeros(1, device=dev)
        rc = lib.sfno_sht_forward_static(plan, _ptr(x), _ptr(x), rows_big, stream)
        assert rc == -4 and lib.sfno_strerror(rc).decode() == "workspace too small"
        assert lib.sfno_sht_forward_static(plan, None, _ptr(x), 1, stream) == -1
    finally:
        torch.cuda.synchronize()
        lib.sfno_sht_plan_destroy(plan)
