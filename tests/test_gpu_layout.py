"""The layout passes between the reference coefficient layout complex64 [rows][lmax][mmax] (what RealSHT.forward returns,
spectral_convolution.py:131-141) and the order-major spectral layout float32 [mmax][lmax][ld]: pure data movement, so every case
is checked bit for bit against the index map written out in torch, including what must NOT be touched."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu

# rows around the tile height (80 complex rows) and the padding of ld (multiples of 16 floats); lmax/mmax around the tile width
# (64 orders), wider than tall and taller than wide
CASES = [
    (1, 7, 9), (5, 33, 32), (73, 64, 64), (79, 65, 129), (80, 130, 70), (81, 12, 12), (161, 20, 67), (384, 24, 25), (8, 1, 1), (3, 200, 3),
]


def _call(name, *args):
    from makani_amd._lib import lib, check

    check(getattr(lib, name)(*args), name)


@pytest.mark.parametrize("rows,lmax,mmax", CASES)
@pytest.mark.parametrize("tri", [1, 0])
def test_layout_passes_move_exactly_the_entries_they_should(lib_built, rows, lmax, mmax, tri):
    from makani_amd._lib import lib

    print(f"case layout rows={rows} lmax={lmax} mmax={mmax} triangular={tri}", flush=True)
    torch.manual_seed(rows * 1000 + lmax * 10 + mmax)
    dev = torch.device("cuda:0")
    ld = int(lib.sfno_spectral_ld(rows))
    assert ld >= 2 * rows and ld % 16 == 0
    sp = ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
    P = lambda t: ctypes.c_void_p(t.data_ptr())
    c = torch.randn(rows, lmax, mmax, dtype=torch.complex64)
    l_idx, m_idx = torch.arange(lmax)[:, None], torch.arange(mmax)[None, :]
    moved = (m_idx <= l_idx) if tri else torch.ones(lmax, mmax, dtype=torch.bool)        # [lmax][mmax]

    # reference layout -> spectral layout: the buffer starts as a sentinel that no input value equals
    SENT = 12345.0
    spec = torch.full((mmax, lmax, ld), SENT, dtype=torch.float32, device=dev)
    cd = c.to(dev).contiguous()
    _call("sfno_coeffs_to_spectral", P(cd), P(spec), rows, lmax, mmax, tri, sp)
    torch.cuda.synchronize()
    want = torch.full((mmax, lmax, ld), SENT, dtype=torch.float32)
    # rows (m, l) that are moved hold (re, im) of channel r at 2r, 2r+1 and zeros in the padding; the others stay untouched
    vals = torch.view_as_real(c).permute(2, 1, 0, 3).reshape(mmax, lmax, 2 * rows)     # [m][l][2r + part]
    row_moved = moved.t()                                                               # [m][l]
    full = torch.zeros(mmax, lmax, ld)
    full[:, :, : 2 * rows] = vals
    want[row_moved] = full[row_moved]
    assert torch.equal(spec.cpu(), want)

    # spectral layout -> reference layout: reads only what it moves (the sentinel rows may hold anything), writes every entry
    out = torch.full((rows, lmax, mmax), complex(SENT, SENT), dtype=torch.complex64, device=dev)
    _call("sfno_spectral_to_coeffs", P(spec), P(out), rows, lmax, mmax, tri, sp)
    torch.cuda.synchronize()
    want_c = torch.where(moved[None], c, torch.zeros((), dtype=torch.complex64))
    assert torch.equal(torch.view_as_real(out.cpu()), torch.view_as_real(want_c))
