"""RealFFT2 / InverseRealFFT2 with the interface of makani/models/common/layers.py:219-287: the planar
counterparts of RealSHT / InverseRealSHT (torch.fft.rfft2 / irfft2 with norm="ortho" and mode truncation),
selected by spectral_transform="fft" in the SFNO network (sfnonet.py:542-556).

They run on the same plan type, layouts and entry points as the spherical pair (grid SFNO_GRID_PLANAR): the
longitude kernels are shared and the Legendre stage is replaced by an FFT along latitude, so SpectralConv keeps
its fused path (no layout conversion between transform and channel mix) and autograd works the same way.
"""
import math

from .sht import RealSHT, InverseRealSHT, _SHTBase


def _modes(nlat, nlon, lmax, mmax):
    return min(lmax or nlat, nlat), min(mmax or nlon // 2 + 1, nlon // 2 + 1)


class _PlanarMixin:
    _planar = True

    def _init_planar(self, nlat, nlon, lmax, mmax):
        lmax, mmax = _modes(nlat, nlon, lmax, mmax)
        _SHTBase.__init__(self, nlat, nlon, lmax, mmax, grid="planar")
        self.truncate = not (self.lmax == self.nlat and self.mmax == self.nlon // 2 + 1)
        self.lmax_high = math.ceil(self.lmax / 2)
        self.lmax_low = math.floor(self.lmax / 2)

    def extra_repr(self):
        return f"nlat={self.nlat}, nlon={self.nlon}, lmax={self.lmax}, mmax={self.mmax}"

    def __deepcopy__(self, memo):
        return type(self)(self.nlat, self.nlon, self.lmax, self.mmax)


class RealFFT2(_PlanarMixin, RealSHT):
    """x [..., nlat, nlon] real -> [..., lmax, mmax] complex: the lmax_high lowest non-negative and the lmax_low
    highest latitude frequencies of rfft2(x, norm="ortho"), first mmax longitude frequencies (layers.py:219-250)."""

    def __init__(self, nlat, nlon, lmax=None, mmax=None):
        self._init_planar(nlat, nlon, lmax, mmax)

    @property
    def weights(self):
        raise AttributeError("RealFFT2 has no quadrature table")


class InverseRealFFT2(_PlanarMixin, InverseRealSHT):
    """[..., lmax, mmax] complex -> [..., nlat, nlon] real: zero-fills the dropped frequencies, then
    irfft2(norm="ortho") (layers.py:253-287)."""

    def __init__(self, nlat, nlon, lmax=None, mmax=None):
        self._init_planar(nlat, nlon, lmax, mmax)

    @property
    def pct(self):
        raise AttributeError("InverseRealFFT2 has no Legendre table")
