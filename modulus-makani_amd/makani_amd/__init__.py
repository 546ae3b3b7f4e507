"""MI355X-native SFNO spectral hot path: RealSHT / InverseRealSHT / SpectralConv (dhconv)
on hand-written HIP kernels behind the C ABI of include/sfno_spectral.h."""
from .sht import RealSHT, InverseRealSHT, quadrature, legendre_table, legendre_gauss_weights, clenshaw_curtiss_weights, lobatto_weights
from .layers import RealFFT2, InverseRealFFT2
from .contractions import _contract_dhconv, _contract_diagonal, get_contract_fun, dhconv_spectral
from .spectral_convolution import SpectralConv
from .losses import GeometricH1Loss, degree_power
from .sfnonet import SphericalFourierNeuralOperatorNet
from .stepper import Preprocessor2D, SingleStepWrapper, MultiStepWrapper, FourierNeuralOperatorNet, get_model

__all__ = [
    "SphericalFourierNeuralOperatorNet", "FourierNeuralOperatorNet", "Preprocessor2D", "SingleStepWrapper", "MultiStepWrapper", "get_model",
    "RealSHT", "InverseRealSHT", "RealFFT2", "InverseRealFFT2", "SpectralConv", "GeometricH1Loss", "degree_power", "quadrature", "legendre_table", "legendre_gauss_weights",
    "clenshaw_curtiss_weights", "lobatto_weights", "_contract_dhconv", "_contract_diagonal", "get_contract_fun", "dhconv_spectral",
]
