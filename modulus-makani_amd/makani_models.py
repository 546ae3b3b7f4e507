"""Entry file for Makani's `nettype: "path/to/file.py:ClassName"` route (makani/models/model_registry.py:63-79), which
executes the named file on its own, outside any package: it puts this directory on the import path and re-exports the
HIP networks, e.g.  nettype: "/path/to/modulus-makani_amd/makani_models.py:SphericalFourierNeuralOperatorNet"."""
import os
import sys

_HERE = os.path.dirname(os.path.abspath(__file__))
if _HERE not in sys.path:
    sys.path.insert(0, _HERE)

from makani_amd.sfnonet import SphericalFourierNeuralOperatorNet  # noqa: E402
from makani_amd.stepper import FourierNeuralOperatorNet  # noqa: E402

__all__ = ["SphericalFourierNeuralOperatorNet", "FourierNeuralOperatorNet"]
