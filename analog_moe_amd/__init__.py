"""MI355X-native CVMM path of Analog-MoE: hand-written HIP kernels (gfx950) behind a C ABI,
with the reference's CVMM / AnalogSigmaMoELayer interface on top."""
from . import _abi  # noqa: F401

__all__ = ["_abi", "ops", "raw"]
