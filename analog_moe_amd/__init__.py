"""MI355X-native CVMM path of Analog-MoE: hand-written HIP kernels (gfx950) behind a C ABI,
with the reference's CVMM / AnalogSigmaMoELayer interface on top.

The names the reference's package exports (analog_moe/__init__.py) are importable from here too:
``AnalogSigmaMoELayerAIHWKITLightning``, ``AnalogSigmaMoELayerAIHWKIT``, ``CVMM``, ``CVMMSel``."""
from . import _abi  # noqa: F401

_EXPORTS = {
    "AnalogSigmaMoELayerAIHWKITLightning": "moe_layer", "AnalogSigmaMoELayerAIHWKIT": "moe_layer",
    "AnalogSigmaMoELayer": "moe_layer", "SigmaMoELayer": "moe_layer", "MoEConifgError": "moe_layer",
    "CVMM": "cvmm", "CVMMSel": "cvmm", "cvmm_prepare_sel": "cvmm", "cvmm_std": "cvmm",
}

__all__ = ["_abi", "ops", "raw", *_EXPORTS]


def __getattr__(name):
    if name in _EXPORTS:
        import importlib
        return getattr(importlib.import_module(f".{_EXPORTS[name]}", __name__), name)
    raise AttributeError(f"module {__name__!r} has no attribute {name!r}")
