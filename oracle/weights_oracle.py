"""CPU oracle for the weight modifier and the weight clip of Analog-MoE.  TEST INFRASTRUCTURE ONLY.

numpy restatement of ``AnalogSigmaMoELayerAIHWKITLightning.modify_weight`` and ``clip_weights``
(analog_moe/moe_layer_aihwkit_lightning.py:313-382, 519-543) and of their AIHWKIT-flavour subset
(analog_moe/moe_layer_aihwkit.py:144-196, 313-340).  Nothing in the shipped package imports it.

Pinned (tests/test_oracle.py): ``weight_std`` / ``clip_weights`` against numpy's ``std(ddof=1)`` and ``clip`` and
against torch's ``std`` / ``clamp`` on the CPU; the ADD_NORMAL arithmetic with injected normals against the same
tensor expression evaluated by torch on the CPU in fp32 and bf16 (op-by-op rounding); the assumed max |W| of every
modifier type, including the reference's type list that leaves ADD_NORMAL_PER_CHANNEL on the per-expert maximum.

PARITY UNPINNED: the discretising step.  The reference calls ``UniformQuantize.apply(w, res, 1.0, True)`` of the
third-party ``aihwkit_lightning`` (not in the reference checkout, no version pinned by it); it is restated here
as ``round(w / res) * res`` with round-half-to-even, which the tests pin only through what any uniform quantiser
with step ``res`` must satisfy (results are multiples of ``res`` within ``res / 2`` of the input, the largest
weight maps to itself, the map is idempotent) and through the same expression evaluated by torch.  The normals
themselves come from ``torch.randn`` in the reference and from ``cvmm_oracle.box_muller_noise`` here.
"""
from __future__ import annotations

from typing import Optional

import numpy as np

from .cvmm_oracle import F32, _cast, box_muller_noise

MODIFIER_STREAM = 0x4D4F44      # the "K-tile" id that keeps the modifier's draws apart from the output noise

PER_CHANNEL_WMAX = ("DISCRETIZE_PER_CHANNEL", "DISCRETIZE_ADD_NORMAL_PER_CHANNEL")   # lightning.py:333-337


def assumed_wmax(w: np.ndarray, per_channel: bool) -> np.ndarray:
    """max |w| over K -> [E, 1, N], or over (K, N) -> [E, 1, 1] (lightning.py:338-344)."""
    a = np.abs(np.asarray(w, dtype=F32))
    return a.max(axis=1, keepdims=True) if per_channel else a.max(axis=(1, 2), keepdims=True)


def modifier_normals(E: int, K: int, N: int, seed: int) -> np.ndarray:
    """The kernel's own draws: row e*K + k of the counter-based generator, column n."""
    n2 = N + (N & 1)
    z = box_muller_noise(np.arange(E * K), n2, MODIFIER_STREAM, seed)
    return z[:, :N].reshape(E, K, N)


def modify_weight(w: np.ndarray, kind: str, res: float = 254.0, std_dev: float = 0.0,
                  z: Optional[np.ndarray] = None, dtype: str = "f32", round_noise: bool = True,
                  wmax: Optional[np.ndarray] = None) -> np.ndarray:
    """lightning.py:331-381 for ``kind`` = the modifier type's name; ``z`` are the standard normals.
    Every tensor operation rounds to ``dtype`` as torch's element-wise kernels do (computed in fp32, stored in
    the tensor's type).  ``wmax`` overrides the assumed maximum (the AIHWKIT flavour picks it by remap type)."""
    w = _cast(w, dtype)
    if kind == "NONE":
        return w
    if wmax is None:
        wmax = assumed_wmax(w, kind in PER_CHANNEL_WMAX)
    wmax = np.asarray(wmax, dtype=F32)
    out = w
    with np.errstate(divide="ignore", invalid="ignore"):
        if kind.startswith("DISCRETIZE"):
            n_states = F32(max(res, 1.0 / res))                                    # :357-358
            # :360; a tensor divided by a host scalar is a multiplication by the scalar's fp32 reciprocal
            # in torch's GPU kernels, the only place the reference runs
            step = _cast(wmax * (F32(1.0) / n_states), dtype)
            out = _cast(np.rint(_cast(out / step, dtype)) * step, dtype)           # UniformQuantize (unpinned)
        if "ADD_NORMAL" in kind:
            zz = _cast(z, dtype) if round_noise else np.asarray(z, dtype=F32)      # randn_like(w) has w's type
            noise = _cast(_cast(F32(std_dev) * wmax, dtype) * zz, dtype)           # :366-367, :374-377
            out = _cast(out + noise, dtype)
    return out


def weight_std(w: np.ndarray, per_channel: bool) -> np.ndarray:
    """Unbiased std over K -> [E, 1, N] or over (K, N) -> [E, 1, 1], two-pass in float64 (lightning.py:529-534)."""
    w64 = np.asarray(w, dtype=np.float64)
    axes = 1 if per_channel else (1, 2)
    n = w64.shape[1] if per_channel else w64.shape[1] * w64.shape[2]
    mean = w64.mean(axis=axes, keepdims=True)
    with np.errstate(divide="ignore", invalid="ignore"):
        return np.sqrt(((w64 - mean) ** 2).sum(axis=axes, keepdims=True) / (n - 1)).astype(F32)


def clip_weights(w: np.ndarray, kind: str, sigma: float, dtype: str = "f32") -> np.ndarray:
    """lightning.py:519-543: clamp to +-sigma * std, per expert (LAYER_GAUSSIAN) or per channel."""
    w = _cast(w, dtype)
    if kind == "NONE":
        return w
    if kind not in ("LAYER_GAUSSIAN", "LAYER_GAUSSIAN_PER_CHANNEL"):
        raise ValueError(f"Unknown clip type {kind}")
    std = _cast(weight_std(w, kind == "LAYER_GAUSSIAN_PER_CHANNEL"), dtype)        # std() returns w's type
    bound = _cast(F32(sigma) * std, dtype)
    return np.minimum(np.maximum(w, -bound), bound)
