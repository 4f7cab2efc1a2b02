"""Duck-typed stand-ins for the rpu_config tree the analog layers read.

The reference takes an ``aihwkit_lightning`` / ``aihwkit`` ``TorchInferenceRPUConfig``; those
packages are third-party and may be absent.  These dataclasses carry the same attribute names
(and only the attributes the CVMM path reads: moe_layer_aihwkit_lightning.py:153-160, 172-189,
331-381, 435-461, 472-492, 513-543; cvmm.py:727-739, 868-877), so a real config object and
one of these are interchangeable wherever this package takes an ``rpu_config``.
Default values are this package's own choice, not a statement about the upstream defaults.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from enum import Enum


class WeightModifierType(Enum):
    NONE = "None"
    COPY = "Copy"                       # the two AIHWKIT-only members (moe_layer_aihwkit.py:166-170)
    MULT_NORMAL = "MultNormal"
    DISCRETIZE = "Discretize"
    DISCRETIZE_PER_CHANNEL = "DiscretizePerChannel"
    ADD_NORMAL = "AddNormal"
    ADD_NORMAL_PER_CHANNEL = "AddNormalPerChannel"
    DISCRETIZE_ADD_NORMAL = "DiscretizeAddNormal"
    DISCRETIZE_ADD_NORMAL_PER_CHANNEL = "DiscretizeAddNormalPerChannel"


class WeightClipType(Enum):
    NONE = "None"
    FIXED_VALUE = "FixedValue"          # AIHWKIT flavour (moe_layer_aihwkit.py:324-340)
    AVERAGE_CHANNEL_MAX = "AverageChannelMax"
    LAYER_GAUSSIAN = "LayerGaussian"
    LAYER_GAUSSIAN_PER_CHANNEL = "LayerGaussianPerChannel"


class WeightRemapType(Enum):
    """``rpu_config.remap.type`` of the AIHWKIT flavour: which max |W| the analog tile is assumed to be
    normalised by (moe_layer_aihwkit.py:172-182, 264-279)."""
    NONE = "None"
    LAYERWISE_SYMMETRIC = "LayerwiseSymmetric"
    CHANNELWISE_SYMMETRIC = "ChannelwiseSymmetric"


class NoiseManagementType(Enum):
    NONE = "None"
    ABS_MAX = "AbsMax"


@dataclass
class IOParameters:
    """``rpu_config.forward``.  The lightning flavour has no ``is_perfect`` attribute; that is how
    cvmm.py:727 tells the two flavours apart, so it is absent here too (see AIHWKITIOParameters)."""
    inp_res: float = -1.0          # 2**8 - 2 or 1 / (2**8 - 2) both mean 8 bit; <= 0: off
    out_res: float = -1.0          # ADC states (same spelling rules); <= 0: off
    out_bound: float = -1.0        # ADC clamp in units of max|W|; <= 0: off
    out_noise: float = 0.0         # Gaussian output noise std in units of max|W|
    out_noise_per_channel: bool = False
    inp_bound: float = 1.0


@dataclass
class AIHWKITIOParameters(IOParameters):
    """``rpu_config.forward`` of the full AIHWKIT flavour (moe_layer_aihwkit.py:47-61)."""
    is_perfect: bool = False
    noise_management: NoiseManagementType = NoiseManagementType.NONE
    bound_management: str = "None"


@dataclass
class InputRangeParameter:
    """``rpu_config.pre_post.input_range``."""
    enable: bool = False
    learn_input_range: bool = True
    init_value: float = 3.0
    init_from_data: int = 0
    init_std_alpha: float = 3.0
    decay: float = 0.0
    input_min_percentage: float = 0.95
    gradient_relative: bool = True
    gradient_scale: float = 1.0


@dataclass
class PrePostProcessing:
    input_range: InputRangeParameter = field(default_factory=InputRangeParameter)


@dataclass
class MappingParameter:
    max_input_size: int = -1       # <= 0: one tile
    max_output_size: int = -1


@dataclass
class WeightModifierParameter:
    type: WeightModifierType = WeightModifierType.NONE
    res: float = 2 ** 8 - 2
    std_dev: float = 0.0
    enable_during_test: bool = False
    per_batch_sample: bool = False


@dataclass
class WeightClipParameter:
    type: WeightClipType = WeightClipType.NONE
    sigma: float = 2.5
    fixed_value: float = -1.0


@dataclass
class WeightRemapParameter:
    type: WeightRemapType = WeightRemapType.LAYERWISE_SYMMETRIC


@dataclass
class TorchInferenceRPUConfig:
    forward: IOParameters = field(default_factory=IOParameters)
    pre_post: PrePostProcessing = field(default_factory=PrePostProcessing)
    mapping: MappingParameter = field(default_factory=MappingParameter)
    modifier: WeightModifierParameter = field(default_factory=WeightModifierParameter)
    clip: WeightClipParameter = field(default_factory=WeightClipParameter)


@dataclass
class AIHWKITTorchInferenceRPUConfig(TorchInferenceRPUConfig):
    """The attributes the AIHWKIT flavour reads on top (moe_layer_aihwkit.py:47-61, 243-279)."""
    forward: AIHWKITIOParameters = field(default_factory=AIHWKITIOParameters)
    remap: WeightRemapParameter = field(default_factory=WeightRemapParameter)


def kernel_inp_res(res: float) -> float:
    """rpu resolution -> quantisation step of the kernel: ``2/res`` for res > 1, ``2*res`` for
    0 < res <= 1, off otherwise (moe_layer_aihwkit_lightning.py:451-456)."""
    if res is not None and res > 0:
        return 2.0 / res if res > 1.0 else 2.0 * res
    return -1.0


def enum_name(v) -> str:
    """Name of an enum member of either this module or the third-party config packages."""
    return getattr(v, "name", str(v)).upper()
