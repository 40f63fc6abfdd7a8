"""Enums shared by the kernels; names and values as in the reference
(src/nkilib_src/nkilib/core/utils/common_types.py:25-62)."""

from enum import Enum


class NormType(Enum):
    NO_NORM = 0
    RMS_NORM = 1
    LAYER_NORM = 2
    RMS_NORM_SKIP_GAMMA = 3


class ActFnType(Enum):
    SiLU = 0
    GELU = 1
    GELU_Tanh_Approx = 2
    Swish = 3


class ExpertAffinityScaleMode(Enum):
    NO_SCALE = 0
    POST_SCALE = 1
    PRE_SCALE = 2
    PRE_SCALE_DELAYED = 3


class QuantizationType(Enum):
    NONE = 0
    STATIC = 1
    ROW = 2
    MX = 3
    STATIC_MX = 4
    ROW_MX = 5


class RouterActFnType(Enum):
    """Activation of the router top-k kernel (common_types.py:39-46 of the reference)."""

    SIGMOID = 0
    SOFTMAX = 1

    def __str__(self):
        return self.name.lower()
