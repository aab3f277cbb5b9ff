"""Quantization scheme / data type enums and the scheme->analyzer maps
(TrainingExtensions/common/src/python/aimet_common/defs.py:47-84, 302-315)."""
from enum import Enum

from . import libpymo


class QuantScheme(Enum):
    """Enumeration of quant schemes (same names and values as the reference)."""
    post_training_tf = 1
    post_training_tf_enhanced = 2
    training_range_learning_with_tf_init = 3
    training_range_learning_with_tf_enhanced_init = 4
    training_range_learning = 5
    post_training_percentile = 6


class QuantizationDataType(Enum):
    """Tensor quantizer data types."""
    undefined = 0
    int = 1
    float = 2


MAP_QUANT_SCHEME_TO_PYMO = {
    QuantScheme.post_training_tf: libpymo.QuantizationMode.QUANTIZATION_TF,
    QuantScheme.post_training_tf_enhanced: libpymo.QuantizationMode.QUANTIZATION_TF_ENHANCED,
    QuantScheme.training_range_learning_with_tf_init: libpymo.QuantizationMode.QUANTIZATION_TF,
    QuantScheme.training_range_learning_with_tf_enhanced_init: libpymo.QuantizationMode.QUANTIZATION_TF_ENHANCED,
    QuantScheme.post_training_percentile: libpymo.QuantizationMode.QUANTIZATION_PERCENTILE,
}

MAP_ROUND_MODE_TO_PYMO = {'nearest': libpymo.RoundingMode.ROUND_NEAREST,
                          'stochastic': libpymo.RoundingMode.ROUND_STOCHASTIC}


class AdaroundConstants:
    """Constants of the rectified sigmoid used by AdaRound."""
    GAMMA = -0.1
    ZETA = 1.1
