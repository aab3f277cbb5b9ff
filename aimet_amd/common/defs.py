"""Quantization scheme / data type enums and the scheme->analyzer maps
(TrainingExtensions/common/src/python/aimet_common/defs.py:47-84, 302-315)."""
import enum

from . import libpymo

# Same member names and values as the reference's enumerations (members are numbered in the order listed).
QuantScheme = enum.Enum('QuantScheme', ['post_training_tf', 'post_training_tf_enhanced',
                                        'training_range_learning_with_tf_init',
                                        'training_range_learning_with_tf_enhanced_init', 'training_range_learning',
                                        'post_training_percentile'], start=1, module=__name__)
QuantScheme.__doc__ = "How encodings are found: post-training calibration schemes and range-learning initialisations."

QuantizationDataType = enum.Enum('QuantizationDataType', ['undefined', 'int', 'float'], start=0, module=__name__)
QuantizationDataType.__doc__ = "Grid of a tensor quantizer: integer (affine) or float."


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
    """Stretch of AdaRound's rectified sigmoid: h = clamp(sigmoid(alpha) * (ZETA - GAMMA) + GAMMA, 0, 1)."""
    GAMMA, ZETA = -0.1, 1.1
