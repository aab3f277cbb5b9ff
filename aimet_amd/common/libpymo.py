"""Value types and enums of the reference's ``_libpymo`` pybind module that the hot path uses.

Mirrors ModelOptimizations/PyModelOptimizations/PyModelOptimizations.cpp:147-177, 232-258 (``TfEncoding`` and the
enums) with identical field names and integer values (the pure-Python mirror of those values is
TrainingExtensions/common/src/python/aimet_common/py_libpymo.py:137-222).
"""
import enum


class TfEncoding:
    """struct TfEncoding {double min, max, delta, offset; int bw}
    (ModelOptimizations/DlQuantization/include/DlQuantization/Quantization.hpp:113-120)."""
    __slots__ = ("min", "max", "delta", "offset", "bw")

    def __init__(self, min=0.0, max=0.0, delta=0.0, offset=0.0, bw=0):  # pylint: disable=redefined-builtin
        self.min, self.max, self.delta, self.offset, self.bw = float(min), float(max), float(delta), float(offset), \
            int(bw)

    def __repr__(self):
        return f"TfEncoding(min={self.min}, max={self.max}, delta={self.delta}, offset={self.offset}, bw={self.bw})"

    def __eq__(self, other):
        return isinstance(other, TfEncoding) and \
            (self.min, self.max, self.delta, self.offset, self.bw) == \
            (other.min, other.max, other.delta, other.offset, other.bw)

    __hash__ = None

    def __getstate__(self):
        return (self.min, self.max, self.delta, self.offset, self.bw)

    def __setstate__(self, state):
        self.min, self.max, self.delta, self.offset, self.bw = state


class ComputationMode(enum.Enum):
    COMP_MODE_CPU = 0
    COMP_MODE_GPU = 1


class QuantizationMode(enum.Enum):
    QUANTIZATION_TF = 0
    QUANTIZATION_TF_ENHANCED = 1
    QUANTIZATION_RANGE_LEARNING = 2
    QUANTIZATION_PERCENTILE = 3
    QUANTIZATION_MSE = 4
    QUANTIZATION_ENTROPY = 5


class RoundingMode(enum.Enum):
    ROUND_NEAREST = 0
    ROUND_STOCHASTIC = 1


class TensorQuantizerOpMode(enum.Enum):
    updateStats = 0
    oneShotQuantizeDequantize = 1
    quantizeDequantize = 2
    passThrough = 3
