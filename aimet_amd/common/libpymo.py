"""Value types, enums and the array-fed encoding analyzer of the reference's ``_libpymo`` pybind module that the hot path
uses.

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


class EncodingAnalyzerForPython:
    """An encoding analyzer of any QuantizationMode fed with arrays: updateStats(array, use_cuda) gathers statistics,
    computeEncoding(bitwidth, isSymmetric, useStrictSymmetric, useUnsignedSymmetric) returns (TfEncoding, is_valid)
    (ModelOptimizations/DlQuantization/src/EncodingAnalyzerForPython.cpp:53-99, bound at
    PyModelOptimizations.cpp:216-219).  The reference takes host arrays and computes on the host unless told to copy
    them to the GPU; here a host array (numpy, or a CPU tensor) is copied to the current GPU, a GPU tensor is used where
    it is, and `use_cuda` does not change where the statistics are gathered."""

    _MODE_NUMBER = {QuantizationMode.QUANTIZATION_TF: 0, QuantizationMode.QUANTIZATION_TF_ENHANCED: 1,
                    QuantizationMode.QUANTIZATION_PERCENTILE: 2, QuantizationMode.QUANTIZATION_MSE: 3,
                    QuantizationMode.QUANTIZATION_ENTROPY: 4}

    def __init__(self, quantizationScheme: QuantizationMode):
        # every other mode gets the TF analyzer, as in getEncodingAnalyzerInstance (QuantizerFactory.cpp:74-97)
        self._mode = self._MODE_NUMBER.get(quantizationScheme, 0)
        self._analyzer = None
        self._is_encoding_valid = False

    def updateStats(self, input, use_cuda: bool = True):           # pylint: disable=redefined-builtin, unused-argument
        import torch                                                 # pylint: disable=import-outside-toplevel
        from .. import ops                                           # pylint: disable=import-outside-toplevel
        tensor = input if isinstance(input, torch.Tensor) else torch.as_tensor(input)
        tensor = tensor.detach().to(device="cuda" if not tensor.is_cuda else tensor.device, dtype=torch.float32)
        if self._analyzer is None or self._analyzer.device != tensor.device:
            self._analyzer = ops.Analyzer(self._mode, tensor.device)
        self._is_encoding_valid = True
        self._analyzer.update_stats(tensor.contiguous())

    def computeEncoding(self, bitwidth: int, isSymmetric: bool, useStrictSymmetric: bool, useUnsignedSymmetric: bool):
        if not self._is_encoding_valid:
            return TfEncoding(), False
        e, _ = self._analyzer.compute_encoding(bitwidth, isSymmetric, useStrictSymmetric, useUnsignedSymmetric)
        return TfEncoding(e.min, e.max, e.delta, e.offset, e.bw), True
