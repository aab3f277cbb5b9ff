"""``AimetTensorQuantizer``: the object the v1 tensor quantizers program against.

Same method names, argument meaning and return values as the reference's pybind class
(TrainingExtensions/torch/src/AimetTensorQuantizer.cpp:75-331), backed by the libmiq C ABI.  Differences, all on
purpose: tensors must live on the GPU (``use_cuda`` False or a CPU tensor raises ``RuntimeError`` -- there is no CPU
compute path in this package); bfloat16 tensors are accepted directly (the conversion is fused into the kernel);
kernels run on torch's current stream instead of the legacy default stream; statistics stay on the device and are
read back only when an encoding is asked for.
"""
from typing import List, Tuple

import torch

from .. import ops
from .libpymo import QuantizationMode, RoundingMode, TfEncoding

_MODE_TO_MIQ = {QuantizationMode.QUANTIZATION_TF: 0, QuantizationMode.QUANTIZATION_TF_ENHANCED: 1,
                QuantizationMode.QUANTIZATION_PERCENTILE: 2, QuantizationMode.QUANTIZATION_MSE: 3,
                QuantizationMode.QUANTIZATION_ENTROPY: 4}


def _round_mode(round_mode) -> int:
    if isinstance(round_mode, RoundingMode):
        return round_mode.value
    return int(round_mode)


def _to_tf_encoding(e) -> TfEncoding:
    return TfEncoding(e.min, e.max, e.delta, e.offset, e.bw)


class AimetTensorQuantizer:
    """Per-tensor quantization object: statistics -> encoding -> quantize-dequantize."""

    def __init__(self, quantizationScheme: QuantizationMode):
        if quantizationScheme not in _MODE_TO_MIQ:
            raise RuntimeError(f"{quantizationScheme} has no encoding analyzer")
        self._scheme = quantizationScheme
        self._percentile = 100.0
        self._analyzer = None          # created on the first updateStats, on that tensor's device
        self._is_encoding_valid = False

    # ------------------------------------------------------------------------------------------------ statistics
    def resetEncodingStats(self):
        self._is_encoding_valid = False
        if self._analyzer is not None:
            self._analyzer.reset()

    def updateStats(self, input: torch.Tensor, use_cuda: bool = True):  # pylint: disable=redefined-builtin
        self._check_gpu(input, use_cuda)
        if self._analyzer is None or self._analyzer.device != input.device:
            self._analyzer = ops.Analyzer(_MODE_TO_MIQ[self._scheme], input.device)
            self._analyzer.set_percentile(self._percentile)
        self._is_encoding_valid = True
        self._analyzer.update_stats(input)

    def getEncoding(self, bitwidth: int, useSymmetricEncodings: bool, useStrictSymmetric: bool,
                    useUnsignedSymmetric: bool) -> Tuple[TfEncoding, bool]:
        if not self._is_encoding_valid or self._analyzer is None:
            return TfEncoding(), False
        enc, valid = self._analyzer.compute_encoding(bitwidth, useSymmetricEncodings, useStrictSymmetric,
                                                     useUnsignedSymmetric)
        return _to_tf_encoding(enc), bool(valid)

    def queueEncoding(self, bitwidth: int, useSymmetricEncodings: bool, useStrictSymmetric: bool,
                      useUnsignedSymmetric: bool) -> None:
        """Start the device work of the next getEncoding call with the same arguments; does not wait."""
        if self._is_encoding_valid and self._analyzer is not None:
            self._analyzer.queue_encoding(bitwidth, useSymmetricEncodings, useStrictSymmetric, useUnsignedSymmetric)

    def getStatsHistogram(self) -> List[Tuple[float, float]]:
        if self._scheme == QuantizationMode.QUANTIZATION_TF:
            raise RuntimeError("no histogram is kept by the TF (min/max) analyzer")
        if self._analyzer is None:
            return []
        x_left, pdf = self._analyzer.get_stats_histogram()
        return list(zip(x_left.tolist(), pdf.tolist()))

    def setPercentileValue(self, percentile: float):
        """Used by the percentile scheme only; a no-op for TF / TF-Enhanced, as in the reference
        (AimetTensorQuantizer.cpp:200-207)."""
        if self._scheme == QuantizationMode.QUANTIZATION_PERCENTILE:
            self._percentile = float(percentile)
            if self._analyzer is not None:
                self._analyzer.set_percentile(self._percentile)

    # ----------------------------------------------------------------------------------------- quantize-dequantize
    @staticmethod
    def _check_gpu(tensor: torch.Tensor, use_cuda: bool):
        if not use_cuda or not tensor.is_cuda:
            raise RuntimeError("AimetTensorQuantizer (aimet_amd) computes on the GPU only: pass a GPU tensor and "
                               "use_cuda=True")

    def quantizeDequantize(self, input: torch.Tensor, encoding: TfEncoding, roundingMode,  # pylint: disable=redefined-builtin
                           use_cuda: bool = True) -> torch.Tensor:
        self._check_gpu(input, use_cuda)
        if input.dtype not in (torch.float32, torch.bfloat16):
            return ops.qdq_per_tensor(input.to(torch.float32), encoding.min, encoding.max, encoding.bw,
                                      _round_mode(roundingMode))
        return ops.qdq_per_tensor(input, encoding.min, encoding.max, encoding.bw, _round_mode(roundingMode))

    def quantize(self, input: torch.Tensor, encoding: TfEncoding, roundingMode, use_cuda: bool,  # pylint: disable=redefined-builtin
                 shiftToSigned: bool) -> torch.Tensor:
        self._check_gpu(input, use_cuda)
        return ops.quantize_per_tensor(input, encoding.min, encoding.max, encoding.bw, shiftToSigned,
                                       _round_mode(roundingMode))

    @staticmethod
    def makeDeltaOffsetTensor(device, encodings: List[TfEncoding]) -> Tuple[torch.Tensor, torch.Tensor]:
        t = torch.tensor([[e.delta for e in encodings], [e.offset for e in encodings]], dtype=torch.float32)
        t = t.to(device)
        return t[0], t[1]

    @staticmethod
    def channelParams(device, encodings: List[TfEncoding]):
        """(min, max, delta, offset) float32 device vectors, derived on the device from the encodings' min/max with
        the reference's float32 recipe (AimetTensorQuantizer.cpp:209-227, 268-297)."""
        mm = torch.tensor([[e.min for e in encodings], [e.max for e in encodings]], dtype=torch.float64)
        mm = mm.to(torch.float32).to(device)
        num_steps = 2.0 ** encodings[0].bw - 1
        if encodings[0].min == -encodings[0].max:
            num_steps -= 1
        return ops.per_channel_params(mm[0], mm[1], num_steps)

    def quantizeDequantizePerChannel(self, input: torch.Tensor, encodings: List[TfEncoding],  # pylint: disable=redefined-builtin
                                     numChannel: int, numElement: int, numElementPerChannel: int, roundingMode,
                                     useCuda: bool = True) -> torch.Tensor:
        self._check_gpu(input, useCuda)
        if input.numel() != numElement:
            raise RuntimeError(f"numElement ({numElement}) does not match the tensor ({input.numel()} elements)")
        mn, mx, delta, offset = self.channelParams(input.device, encodings)
        if input.dtype not in (torch.float32, torch.bfloat16):
            input = input.to(torch.float32)
        return ops.qdq_per_channel(input, numChannel, numElementPerChannel, mn, mx, delta, offset,
                                   _round_mode(roundingMode))
