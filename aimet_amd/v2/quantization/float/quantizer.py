"""v2 float quantizer: the input rounded to the grid of a narrow float format.

Mirrors TrainingExtensions/torch/src/python/aimet_torch/v2/quantization/float/quantizer.py:77-334
(FloatQuantizeDequantize): a format is given as a torch dtype (float16 / bfloat16) or as exponent and mantissa bits;
without an encoding analyzer its largest value is the format's own (:56-59), and float16 / bfloat16 are then a cast
there and back (:309-314); with an analyzer the largest value follows the observed |input| maximum (compute_encodings,
:253-300) and the grid's exponent bias with it (aimet_torch/fp_quantization.py:171-209).  The arithmetic runs in the HIP
kernels (aimet_amd.ops.float_fake_cast / fp16_round_trip / bf16_round_trip).
"""
import contextlib
import functools
import math
from typing import Dict, List, Optional

import numpy as np
import torch

from .... import ops
from ...utils import StatisticsNotFoundError, patch_attr
from ..affine.quantizer import _flag_extreme_min_max
from ..base import QuantizerBase
from ..encoding_analyzer import EncodingAnalyzer
from .encoding import FloatEncoding

__all__ = ['QuantizeDequantize', 'FloatQuantizeDequantize']

_FLOAT16 = (5, 10)     # exponent, mantissa bits
_BFLOAT16 = (8, 7)


def _ieee_float_max_representable_value(exponent_bits, mantissa_bits):
    """(2 - 2^-M) * 2^(floor(exponent_max / 2)), exponent_max = 2^E - 1 (reference :56-59)"""
    exponent_max = 2 ** exponent_bits - 1
    exponent_bias = exponent_max // 2
    return (2 - 2 ** -mantissa_bits) * 2 ** (exponent_max - exponent_bias - 1)


assert _ieee_float_max_representable_value(*_FLOAT16) == torch.finfo(torch.float16).max
assert _ieee_float_max_representable_value(*_BFLOAT16) == torch.finfo(torch.bfloat16).max


class _FakeCast(torch.autograd.Function):
    """Forward through the kernels.  Backward as autograd differentiates the reference's expressions: a cast to
    float16 / bfloat16 and back passes the gradient on, round(x / step) * step has none."""

    @staticmethod
    def forward(ctx, x, run, passes_gradient):  # pylint: disable=arguments-differ
        ctx.passes_gradient = passes_gradient
        return run(x)

    @staticmethod
    def backward(ctx, grad):  # pylint: disable=arguments-differ
        return (grad if ctx.passes_gradient else torch.zeros_like(grad)), None, None


class FloatQuantizeDequantize(QuantizerBase):
    """out = input rounded to the nearest value of a float format with `exponent_bits` and `mantissa_bits`.

    Unlike the affine quantizers it needs no calibration: is_initialized() is always True.  With an
    `encoding_analyzer`, compute_encodings() moves the format's largest value to the observed maximum of |input|
    (one per entry of the analyzer's shape)."""

    def __init__(self, exponent_bits: int = None, mantissa_bits: int = None, dtype: torch.dtype = None,
                 encoding_analyzer: EncodingAnalyzer = None):
        super().__init__()
        if dtype is None:
            if exponent_bits is None or mantissa_bits is None:
                raise ValueError('Neither "dtype" nor "exponent/mantissa_bits" was specified.')
        else:
            if exponent_bits is not None or mantissa_bits is not None:
                raise ValueError('Argument "dtype" is mutually exclusive with "exponent/mantissa_bits".')
            if dtype not in (torch.float16, torch.bfloat16):
                raise ValueError(f"Float quantizer only supports torch.float16 and torch.bfloat16. Got {dtype}.")
            exponent_bits, mantissa_bits = _FLOAT16 if dtype == torch.float16 else _BFLOAT16
        self.exponent_bits = exponent_bits
        self.mantissa_bits = mantissa_bits
        self.encoding_analyzer = encoding_analyzer
        self._allow_overwrite = True
        self._grid = None   # (key, grid tensors) of the last forward
        if encoding_analyzer is not None:
            largest = _ieee_float_max_representable_value(exponent_bits, mantissa_bits)
            self.register_buffer('maxval', torch.full(tuple(encoding_analyzer.observer.shape), float(largest)))
        else:
            self.register_buffer('maxval', None)

    # ------------------------------------------------------------------------------------------------ properties
    @property
    def bitwidth(self) -> int:
        return self.exponent_bits + self.mantissa_bits + 1

    def is_float16(self) -> bool:
        return (self.exponent_bits, self.mantissa_bits) == _FLOAT16

    def is_bfloat16(self) -> bool:
        return (self.exponent_bits, self.mantissa_bits) == _BFLOAT16

    def is_initialized(self) -> bool:  # pylint: disable=no-self-use
        return True

    def allow_overwrite(self, mode: bool):
        """With False, compute_encodings() leaves maxval alone."""
        self._allow_overwrite = mode

    def extra_repr(self) -> str:
        return f'exponent_bits={self.exponent_bits}, mantissa_bits={self.mantissa_bits}'

    # ------------------------------------------------------------------------------------------------ persistence
    def get_extra_state(self):
        return {'exponent_bits': torch.tensor(self.exponent_bits), 'mantissa_bits': torch.tensor(self.mantissa_bits)}

    def set_extra_state(self, state):
        self.exponent_bits = int(state['exponent_bits'])
        self.mantissa_bits = int(state['mantissa_bits'])
        self._grid = None

    def load_state_dict(self, state_dict, strict: bool = True):  # pylint: disable=arguments-differ
        # a state with maxval turns this quantizer into one with maxval, a state without into one without
        # (reference :179-190)
        if 'maxval' in state_dict:
            if self.maxval is None:
                del self.maxval
                self.register_buffer('maxval', state_dict['maxval'].clone())
        elif self.maxval is not None:
            del self.maxval
            self.register_buffer('maxval', None)
        self._grid = None
        return super().load_state_dict(state_dict, strict)

    def get_legacy_encodings(self) -> Optional[List[Dict]]:
        return [{'bitwidth': self.bitwidth, 'dtype': 'float'}]

    def set_legacy_encodings(self, encodings: List[Dict]):
        if encodings[0]['bitwidth'] != 16:
            raise RuntimeError(f"{self.__class__} can only import 16-bit legay encodings.")
        self.exponent_bits, self.mantissa_bits = _FLOAT16
        self._grid = None

    def get_encoding(self) -> Optional[FloatEncoding]:
        return FloatEncoding(self.mantissa_bits, self.exponent_bits, self.maxval)

    # ------------------------------------------------------------------------------------------------ calibration
    @contextlib.contextmanager
    def compute_encodings(self):
        """Observe |input| and set maxval from it on exit; while inside, forward uses the batch's own maximum
        (reference :253-300)."""
        if self.encoding_analyzer is None or not self._allow_overwrite:
            yield
            return
        original_forward = self.forward
        num_steps = math.pow(2, self.bitwidth) - 1

        def absmax_of(lo, hi):
            return torch.maximum(lo.abs(), hi.abs()).to(dtype=self.maxval.dtype,
                                                        device=self.maxval.device).expand_as(self.maxval)

        @functools.wraps(original_forward)
        def forward_wrapper(input):  # pylint: disable=redefined-builtin
            statistics = self.encoding_analyzer.update_stats(input)
            lo, hi = self.encoding_analyzer.compute_encodings_from_stats(statistics, num_steps, False)
            with patch_attr(self, 'maxval', absmax_of(lo, hi)):
                return original_forward(input)

        self.encoding_analyzer.reset_stats()
        with patch_attr(self, 'forward', forward_wrapper):
            yield
        try:
            lo, hi = self.encoding_analyzer.compute_encodings(num_steps, False)
        except StatisticsNotFoundError:
            return
        if lo is None or hi is None:
            return
        _flag_extreme_min_max(lo, hi)
        with torch.no_grad():
            self.maxval.copy_(absmax_of(lo, hi))

    # --------------------------------------------------------------------------------------------------- forward
    def _varying_axis(self, input):  # pylint: disable=redefined-builtin
        """Axis of `input` along which maxval varies (maxval broadcasts against input from the right)."""
        shape = tuple(self.maxval.shape)
        if len(shape) > input.dim():
            raise RuntimeError(f"maxval of shape {shape} does not broadcast against an input of shape "
                               f"{tuple(input.shape)}")
        varying = [axis for axis, size in enumerate(shape) if size > 1]
        if len(varying) != 1:
            raise NotImplementedError("the largest value may vary along one axis of the input only")
        axis = varying[0] + input.dim() - len(shape)
        if input.shape[axis] != shape[varying[0]]:
            raise RuntimeError(f"maxval of shape {shape} does not broadcast against an input of shape "
                               f"{tuple(input.shape)}")
        return axis

    def _fake_cast(self, x):
        """x: float32 GPU tensor"""
        maxval = self.maxval
        exponent_bits, mantissa_bits = self.exponent_bits, self.mantissa_bits
        if maxval is None:
            # the format's own largest value: every constant of the expression is a Python float, so the bias is a
            # float64 that meets the tensor rounded to float32 once
            largest = _ieee_float_max_representable_value(exponent_bits, mantissa_bits)
            key = (x.device, exponent_bits, mantissa_bits)
            if self._grid is None or self._grid[0] != key:
                bias = 2 ** exponent_bits - np.log2(largest) + np.log2(2 - 2 ** (-mantissa_bits)) - 1
                grid = ops.float_grid(torch.tensor([largest], dtype=torch.float32, device=x.device), exponent_bits,
                                      mantissa_bits, host_bias=bias)
                self._grid = (key, grid)
            return ops.float_fake_cast(x, None, exponent_bits, mantissa_bits, 0, grid=self._grid[1])
        axis = 0 if maxval.numel() == 1 else self._varying_axis(x)
        key = (x.device, exponent_bits, mantissa_bits, maxval.data_ptr(), maxval._version)  # pylint: disable=protected-access
        if self._grid is None or self._grid[0] != key:
            self._grid = (key, ops.float_grid(maxval.to(x.device), exponent_bits, mantissa_bits, host_constants=True))
        return ops.float_fake_cast(x, None, exponent_bits, mantissa_bits, axis, grid=self._grid[1])

    def forward(self, input: torch.Tensor) -> torch.Tensor:  # pylint: disable=redefined-builtin
        if not input.is_cuda:
            raise RuntimeError("aimet_amd computes on the GPU only: pass a GPU tensor")
        cast_only = self.maxval is None and (self.is_float16() or self.is_bfloat16())
        if cast_only:
            kernel = ops.fp16_round_trip if self.is_float16() else ops.bf16_round_trip
        else:
            kernel = self._fake_cast

        def run(x):
            return kernel(x.detach().to(torch.float32)).to(x.dtype)

        if torch.is_grad_enabled() and input.requires_grad:
            return _FakeCast.apply(input, run, cast_only)
        return run(input)


class QuantizeDequantize(FloatQuantizeDequantize):
    """Alias of FloatQuantizeDequantize (reference :330-334)."""
