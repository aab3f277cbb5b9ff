"""AffineEncoding: the value object a v2 affine quantizer hands out -- scale, offset and the integer grid [qmin, qmax]
(aimet_torch/v2/quantization/affine/encoding.py:55-283; the grid rules are those of affine/_utils.py:89-188).
quantize() / dequantize() run the library's kernels through the affine backend functions."""
import math
from typing import Optional, Tuple

import torch

from .backends import _derive_qmin_qmax, dequantize, quantize

__all__ = ['AffineEncoding']


class _GridMixin:
    """bitwidth / signed as views of (qmin, qmax).  Both are defined for the two regular grids, [0, 2^B - 1] and
    [-2^(B-1), 2^(B-1) - 1], and raise for any other."""
    qmin: int
    qmax: int

    def _grid_is_regular(self) -> bool:
        return self.qmin + self.qmax == -1 or self.qmin == 0

    def _undefined(self, what: str):
        return RuntimeError(f"{what} is undefined for a quantization grid of [{self.qmin}, {self.qmax}]")

    @property
    def bitwidth(self) -> int:
        if self._grid_is_regular():
            bitwidth = math.log2(self.qmax - self.qmin + 1)
            if bitwidth == int(bitwidth):
                return int(bitwidth)
        raise self._undefined("bitwidth")

    @bitwidth.setter
    def bitwidth(self, bitwidth: int):
        if bitwidth == int(bitwidth):
            bitwidth = int(bitwidth)
        if not isinstance(bitwidth, int):
            raise TypeError(f"Setting bitwidth to a non-integer value {bitwidth:.3f} is not supported; set "
                            f"{type(self).__qualname__}.qmin and .qmax instead.")
        if bitwidth < 1:
            raise ValueError(f"Bitwidth can't be smaller than 1. Got {bitwidth}")
        if self.qmin + self.qmax == -1:
            self.qmin, self.qmax = -2 ** (bitwidth - 1), 2 ** (bitwidth - 1) - 1
        elif self.qmin == 0:
            self.qmin, self.qmax = 0, 2 ** bitwidth - 1
        else:
            raise self._undefined("bitwidth")

    @property
    def signed(self) -> bool:
        if self._grid_is_regular():
            return self.qmin < 0 <= self.qmax
        raise self._undefined("signed")

    @signed.setter
    def signed(self, signed: bool):
        bitwidth = self.bitwidth
        if signed:
            self.qmin, self.qmax = -2 ** (bitwidth - 1), 2 ** (bitwidth - 1) - 1
        else:
            self.qmin, self.qmax = 0, 2 ** bitwidth - 1


def _destination(args, kwargs, current: torch.Tensor):
    """(device, dtype) a Tensor.to()-style call asks for; what it does not name stays as `current` has it."""
    device, dtype = kwargs.get('device'), kwargs.get('dtype')
    for arg in args:
        if isinstance(arg, torch.dtype):
            dtype = arg
        elif isinstance(arg, torch.Tensor):
            device, dtype = arg.device, arg.dtype
        elif isinstance(arg, (str, int, torch.device)):
            device = arg
    device = current.device if device is None else torch.device(device)
    return device, (current.dtype if dtype is None else dtype)


class AffineEncoding(_GridMixin):
    """AffineEncoding(scale, offset, qmin, qmax, symmetry=False, block_size=None) or
    AffineEncoding(scale, offset, bitwidth, signed=False, symmetry=False, block_size=None).

    A bool (or nothing) in the place of qmax / signed means the bitwidth form."""

    def __init__(self, scale: torch.Tensor, offset: torch.Tensor, *args, **kwargs):
        slots = list(args[:4]) + [None] * max(0, 4 - len(args))
        for position, names in enumerate((('qmin', 'bitwidth'), ('qmax', 'signed'), ('symmetry',), ('block_size',))):
            for name in names:
                if name in kwargs:
                    slots[position] = kwargs.pop(name)
        if kwargs:
            raise TypeError(f"{type(self).__qualname__}.__init__ got unexpected keyword argument: "
                            f"{', '.join(kwargs)}")
        first, second, symmetry, block_size = slots
        if first is None:
            raise TypeError(f"{type(self).__qualname__}.__init__ needs (qmin, qmax) or (bitwidth[, signed]); "
                            f"got {args}")
        if second is None or isinstance(second, bool):
            qmin, qmax = _derive_qmin_qmax(bitwidth=first, signed=bool(second))
        else:
            qmin, qmax = first, second
        if qmin >= qmax:
            raise ValueError(f"qmax should be strictly larger than qmin. Got qmax={qmax}, qmin={qmin}")
        self._scale, self._offset = scale, offset
        self.qmin, self.qmax = qmin, qmax
        self._symmetry = bool(symmetry)
        self._block_size = block_size

    @classmethod
    def _on_grid(cls, scale, offset, qmin, qmax, symmetry, block_size):
        """The quantizers' own constructor (once per forward pass and quantizer): the arguments are known to be a
        grid, nothing is parsed or checked."""
        self = object.__new__(cls)
        self._scale, self._offset, self.qmin, self.qmax = scale, offset, qmin, qmax
        self._symmetry, self._block_size = symmetry, block_size
        return self

    # --------------------------------------------------------------------------------------------------- description
    mapping = "affine"

    @property
    def granularity(self) -> str:
        if self._scale.dim() == 0:
            return "pertensor"
        if self._block_size is not None:
            return "blockwise"
        return "perchannel" if sum(1 for d in self._scale.shape if d > 1) <= 1 else "unknown"

    @property
    def scale(self) -> torch.Tensor:
        return self._scale

    @property
    def offset(self) -> torch.Tensor:
        return self._offset

    @property
    def num_steps(self) -> int:
        return self.qmax - self.qmin

    @property
    def min(self) -> torch.Tensor:
        return (self._offset + self.qmin) * self._scale

    @property
    def max(self) -> torch.Tensor:
        return (self._offset + self.qmax) * self._scale

    @property
    def symmetry(self) -> bool:
        return self._symmetry

    @property
    def block_size(self) -> Optional[Tuple[int, ...]]:
        return self._block_size

    @property
    def dtype(self) -> torch.dtype:
        """The smallest integer type that holds the grid."""
        for dtype, low, high in ((torch.uint8, 0, 255), (torch.int8, -128, 127), (torch.int16, -32768, 32767)):
            if low <= self.qmin and self.qmax <= high:
                return dtype
        return torch.int32

    # --------------------------------------------------------------------------------------------------- conversion
    def to(self, *args, **kwargs):
        """As Tensor.to(): an encoding whose scale and offset live on the given device / in the given floating-point
        type; this object itself when nothing changes."""
        device, dtype = _destination(args, kwargs, self._scale)
        if dtype == self._scale.dtype and device == self._scale.device:
            return self
        if not dtype.is_floating_point:
            raise RuntimeError(f"Cannot change encoding data dtype to {dtype}, only floating point data types are "
                               "supported")
        return type(self)(self._scale.to(device=device, dtype=dtype), self._offset.to(device=device, dtype=dtype),
                          self.qmin, self.qmax, self._symmetry, self._block_size)

    def quantize(self, input: torch.Tensor) -> torch.Tensor:  # pylint: disable=redefined-builtin
        """clamp(round(input / scale) - offset, qmin, qmax), in input's type"""
        return quantize(input, self._scale.to(input.dtype), self._offset.to(input.dtype), self.qmin, self.qmax,
                        block_size=self._block_size)

    def dequantize(self, input: torch.Tensor) -> torch.Tensor:  # pylint: disable=redefined-builtin
        """(input + offset) * scale"""
        return dequantize(input, self._scale.to(input.dtype), self._offset.to(input.dtype),
                          block_size=self._block_size)
