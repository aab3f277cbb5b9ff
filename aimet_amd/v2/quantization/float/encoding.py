"""What a float quantizer's get_encoding() returns (aimet_torch/v2/quantization/float/encoding.py:48-125)."""
from typing import Optional

import torch


class FloatEncoding:
    """Mantissa bits, exponent bits and the largest representable value (None: the format's own)."""

    def __init__(self, mantissa_bits: int, exponent_bits: int, maxval: Optional[torch.Tensor]):
        self._mantissa_bits = mantissa_bits
        self._exponent_bits = exponent_bits
        self._maxval = maxval

    mapping = "float"

    @property
    def mantissa_bits(self) -> int:
        return self._mantissa_bits

    @property
    def exponent_bits(self) -> int:
        return self._exponent_bits

    @property
    def maxval(self) -> Optional[torch.Tensor]:
        return self._maxval

    @property
    def bitwidth(self) -> int:
        return self._mantissa_bits + self._exponent_bits + 1

    @property
    def granularity(self) -> str:
        if self._maxval is None or self._maxval.numel() == 1:
            return "pertensor"
        if sum(1 for d in self._maxval.shape if d > 1) == 1:
            return "perchannel"
        return "unknown"

    def to(self, *args, **kwargs):
        maxval = None if self._maxval is None else self._maxval.to(*args, **kwargs)
        return type(self)(self._mantissa_bits, self._exponent_bits, maxval)
