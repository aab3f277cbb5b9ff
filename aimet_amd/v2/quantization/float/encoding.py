"""What a float quantizer's get_encoding() returns: the format and, when statistics set it, the largest representable
value (interface of aimet_torch/v2/quantization/float/encoding.py:48-125)."""
import dataclasses
from typing import Optional

import torch


@dataclasses.dataclass(frozen=True)
class FloatEncoding:
    """Immutable record; `maxval` is None when the format's own largest value applies."""
    mantissa_bits: int
    exponent_bits: int
    maxval: Optional[torch.Tensor] = None
    mapping: str = dataclasses.field(default="float", init=False)

    @property
    def bitwidth(self) -> int:
        """sign + exponent + mantissa"""
        return 1 + self.exponent_bits + self.mantissa_bits

    @property
    def granularity(self) -> str:
        """'pertensor', 'perchannel' (maxval varies along exactly one axis) or 'unknown'"""
        varying = 0 if self.maxval is None else sum(size > 1 for size in self.maxval.shape)
        return ("pertensor", "perchannel")[varying] if varying < 2 else "unknown"

    def to(self, *args, **kwargs) -> "FloatEncoding":
        """The same encoding with maxval moved / cast as torch.Tensor.to would."""
        if self.maxval is None:
            return self
        return dataclasses.replace(self, maxval=self.maxval.to(*args, **kwargs))
