"""What every v2 quantizer module is (aimet_torch/v2/quantization/base/quantizer.py:59-230): a module that can observe
what passes through it inside compute_encodings(), hand its encodings out and take them back in the exported format,
and be frozen against later calibration."""
import contextlib
from typing import Dict, List, Optional

from torch import nn


class QuantizerBase(nn.Module):
    """Base of the affine and float quantizers; isinstance(module, QuantizerBase) finds the quantizers of a model."""

    def __init__(self):
        super().__init__()
        self._allow_overwrite = True

    def allow_overwrite(self, mode: bool):
        """With False, compute_encodings() and encoding imports leave the current parameters alone."""
        self._allow_overwrite = mode

    @contextlib.contextmanager
    def compute_encodings(self):
        raise NotImplementedError
        yield                                                           # pylint: disable=unreachable

    def is_initialized(self) -> bool:
        raise NotImplementedError

    def get_encoding(self):
        raise NotImplementedError

    def get_legacy_encodings(self) -> Optional[List[Dict]]:
        raise NotImplementedError

    def set_legacy_encodings(self, encodings: List[Dict]):
        raise NotImplementedError
