"""Encoding analyzers of the v2 path.

MinMaxEncodingAnalyzer mirrors TrainingExtensions/torch/src/python/aimet_torch/v2/quantization/encoding_analyzer.py:
_MinMaxObserver (:91-129), EncodingAnalyzer (:272-319) and MinMaxEncodingAnalyzer (:325-386): same methods
(update_stats, reset_stats, compute_encodings, compute_encodings_from_stats, compute_dynamic_encodings) and
``observer.shape``.  Statistics are collected by the fused min/max kernels (one pass for min and max together;
per-channel shapes in one launch) instead of two torch reductions over a permuted copy.
"""
import math
from dataclasses import dataclass
from typing import Optional, Tuple

import torch

from ... import ops
from ..utils import StatisticsNotFoundError, _is_expandable


@dataclass
class _MinMaxRange:
    min: Optional[torch.Tensor] = None
    max: Optional[torch.Tensor] = None


_MINIMUM_SCALE = torch.finfo(torch.float32).eps


class _MinMaxObserver:
    """Running minimum / maximum reduced to `shape`."""

    def __init__(self, shape: tuple):
        self.shape = (shape,) if isinstance(shape, int) else tuple(shape)
        self.stats = _MinMaxRange()

    @torch.no_grad()
    def collect_stats(self, input_tensor: torch.Tensor) -> _MinMaxRange:
        if not _is_expandable(self.shape, input_tensor.shape):
            raise RuntimeError(f"Input of shape {list(input_tensor.shape)} can't be reduced to shape "
                               f"{list(self.shape)}")
        padded = (1,) * (input_tensor.dim() - len(self.shape)) + self.shape
        axes = [a for a, d in enumerate(padded) if d != 1]
        if not axes:
            mm = ops.minmax(input_tensor)
            return _MinMaxRange(mm[0].reshape(self.shape).to(input_tensor.dtype),
                                mm[1].reshape(self.shape).to(input_tensor.dtype))
        if len(axes) > 1:
            raise RuntimeError(f"observer shape {self.shape} varies along more than one axis: not implemented")
        axis = axes[0]
        n_per_channel = math.prod(input_tensor.shape[axis + 1:])
        mm = ops.minmax_per_channel(input_tensor, input_tensor.shape[axis], n_per_channel)
        return _MinMaxRange(mm[0].reshape(self.shape).to(input_tensor.dtype),
                            mm[1].reshape(self.shape).to(input_tensor.dtype))

    @torch.no_grad()
    def merge_stats(self, stats: _MinMaxRange):
        new_min, new_max = self.stats.min, self.stats.max
        if stats.min is not None:
            new_min = stats.min.clone() if new_min is None else torch.minimum(new_min, stats.min)
        if stats.max is not None:
            new_max = stats.max.clone() if new_max is None else torch.maximum(new_max, stats.max)
        self.stats = _MinMaxRange(new_min, new_max)

    def reset_stats(self):
        self.stats = _MinMaxRange()

    def get_stats(self) -> _MinMaxRange:
        return self.stats


class EncodingAnalyzer:
    """Gathers statistics of input data and computes encodings."""

    def __init__(self, observer):
        self.observer = observer

    @torch.no_grad()
    def update_stats(self, input_tensor: torch.Tensor):
        new_stats = self.observer.collect_stats(input_tensor)
        self.observer.merge_stats(new_stats)
        return new_stats

    def reset_stats(self):
        self.observer.reset_stats()

    def compute_encodings(self, num_steps: int, is_symmetric: bool):
        return self.compute_encodings_from_stats(self.observer.get_stats(), num_steps, is_symmetric)

    def compute_dynamic_encodings(self, input_tensor: torch.Tensor, num_steps: int, is_symmetric: bool):
        return self.compute_encodings_from_stats(self.observer.collect_stats(input_tensor), num_steps, is_symmetric)

    def compute_encodings_from_stats(self, stats, num_steps: int, is_symmetric: bool):
        raise NotImplementedError


class MinMaxEncodingAnalyzer(EncodingAnalyzer):
    """Min-max calibration: the range is [min(input), max(input)], widened to contain zero."""

    def __init__(self, shape: tuple):
        super().__init__(_MinMaxObserver(shape))

    @torch.no_grad()
    def compute_encodings_from_stats(self, stats: _MinMaxRange, num_steps: int, is_symmetric: bool) \
            -> Tuple[torch.Tensor, torch.Tensor]:
        # reference :349-386, parameter-sized tensors: plain tensor arithmetic, not a hot loop
        if num_steps <= 0:
            raise ValueError('The number of quantization bins cannot be less than or equal to 0.')
        if stats.min is None or stats.max is None:
            raise StatisticsNotFoundError('No statistics present to compute encodings.')
        min_with_zero = torch.clamp(stats.min, max=0)
        max_with_zero = torch.clamp(stats.max, min=0)
        tensor_diff = (max_with_zero - min_with_zero) / num_steps
        adjustment_step = _MINIMUM_SCALE * (tensor_diff < _MINIMUM_SCALE)
        if is_symmetric:
            updated_max = max_with_zero + math.floor(num_steps / 2) * adjustment_step
            updated_min = min_with_zero - math.ceil(num_steps / 2) * adjustment_step
            num_pos_steps = math.floor(num_steps / 2)
            num_neg_steps = math.ceil(num_steps / 2)
            delta = torch.maximum(updated_max / num_pos_steps, -updated_min / num_neg_steps)
            updated_min = -1 * num_neg_steps * delta
            updated_max = num_pos_steps * delta
        else:
            updated_max = max_with_zero + num_steps * adjustment_step
            updated_min = min_with_zero
        updated_max = torch.clamp(updated_max, max=torch.finfo(stats.min.dtype).max).to(stats.min.dtype)
        updated_min = torch.clamp(updated_min, min=torch.finfo(stats.max.dtype).min).to(stats.max.dtype)
        return updated_min, updated_max
