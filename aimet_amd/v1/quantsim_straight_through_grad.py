"""Straight-through-estimator gradient of the v1 path.

compute_dloss_by_dx mirrors TrainingExtensions/torch/src/python/aimet_torch/v1/quantsim_straight_through_grad.py:91-118:
grad * ((encoding_min <= x) & (x <= encoding_max)), one fused kernel instead of three elementwise passes and a bool
temporary.
"""
import functools

import torch

from .. import ops


def broadcast_to_tensor(tensor, encoding, ch_axis):
    """1-d per-channel encoding values -> shape broadcastable against `tensor` (reference :66-88)."""
    if not isinstance(encoding, torch.Tensor):
        encoding = torch.tensor(encoding).to(tensor.device)
    assert len(encoding.shape) <= 1
    if encoding.numel() == 1:
        return encoding
    assert encoding.numel() == tensor.shape[ch_axis]
    shape = tuple(dim if axis == ch_axis else 1 for axis, dim in enumerate(tensor.shape))
    return encoding.view(shape)


def compute_dloss_by_dx(x, grad, encoding_min, encoding_max, ch_axis=0):
    """dL/dx = grad where encoding_min <= x <= encoding_max (both ends inclusive), 0 elsewhere.

    encoding_min / encoding_max: python floats (per-tensor), or sequences / 1-d tensors with one value per channel
    along `ch_axis`.
    """
    per_channel = isinstance(encoding_min, (list, tuple)) or \
        (isinstance(encoding_min, torch.Tensor) and encoding_min.numel() > 1)
    if not per_channel:
        mn = float(encoding_min[0] if isinstance(encoding_min, (list, tuple, torch.Tensor)) else encoding_min)
        mx = float(encoding_max[0] if isinstance(encoding_max, (list, tuple, torch.Tensor)) else encoding_max)
        if x.dtype != torch.float32:
            # the reference compares against a 0-dim tensor, which torch's type promotion casts to x's dtype
            mn = float(torch.tensor(mn, dtype=torch.float32).to(x.dtype))
            mx = float(torch.tensor(mx, dtype=torch.float32).to(x.dtype))
        return ops.ste_bwd_per_tensor(x, grad, mn, mx)
    mn = torch.as_tensor(encoding_min, dtype=torch.float32).to(x.device)
    mx = torch.as_tensor(encoding_max, dtype=torch.float32).to(x.device)
    num_channel = x.shape[ch_axis]
    assert mn.numel() == num_channel and mx.numel() == num_channel
    n_per_channel = functools.reduce(lambda a, b: a * b, x.shape[ch_axis + 1:], 1)
    return ops.ste_bwd_per_channel(x, grad, num_channel, n_per_channel, mn, mx)
