"""Small helpers shared by the v2 modules (TrainingExtensions/torch/src/python/aimet_torch/v2/utils.py:46-204)."""
import contextlib
import functools
from typing import Any, Callable, Tuple

import torch


def _is_expandable(src_shape: Tuple[int, ...], target_shape: Tuple[int, ...]) -> bool:
    """True if src_shape can be expanded (numpy-style broadcast) to target_shape."""
    if len(src_shape) > len(target_shape):
        return False
    for src_dim, dst_dim in zip(src_shape[::-1], target_shape[::-1]):
        if src_dim not in (1, dst_dim):
            return False
    return True


class StatisticsNotFoundError(RuntimeError):
    """Raised when compute_encodings() is invoked without statistics."""


class _ContextManager:
    def __init__(self, action: Callable[[], Any], cleanup: Callable[[], Any]):
        self._action, self._cleanup = action, cleanup

    def __enter__(self):
        self._action()
        return self

    def __exit__(self, *_):
        self._cleanup()

    def __call__(self, fn: Callable):
        @functools.wraps(fn)
        def wrapper(*args, **kwargs):
            with self:
                return fn(*args, **kwargs)
        return wrapper


@contextlib.contextmanager
def patch_attr(obj, attr_name, new_attr):
    """Temporarily replace obj.attr_name."""
    if isinstance(obj, torch.nn.Module):
        # bypass nn.Module.__setattr__ type checks for parameters being replaced by plain tensors
        had, old = attr_name in obj.__dict__, obj.__dict__.get(attr_name)
        obj.__dict__[attr_name] = new_attr
        try:
            yield
        finally:
            if had:
                obj.__dict__[attr_name] = old
            else:
                del obj.__dict__[attr_name]
        return
    old = getattr(obj, attr_name)
    setattr(obj, attr_name, new_attr)
    try:
        yield
    finally:
        setattr(obj, attr_name, old)


class _RoundSte(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x):  # pylint: disable=arguments-differ
        return torch.round(x)

    @staticmethod
    def backward(ctx, grad):  # pylint: disable=arguments-differ
        return grad


def ste_round(x):
    """Rounding (half to even) with a straight-through gradient."""
    return _RoundSte.apply(x)
