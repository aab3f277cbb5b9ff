"""Small helpers shared by the v2 modules (TrainingExtensions/torch/src/python/aimet_torch/v2/utils.py:46-204)."""
import contextlib
import functools
import math
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


def channel_view(tensor: torch.Tensor, param_shape: Tuple[int, ...]):
    """Lays `tensor` out as [outer, num_channel, n_per_channel] so that every [n_per_channel] run shares the element
    of a parameter of shape `param_shape` (numpy-style broadcastable to the tensor) it is quantized with, channels in
    the parameter's row-major order.

    Returns (tensor3, perm).  When the axes along which the parameter varies are adjacent in memory this is a plain
    reshape (perm None): per-tensor, per-channel along one axis, and blocks that cut only the last varying axis
    (e.g. a Linear weight [out, in] with scale [out, in / block]).  Otherwise the varying axes are moved to the front
    with one permuted copy; `perm` is then the permutation that channel_view_restore undoes."""
    shape = tuple(tensor.shape)
    padded = (1,) * (len(shape) - len(param_shape)) + tuple(param_shape)
    varying = [a for a, p in enumerate(padded) if p != 1]
    if not varying:
        return tensor.reshape(1, 1, tensor.numel()), None
    first, last = varying[0], varying[-1]
    num_channel = math.prod(padded)
    if all(padded[a] == shape[a] for a in range(first, last + 1)):
        return tensor.reshape(math.prod(shape[:first]), num_channel, math.prod(shape[last + 1:])), None
    shared = [a for a in range(len(shape)) if a not in varying]
    perm = varying + shared
    return tensor.permute(perm).reshape(1, num_channel, math.prod(shape[a] for a in shared)), perm


def channel_view_restore(tensor3: torch.Tensor, shape: Tuple[int, ...], perm) -> torch.Tensor:
    """Inverse of channel_view for a result of the same layout."""
    if perm is None:
        return tensor3.reshape(shape)
    inverse = [0] * len(perm)
    for i, a in enumerate(perm):
        inverse[a] = i
    return tensor3.reshape([shape[a] for a in perm]).permute(inverse).contiguous()


def reshape_tensor_for_blocks(tensor: torch.Tensor, encoding_shape, block_size) -> torch.Tensor:
    """Splits each of the last len(block_size) axes into (number of blocks, block length); -1 means "derive the
    block length from the shapes" (reference torch_builtins.py:364-399)."""
    if block_size is None:
        return tensor
    nb = len(block_size)
    split = []
    for axis in range(nb):
        dim, blocks = tensor.shape[tensor.dim() - nb + axis], encoding_shape[axis]
        split += [blocks, dim // blocks if block_size[axis] == -1 else block_size[axis]]
    return tensor.reshape(list(tensor.shape[:tensor.dim() - nb]) + split)


def get_encoding_shape_with_blocks(encoding_shape, block_size):
    """Parameter shape that broadcasts against reshape_tensor_for_blocks' result: a 1 after every axis (reference
    torch_builtins.py:347-362)."""
    if block_size is None:
        return tuple(encoding_shape)
    out = []
    for d in encoding_shape:
        out += [d, 1]
    return tuple(out)


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


def _remove_from_qmodules(modules, kind: str):
    """Calls `_remove_<kind>_quantizers()` on every quantized module under `modules` (a module or several); the result
    puts all of them back when used as a context manager (reference v2/utils.py:283-344)."""
    from .nn.base import BaseQuantizationMixin                      # pylint: disable=import-outside-toplevel
    if isinstance(modules, torch.nn.Module):
        modules = (modules,)
    undo = []

    def put_back():
        while undo:
            undo.pop()._cleanup()                                   # pylint: disable=protected-access
    try:
        for root in modules:
            for module in root.modules():
                if isinstance(module, BaseQuantizationMixin):
                    undo.append(getattr(module, f"_remove_{kind}_quantizers")())
    except Exception:
        put_back()
        raise
    return _ContextManager(action=lambda: None, cleanup=put_back)


def remove_input_quantizers(modules):
    """Takes the input quantizers out of the quantized modules given."""
    return _remove_from_qmodules(modules, "input")


def remove_output_quantizers(modules):
    """Takes the output quantizers out of the quantized modules given."""
    return _remove_from_qmodules(modules, "output")


def remove_param_quantizers(modules):
    """Takes the parameter quantizers out of the quantized modules given."""
    return _remove_from_qmodules(modules, "param")


def remove_activation_quantizers(modules):
    """Takes the input and output quantizers out of the quantized modules given."""
    return _remove_from_qmodules(modules, "activation")


def remove_all_quantizers(modules):
    """Takes every quantizer out of the quantized modules given."""
    return _remove_from_qmodules(modules, "all")
