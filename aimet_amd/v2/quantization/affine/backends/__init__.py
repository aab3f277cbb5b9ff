"""v2 affine quantization functions, dispatched to the current backend
(TrainingExtensions/torch/src/python/aimet_torch/v2/quantization/affine/backends/__init__.py:178-179, 325-370)."""
import math

from .utils import add_backend, get_backend, set_backend, set_global_backend


def quantize(tensor, scale, offset, *args, **kwargs):
    """out = clamp(round(tensor / scale) - offset, qmin, qmax).  Three call forms, as in the reference (:44-64):
    (bitwidth, signed=False, block_size=None), (*, num_steps, signed=False, block_size=None) and
    (qmin, qmax, block_size=None)."""
    qmin, qmax, block_size = _parse_args(args, kwargs)
    return get_backend().quantize(tensor, scale, offset, qmin, qmax, block_size)


def quantize_dequantize(tensor, scale, offset, *args, **kwargs):
    """out = (clamp(round(tensor / scale) - offset, qmin, qmax) + offset) * scale; call forms as for quantize."""
    qmin, qmax, block_size = _parse_args(args, kwargs)
    return get_backend().quantize_dequantize(tensor, scale, offset, qmin, qmax, block_size)


def dequantize(tensor, scale, offset, block_size=None):
    return get_backend().dequantize(tensor, scale, offset, block_size)


def _parse_args(args, kwargs):
    """(qmin, qmax, block_size) from any of the three call forms (reference :334-356)."""
    args = tuple(args) + (None,) * (3 - len(args))
    first = kwargs.get('qmin', kwargs.get('bitwidth', args[0]))
    second = kwargs.get('qmax', kwargs.get('signed', args[1]))
    block_size = kwargs.get('block_size', None) or args[2]
    if first is None:
        qmin, qmax = _derive_qmin_qmax(num_steps=kwargs['num_steps'], signed=kwargs['signed'])
    elif second is None or isinstance(second, bool):
        qmin, qmax = _derive_qmin_qmax(bitwidth=first, signed=bool(second))
    else:
        qmin, qmax = first, second
    return qmin, qmax, block_size


def _derive_qmin_qmax(*, bitwidth: int = None, num_steps: int = None, signed: bool):
    if bitwidth is not None:
        num_steps = 2 ** bitwidth - 1
    if signed:
        return -math.ceil(num_steps / 2), math.floor(num_steps / 2)
    return 0, num_steps


__all__ = ['quantize', 'quantize_dequantize', 'dequantize', 'add_backend', 'get_backend', 'set_backend',
           'set_global_backend']
