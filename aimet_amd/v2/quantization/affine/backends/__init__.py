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
    """(qmin, qmax, block_size) from any of the three call forms (reference :334-356): the first grid argument is
    qmin or the bitwidth, the second qmax or the signed flag -- a bool (or nothing) there means the bitwidth form; with
    no first argument at all the grid comes from the num_steps / signed keywords."""
    slots = list(args[:3]) + [None] * max(0, 3 - len(args))
    for position, names in enumerate((('qmin', 'bitwidth'), ('qmax', 'signed'))):
        for name in names:
            if name in kwargs:
                slots[position] = kwargs[name]
                break
    lower, upper = slots[0], slots[1]
    block_size = kwargs.get('block_size') or slots[2]
    if lower is None:
        return (*_derive_qmin_qmax(num_steps=kwargs['num_steps'], signed=kwargs['signed']), block_size)
    if upper is None or isinstance(upper, bool):
        return (*_derive_qmin_qmax(bitwidth=lower, signed=bool(upper)), block_size)
    return lower, upper, block_size


def _derive_qmin_qmax(*, bitwidth: int = None, num_steps: int = None, signed: bool):
    if bitwidth is not None:
        num_steps = 2 ** bitwidth - 1
    if signed:
        return -math.ceil(num_steps / 2), math.floor(num_steps / 2)
    return 0, num_steps


__all__ = ['quantize', 'quantize_dequantize', 'dequantize', 'add_backend', 'get_backend', 'set_backend',
           'set_global_backend']
