"""Helpers that swap the weight quantizers of chosen layers of a v2 simulation model for blockwise or grouped blockwise
ones, and the activation quantizers for float quantizers.

Mirrors TrainingExtensions/torch/src/python/aimet_torch/v2/quantsim/config_utils.py: which layers are meant is given as
a list of module types, a list of the simulation model's own layers, or a predicate (:134-147); a single block size
applies to the weight's input-channel axis with one scale per output channel (:85-107), a single block grouping to the
input-channel axis (:110-131); -1 spans the axis; a weight whose shape a block size does not divide is an error that
names the layer (:312-331).
"""
import itertools
from typing import Callable, List, Optional, Tuple, Union

import torch

from ..quantization.affine import GroupedBlockQuantizeDequantize, QuantizeDequantize
from ..quantization.float import FloatQuantizeDequantize

_TRANSPOSED = (torch.nn.ConvTranspose1d, torch.nn.ConvTranspose2d, torch.nn.ConvTranspose3d)
modules_with_in_out_channels = (torch.nn.Linear, torch.nn.Conv1d, torch.nn.Conv2d, torch.nn.Conv3d) + _TRANSPOSED


def _channel_axes(module: torch.nn.Module, what: str) -> Tuple[int, int]:
    """(input-channel axis, output-channel axis) of the module's weight"""
    if not isinstance(module, modules_with_in_out_channels):
        raise RuntimeError(f'Single value {what} is only supported for modules of types in '
                           f'config_utils.modules_with_in_out_channels, but got module of type {type(module)}. Update '
                           f'the argument for identifying modules to set to exclude unsupported types.')
    return (0, 1) if isinstance(module, _TRANSPOSED) else (1, 0)


def _block_size_per_axis(module: torch.nn.Module, block_size: Union[int, Tuple[int, ...]]):
    if isinstance(block_size, (tuple, list)):
        return list(block_size)
    in_axis, out_axis = _channel_axes(module, 'block size')
    per_axis = [-1] * module.weight.dim()
    per_axis[in_axis], per_axis[out_axis] = block_size, 1
    return per_axis


def _block_grouping_per_axis(module: torch.nn.Module, block_grouping: Union[int, Tuple[int, ...]]):
    if isinstance(block_grouping, (tuple, list)):
        return list(block_grouping)
    in_axis, _ = _channel_axes(module, 'block grouping')
    per_axis = [1] * module.weight.dim()
    per_axis[in_axis] = block_grouping
    return per_axis


def _as_condition(arg) -> Callable[[torch.nn.Module], bool]:
    if isinstance(arg, list) and arg and isinstance(arg[0], type) and issubclass(arg[0], torch.nn.Module):
        types = tuple(arg)
        return lambda module: isinstance(module, types)
    if isinstance(arg, list):
        if not arg or not isinstance(arg[0], torch.nn.Module):
            raise RuntimeError('List given as arg must contain either torch.nn.Module types or specific '
                               'torch.nn.Module objects.')
        chosen = list(arg)
        return lambda module: any(module is m for m in chosen)
    return arg


def _quantizer_shape(weight_shape, block_size) -> Optional[List[int]]:
    """Blocks per axis, or None when a block size does not divide its axis."""
    assert len(block_size) == len(weight_shape)
    shape = []
    for size, block in zip(weight_shape, block_size):
        if block == -1:
            shape.append(1)
        elif size % block:
            return None
        else:
            shape.append(size // block)
    return shape


def _layers_and_shapes(sim, condition, block_size):
    chosen, misfits = [], []
    for name, layer in sim.named_qmodules():
        if condition(layer) and 'weight' in layer.param_quantizers and layer.param_quantizers['weight'] is not None:
            per_axis = _block_size_per_axis(layer, block_size)
            shape = _quantizer_shape(layer.weight.shape, per_axis)
            if shape is None:
                misfits.append(f"Quant layer {name} has shape {tuple(layer.weight.shape)} which does not align with "
                               f"block_size {block_size}. Each dimension's shape must divide evenly with the "
                               f"corresponding block size.")
            chosen.append((layer, shape, per_axis))
    if misfits:
        raise RuntimeError('Quant layers found whose weights do not align with block size.\n' + '\n'.join(misfits))
    return chosen


def _device_of(quantizer: torch.nn.Module, default):
    for tensor in itertools.chain(quantizer.parameters(), quantizer.buffers()):
        return tensor.device
    return default


def set_blockwise_quantization_for_weights(sim, arg, bitwidth: int, symmetric: bool,
                                           block_size: Union[int, Tuple[int, ...]]):
    """Weight quantizers of the layers `arg` selects become blockwise QuantizeDequantize modules (reference :262-344).

    arg: list of module types | list of layers of sim.model | predicate on a layer.
    block_size: one entry per weight axis, or an int for the input-channel axis (one scale per output channel)."""
    model_device = next(sim.model.parameters()).device
    for layer, shape, per_axis in _layers_and_shapes(sim, _as_condition(arg), block_size):
        device = _device_of(layer.param_quantizers['weight'], model_device)
        layer.param_quantizers['weight'] = QuantizeDequantize(shape, bitwidth, symmetric, None, per_axis).to(device)


def set_grouped_blockwise_quantization_for_weights(sim, arg, bitwidth: int, symmetric: bool, decompressed_bw: int,
                                                   block_size: Union[int, Tuple[int, ...]],
                                                   block_grouping: Union[int, Tuple[int, ...]] = -1):
    """Weight quantizers of the layers `arg` selects become GroupedBlockQuantizeDequantize modules (reference
    :371-452): block scales are integers of decompressed_bw - bitwidth bits times one scale per group of blocks.

    block_grouping: one entry per weight axis, or an int for the input-channel axis; -1 groups all blocks of the
    axis."""
    model_device = next(sim.model.parameters()).device
    for layer, shape, per_axis in _layers_and_shapes(sim, _as_condition(arg), block_size):
        grouping = _block_grouping_per_axis(layer, block_grouping)
        device = _device_of(layer.param_quantizers['weight'], model_device)
        layer.param_quantizers['weight'] = GroupedBlockQuantizeDequantize(shape, bitwidth, symmetric, decompressed_bw,
                                                                          None, per_axis, grouping).to(device)


def set_activation_quantizers_to_float(sim, arg, exponent_bits: int = None, mantissa_bits: int = None,
                                       dtype: torch.dtype = None):
    """Input and output quantizers of the layers `arg` selects become float quantizers of the given format (a torch
    dtype, or exponent and mantissa bits); slots without a quantizer stay empty (reference :187-242)."""
    condition = _as_condition(arg)
    model_device = next(sim.model.parameters()).device
    for _, layer in sim.named_qmodules():
        if not condition(layer):
            continue
        for slots in (layer.input_quantizers, layer.output_quantizers):
            for index, quantizer in enumerate(slots):
                if quantizer is not None:
                    device = _device_of(quantizer, model_device)
                    slots[index] = FloatQuantizeDequantize(exponent_bits, mantissa_bits, dtype).to(device)
