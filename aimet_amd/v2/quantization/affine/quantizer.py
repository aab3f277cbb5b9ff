"""v2 affine quantizer modules.

Mirrors TrainingExtensions/torch/src/python/aimet_torch/v2/quantization/affine/quantizer.py: AffineQuantizerBase
constructor signatures (:64-148), MinMaxQuantizer (:303-445: learnable ``min`` / ``max`` parameters, compute_encodings
context, get_min / get_max / get_scale / get_offset / set_range), Quantize (:448-563) and QuantizeDequantize
(:566-697).  The arithmetic is dispatched through the backend registry to the HIP kernels.
"""
import contextlib
import functools
import warnings
import weakref
from typing import Optional

import torch
from torch import nn

from .... import ops
from ...utils import (StatisticsNotFoundError, _is_expandable, get_encoding_shape_with_blocks, patch_attr,
                      reshape_tensor_for_blocks, ste_round)
from ..base import QuantizerBase
from ..encoding_analyzer import EncodingAnalyzer, MinMaxEncodingAnalyzer
from .backends import _derive_qmin_qmax, get_backend, quantize, quantize_dequantize
from .encoding import AffineEncoding, _GridMixin


_pending_range_checks = None     # a list while batched_range_checks() is active


def _examine_bounds(bounds: torch.Tensor, dtype: torch.dtype):
    """bounds: float64 host tensor of range bounds that were computed in `dtype`."""
    if not bool(torch.isfinite(bounds).all()):
        warnings.warn('Infinite or NaN values detected within input! This may skew the associated encodings')
    extreme = float(torch.finfo(dtype).max)
    # torch.isclose(|x|, extreme, rtol=0.05) with its default atol of 1e-8
    if bool(((bounds.abs() - extreme).abs() <= 1e-8 + 0.05 * extreme).any()):
        warnings.warn('Extreme values detected within input! This may skew the associated encodings')


def _flag_extreme_min_max(curr_min: torch.Tensor, curr_max: torch.Tensor):
    """Warns about ranges that are not finite or sit at the edge of the dtype (reference
    encoding_analyzer.py:388-395).  The bounds are parameter-sized: they are read back once and examined on the host,
    instead of four reductions that each wait for the device; inside batched_range_checks() the read-back is shared
    with every other quantizer's."""
    bounds = torch.cat((curr_min.detach().reshape(-1), curr_max.detach().reshape(-1))).to(torch.float64)
    if _pending_range_checks is not None:
        _pending_range_checks.append((bounds, curr_min.dtype))
        return
    _examine_bounds(bounds.cpu(), curr_min.dtype)


@contextlib.contextmanager
def batched_range_checks():
    """While active, the range warnings of every quantizer that leaves compute_encodings() are held back and issued
    together at the end, from one device-to-host copy per device."""
    global _pending_range_checks       # pylint: disable=global-statement
    outer, _pending_range_checks = _pending_range_checks, []
    try:
        yield
    finally:
        pending, _pending_range_checks = _pending_range_checks, outer
        groups = {}
        for bounds, dtype in pending:
            groups.setdefault((bounds.device, dtype), []).append(bounds)
        for (_, dtype), tensors in groups.items():
            _examine_bounds(torch.cat(tensors).cpu(), dtype)


def _grid_arguments(owner: str, args, kwargs):
    """(qmin, qmax, symmetric, encoding_analyzer, block_size) from either call form of the constructor
    (reference affine/quantizer.py:91-140):

        (shape, qmin, qmax, symmetric, encoding_analyzer=None, block_size=None)
        (shape, bitwidth, symmetric, encoding_analyzer=None, block_size=None)

    The two forms are told apart by what follows the first number: another number (or a `qmax` keyword) means a
    grid, a bool means `symmetric` and the first number was a bit-width.  Python's own argument binding then reports
    what is missing or unknown."""
    def from_grid(qmin, qmax, symmetric, encoding_analyzer=None, block_size=None):
        return qmin, qmax, symmetric, encoding_analyzer, block_size

    def from_bitwidth(bitwidth, symmetric, encoding_analyzer=None, block_size=None):
        return (*_derive_qmin_qmax(bitwidth=bitwidth, signed=symmetric), symmetric, encoding_analyzer, block_size)

    second = args[1] if len(args) > 1 else None
    grid_form = 'qmax' in kwargs or 'qmin' in kwargs or (second is not None and not isinstance(second, bool))
    try:
        return (from_grid if grid_form else from_bitwidth)(*args, **kwargs)
    except TypeError as error:
        raise TypeError(f"{owner}.__init__ expects (shape, qmin, qmax, symmetric) or (shape, bitwidth, symmetric), each "
                        f"optionally followed by encoding_analyzer and block_size: {error}") from None


class MinMaxQuantizer(_GridMixin, QuantizerBase):
    """Affine quantizer with min / max as trainable parameters."""

    def __init__(self, shape, *args, **kwargs):
        super().__init__()
        if isinstance(shape, int):
            shape = (shape,)
        self.shape = tuple(shape)
        qmin, qmax, symmetric, encoding_analyzer, block_size = _grid_arguments(type(self).__qualname__, args, kwargs)
        if qmin >= qmax:
            raise ValueError(f"qmax should be strictly larger than qmin. Got qmax={qmax}, qmin={qmin}")
        self.qmin, self.qmax = qmin, qmax
        self._symmetric = symmetric
        self.block_size = block_size   # kept as given (list or tuple), as the reference does
        # with blocks, statistics are gathered on the tensor split into (blocks, block length) per axis, by an
        # analyzer whose shape has a 1 after every axis (reference :140-148)
        self.encoding_analyzer: EncodingAnalyzer = encoding_analyzer or MinMaxEncodingAnalyzer(
            get_encoding_shape_with_blocks(self.shape, self.block_size))
        if self.block_size is None and not _is_expandable(self.encoding_analyzer.observer.shape, self.shape):
            raise RuntimeError(f'Encoding analyzer of shape {self.encoding_analyzer.observer.shape} '
                               f'is incompatible with quantizer of shape {self.shape}.')
        self._initial_parameters = {}
        self.register_quantization_parameter('min', nn.Parameter(-torch.ones(self.shape)))
        self.register_quantization_parameter('max', nn.Parameter(torch.ones(self.shape)))
        self._allow_overwrite = True

    # ---------------------------------------------------------------------------------------------- properties
    @property
    def symmetric(self) -> bool:
        return self._symmetric

    @symmetric.setter
    def symmetric(self, symmetric: bool):
        self._symmetric = symmetric

    # bitwidth / signed: views of (qmin, qmax), from _GridMixin

    # A parameter counts as initialised once it is no longer the untouched object it was created as: it has been
    # assigned anew, or modified in place (its version counter moved) -- reference base/quantizer.py:100-140.
    def register_quantization_parameter(self, name: str, param: nn.Parameter):
        """A parameter of the module whose initialisation is tracked (reference base/quantizer.py:99-107); min and max
        are registered this way, and a subclass may add its own."""
        self.register_parameter(name, param)
        self._remember_initial(name, getattr(self, name))

    def _remember_initial(self, name: str, param: nn.Parameter):
        self._initial_parameters[name] = (weakref.ref(param), param._version)  # pylint: disable=protected-access

    def _is_initialized(self, name: str) -> bool:
        initial_ref, initial_version = self._initial_parameters[name]
        initial = initial_ref() if initial_ref is not None else None
        if initial is None:
            return True
        current = getattr(self, name)
        return not (current is initial and current._version == initial_version)  # pylint: disable=protected-access

    def is_initialized(self) -> bool:
        return all(self._is_initialized(name) for name in self._initial_parameters)

    def allow_overwrite(self, mode: bool):
        """With False, compute_encodings() leaves the current parameters alone."""
        self._allow_overwrite = mode

    def get_extra_state(self):
        return {name: torch.tensor(self._is_initialized(name)) for name in self._initial_parameters}

    @torch.no_grad()
    def set_extra_state(self, state):
        for name in list(self._initial_parameters):
            if bool(state.get(name, False)):
                self._initial_parameters[name] = (None, -1)
            else:
                self._remember_initial(name, getattr(self, name))

    def __getstate__(self):
        state = self.__dict__.copy()
        state['_initial_parameters'] = {name: self._is_initialized(name) for name in self._initial_parameters}
        state.pop('_kept_encoding', None)
        return state

    def __setstate__(self, state):
        flags = state.pop('_initial_parameters')
        super().__setstate__(state)
        self._initial_parameters = {}
        for name, initialized in flags.items():
            if initialized:
                self._initial_parameters[name] = (None, -1)
            else:
                self._remember_initial(name, getattr(self, name))

    def extra_repr(self) -> str:
        return f'shape={self.shape}, qmin={self.qmin}, qmax={self.qmax}, symmetric={self.symmetric}'

    # ------------------------------------------------------------------------------------------------ calibration
    @contextlib.contextmanager
    def compute_encodings(self):
        """Observe inputs and set min / max from their statistics on exit; while inside, forward performs dynamic
        quantization with the batch statistics (reference :317-374)."""
        if not self._allow_overwrite:
            yield
            return
        analyzer = self.encoding_analyzer
        analyzer.reset_stats()
        plain_forward = self.forward
        with patch_attr(self, 'forward', functools.wraps(plain_forward)(
                lambda tensor: self._forward_on_batch_statistics(plain_forward, tensor))):
            yield
        # on exit: the statistics gathered inside become the parameters, if there are any
        try:
            found = analyzer.compute_encodings(self.qmax - self.qmin, self.symmetric)
        except StatisticsNotFoundError:
            return
        if any(bound is None for bound in found):
            return
        new_min, new_max = (self._in_parameter_shape(bound) for bound in found)
        _flag_extreme_min_max(new_min, new_max)
        self.set_range(new_min, new_max)

    def _in_parameter_shape(self, bound: torch.Tensor) -> torch.Tensor:
        """Blockwise statistics come with a singleton axis after every axis; the parameters do not have them."""
        return bound if self.block_size is None else bound.view(self.min.shape)

    def _forward_on_batch_statistics(self, plain_forward, tensor):
        """One forward inside compute_encodings(): the batch enters the running statistics, and the output is
        quantized with the range of this batch alone (reference :330-352)."""
        per_block = reshape_tensor_for_blocks(tensor, self.shape, self.block_size)
        batch = self.encoding_analyzer.update_stats(per_block)
        if getattr(plain_forward, 'is_pass_through', False):
            # a quantized module calibrates with its activation quantizers switched to pass-through: the range of
            # this batch alone would be computed (another pass over the batch, a search, a wait) and not used
            return plain_forward(tensor)
        bounds = self.encoding_analyzer.compute_encodings_from_stats(batch, self.qmax - self.qmin, self.symmetric)
        stand_ins = {}
        for name, bound in zip(('min', 'max'), bounds):
            param = getattr(self, name)
            stand_ins[name] = self._in_parameter_shape(bound).to(dtype=param.dtype, device=param.device) \
                .expand_as(param)
        with contextlib.ExitStack() as stack:
            for name, value in stand_ins.items():
                stack.enter_context(patch_attr(self, name, value))
            return plain_forward(tensor)

    def set_range(self, min: torch.Tensor, max: torch.Tensor):  # pylint: disable=redefined-builtin
        with torch.no_grad():
            self.min.copy_(min)
            self.max.copy_(max)

    def get_scale(self, dtype=None) -> Optional[torch.Tensor]:
        if not self.is_initialized():
            return None
        dtype = dtype or torch.float32
        num_steps = self.qmax - self.qmin
        return ((self.max.to(dtype) - self.min.to(dtype)) / num_steps).to(dtype)

    def get_offset(self, dtype=None) -> Optional[torch.Tensor]:
        if not self.is_initialized():
            return None
        dtype = dtype or torch.float32
        if self.symmetric:
            return torch.zeros_like(self.min, requires_grad=False, dtype=dtype)
        return (ste_round(self.min.to(dtype) / self.get_scale(dtype)) - self.qmin).to(dtype)

    def get_min(self, dtype=None) -> Optional[torch.Tensor]:
        if not self.is_initialized():
            return None
        return self.get_scale(dtype) * (self.get_offset(dtype) + self.qmin)

    def get_max(self, dtype=None) -> Optional[torch.Tensor]:
        if not self.is_initialized():
            return None
        return self.get_scale(dtype) * (self.get_offset(dtype) + self.qmax)

    def get_encoding(self) -> Optional[AffineEncoding]:
        if not self.is_initialized():
            return None
        # Scale and offset are a handful of parameter-sized tensor operations per call (the reference performs them in
        # every forward).  When no gradient can flow into min / max they depend on nothing but the parameters' values:
        # kept until a parameter object is replaced or modified in place (its version counter moves), or the grid
        # changes.  An edit through a `.data` alias moves no counter: assign, or use set_range().
        mn, mx = self.min, self.max
        learning = torch.is_grad_enabled() and (mn.requires_grad or mx.requires_grad)
        stream = ops.current_stream_handle(mn.device) if mn.is_cuda else None    # (kept per stream, as the parameters)
        key = None if learning else (id(mn), mn._version, id(mx), mx._version, self.qmin, self.qmax,  # pylint: disable=protected-access
                                     self._symmetric, stream)
        kept = self.__dict__.get('_kept_encoding')
        if key is not None and kept is not None and kept[0] == key and kept[1] is mn and kept[2] is mx:
            scale, offset = kept[3], kept[4]
        else:
            scale, offset = self.get_scale(torch.float32), self.get_offset(torch.float32)
            if key is not None:
                with torch.no_grad():
                    scale, offset = scale.detach(), offset.detach()
                self.__dict__['_kept_encoding'] = (key, mn, mx, scale, offset)
        return AffineEncoding._on_grid(scale, offset, self.qmin, self.qmax, self._symmetric, self.block_size)  # pylint: disable=protected-access

    def lower_bound_is_zero(self) -> bool:
        """True when the kept encoding's grid starts exactly at zero (offset == -qmin everywhere), known on the host:
        one read-back per kept encoding, none when no encoding is being kept (then the answer is False)."""
        if self.get_encoding() is None:
            return False
        kept = self.__dict__.get('_kept_encoding')
        if kept is None or kept[1] is not self.min or kept[2] is not self.max:
            return False
        if len(kept) == 5:
            if kept[4].is_cuda and torch.cuda.is_current_stream_capturing():
                return False             # would have to wait for the device: not while a graph is being captured
            kept = kept + (bool((kept[4] == -self.qmin).all()),)
            self.__dict__['_kept_encoding'] = kept
        return kept[5]

    @torch.no_grad()
    def get_legacy_encodings(self):
        if not self.is_initialized():
            return None
        enc = self.get_encoding()
        mn, mx = enc.min.flatten().tolist(), enc.max.flatten().tolist()
        sc, of = enc.scale.flatten().tolist(), enc.offset.flatten().tolist()
        return [{'min': a, 'max': b, 'scale': s, 'offset': int(o), 'bitwidth': self.bitwidth, 'dtype': 'int',
                 'is_symmetric': str(self.symmetric)} for a, b, s, o in zip(mn, mx, sc, of)]

    @torch.no_grad()
    def set_legacy_encodings(self, encodings):
        bitwidth = encodings[0]['bitwidth']
        symmetric = encodings[0]['is_symmetric'].lower() == 'true'
        self.qmin, self.qmax = _derive_qmin_qmax(bitwidth=bitwidth, signed=symmetric)
        self.symmetric = symmetric
        dev = self.min.device
        self.set_range(torch.tensor([e['min'] for e in encodings]).view(self.shape).to(dev),
                       torch.tensor([e['max'] for e in encodings]).view(self.shape).to(dev))


# The reference splits this class in two, AffineQuantizerBase (grid and encodings) and MinMaxQuantizer (min / max as
# parameters, :62-300); here they are one, under both names.
AffineQuantizerBase = MinMaxQuantizer


class Quantize(MinMaxQuantizer):
    """out = clamp(round(input / scale) - offset, qmin, qmax)"""

    def forward(self, input: torch.Tensor) -> torch.Tensor:  # pylint: disable=redefined-builtin
        if not self.is_initialized():
            raise RuntimeError('Failed to run Quantize since quantization parameters are not initialized.'
                               ' Please initialize the quantization parameters using `compute_encodings()`.')
        encoding = self.get_encoding()
        return quantize(input, encoding.scale, encoding.offset, encoding.qmin, encoding.qmax,
                        block_size=self.block_size)


class QuantizeDequantize(MinMaxQuantizer):
    """out = (clamp(round(input / scale) - offset, qmin, qmax) + offset) * scale"""

    # Training with a learnable range: min / max go to the backend as they are, which forms the grid and the range
    # gradients in its kernels.  False: scale and offset are formed here by tensor operations, as in the reference, and
    # autograd carries their gradients back to min / max.
    fuse_range_learning = True

    def forward(self, input: torch.Tensor) -> torch.Tensor:  # pylint: disable=redefined-builtin
        if not self.is_initialized():
            raise RuntimeError('Failed to run QuantizeDequantize since quantization parameters are not initialized.'
                               ' Please initialize the quantization parameters using `compute_encodings()`.')
        mn, mx = self.min, self.max
        own_grid = type(self).get_scale is not MinMaxQuantizer.get_scale or \
            type(self).get_offset is not MinMaxQuantizer.get_offset     # e.g. the grouped blockwise quantizer
        if self.fuse_range_learning and torch.is_grad_enabled() and (mn.requires_grad or mx.requires_grad) and \
                not own_grid:
            backend = get_backend()
            fused = getattr(backend, 'quantize_dequantize_learned_range', None)
            if fused is not None and backend.takes_learned_range(input, mn, mx):
                return fused(input, mn, mx, self.qmin, self.qmax, self._symmetric, block_size=self.block_size)
        encoding = self.get_encoding()
        return quantize_dequantize(input, encoding.scale, encoding.offset, encoding.qmin, encoding.qmax,
                                   block_size=self.block_size)


class GroupedBlockQuantizeDequantize(QuantizeDequantize):
    """Blockwise quantize-dequantize whose block scales are small integers times one scale per group of blocks
    (reference :700-822).

    The block scales that min / max define are themselves put on a grid: within a group of ``block_grouping`` blocks
    per axis, gamma = (largest block scale) / 2^(decompressed_bw - bitwidth), and every block of the group uses
    clamp(round(scale / gamma), 1, 2^(decompressed_bw - bitwidth)) * gamma.  A weight quantized this way expands to
    ``decompressed_bw``-bit integers times one floating-point scale per group.  -1 in ``block_grouping`` groups all
    blocks of that axis; the default groups nothing (every block is its own group, so its scale is kept).
    """

    def __init__(self, shape, bitwidth: int, symmetric: bool, decompressed_bw: int,
                 encoding_analyzer: EncodingAnalyzer = None, block_size=None, block_grouping=None):
        super().__init__(shape, bitwidth, symmetric, encoding_analyzer, block_size)
        self.decompressed_bw = decompressed_bw
        if block_grouping is None:
            self.block_grouping = tuple(1 for _ in self.shape)
        else:
            self.block_grouping = block_grouping   # kept as given
            if len(self.block_grouping) != len(self.shape):
                raise RuntimeError(f'Length of block grouping {block_grouping} must equal length of shape {shape}.')
            for size, group in zip(self.shape, self.block_grouping):
                if group != -1 and size % group != 0:
                    raise RuntimeError(f'Quantizer shape dimensions must divide evenly with corresponding block '
                                       f'grouping values for shapes {shape} and block grouping {block_grouping}.')
        if self.decompressed_bw < self.bitwidth:
            raise RuntimeError(f'Decompressed bitwidth {decompressed_bw} cannot be smaller than self.bitwidth '
                               f'{bitwidth}')
        if not symmetric:
            raise RuntimeError('GroupedBlockQuantizeDequantize only supports symmetric quantization.')

    def get_expanded_scale_shape(self):
        """The scale's shape with every axis split into (groups, blocks per group)."""
        expanded = []
        for size, group in zip(self.shape, self.block_grouping):
            per_group = size if group == -1 else group
            expanded += [size // per_group, per_group]
        return expanded

    def _block_scales_by_group(self, dtype):
        """(block scales viewed as [groups, blocks per group] per axis, gamma of every group)"""
        grouped = super().get_scale(dtype).view(self.get_expanded_scale_shape())
        within_group = list(range(1, grouped.dim(), 2))
        gamma = torch.amax(grouped, within_group, keepdim=True) / 2 ** (self.decompressed_bw - self.bitwidth)
        return grouped, gamma

    def get_per_channel_scale(self, dtype=None) -> Optional[torch.Tensor]:
        """gamma: the floating-point scale every block of a group shares."""
        if not self.is_initialized():
            return None
        return self._block_scales_by_group(dtype)[1]

    def get_scale(self, dtype=None) -> Optional[torch.Tensor]:
        """The block scales after rounding to integer multiples of their group's gamma."""
        if not self.is_initialized():
            return None
        grouped, gamma = self._block_scales_by_group(dtype)
        on_grid = quantize_dequantize(grouped, gamma, torch.zeros_like(gamma), 1,
                                      2 ** (self.decompressed_bw - self.bitwidth))
        return on_grid.view(self.shape)

    def get_per_block_integer_scale(self) -> Optional[torch.Tensor]:
        """The integer of every block: its scale divided by its group's gamma."""
        if not self.is_initialized():
            return None
        gamma = self.get_per_channel_scale()
        grouped = self.get_scale().view(self.get_expanded_scale_shape())
        return torch.round(grouped / gamma).int().view(self.shape)
