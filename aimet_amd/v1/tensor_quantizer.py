"""v1 static-grid tensor quantizers.

Mirrors TrainingExtensions/torch/src/python/aimet_torch/v1/tensor_quantizer.py (TensorQuantizer :61-123,
StaticGridTensorQuantizer :143-395, StaticGridPerTensorQuantizer :398-480, StaticGridPerChannelQuantizer :483-570,
autograd functions QuantizeDequantize / Quantize :1098-1277): same class names, attributes, method names and
semantics.  What differs is below the interface:

* per-channel quantizers keep their per-channel (min, max, delta, offset) as four device vectors built once per
  encoding, instead of rebuilding a host vector and copying it to the device on every forward;
* per-channel min/max (TF) statistics are one fused kernel over the whole weight instead of one
  select().contiguous() copy plus two reductions per channel;
* bfloat16 tensors go through the kernels directly (conversion fused) instead of .to(float32) / .to(dtype) passes;
* the per-channel straight-through backward works (the reference's QuantizeDequantize.backward reads ``.min`` of a
  list for per-channel quantizers).
"""
import functools
import io
from typing import List, Optional, Tuple, Union

import torch

from .. import ops
from ..common import libpymo
from ..common.AimetTensorQuantizer import AimetTensorQuantizer
from ..common.defs import MAP_QUANT_SCHEME_TO_PYMO, QuantizationDataType, QuantScheme
from . import quantsim_straight_through_grad as grad_fn


class TensorQuantizer:
    """Base class: simulation of quantization for one tensor (a parameter, a layer input or a layer output)."""

    def __init__(self, bitwidth: int, round_mode: libpymo.RoundingMode, quant_scheme: QuantScheme,
                 use_symmetric_encodings: bool, enabled_by_default: bool,
                 data_type: QuantizationDataType = QuantizationDataType.int):
        super().__init__()
        self.round_mode = round_mode
        self._quant_scheme = quant_scheme
        self.use_symmetric_encodings = use_symmetric_encodings
        self.use_strict_symmetric = False
        self.use_unsigned_symmetric = False
        self.is_unsigned_symmetric = False
        self.bitwidth = bitwidth
        self.enabled = enabled_by_default
        self.data_type = data_type
        self.is_const = False
        self._encoding_min_max_fixed_vals = None
        self._is_encoding_frozen = False

    @property
    def quant_scheme(self):
        return self._quant_scheme

    @property
    def is_encoding_frozen(self):
        return self._is_encoding_frozen

    @property
    def channel_axis(self):
        return None

    @property
    def encoding_min_max_fixed_vals(self) -> Optional[Tuple[float, float]]:
        return self._encoding_min_max_fixed_vals


class StaticGridTensorQuantizer(TensorQuantizer):
    """Simulates quantization for the given tensor post training."""

    def __init__(self, bitwidth, round_mode, quant_scheme, use_symmetric_encodings, enabled_by_default,
                 data_type=QuantizationDataType.int):
        if data_type != QuantizationDataType.int:
            raise ValueError("only QuantizationDataType.int is implemented for the static-grid quantizers")
        super().__init__(bitwidth, round_mode, quant_scheme, use_symmetric_encodings, enabled_by_default, data_type)
        self._cppOp = None
        self._encoding = None

    def __str__(self):
        stream = io.StringIO(newline='\n')
        stream.write('StaticGrid TensorQuantizer:\n')
        stream.write(f'    quant-scheme:{self._quant_scheme}, round_mode={self.round_mode}, '
                     f'bitwidth={self.bitwidth}, enabled={self.enabled}\n')
        if self._encoding:
            for enc in self._encoding:
                stream.write(f'    min:{enc.min}, max={enc.max}, delta={enc.delta}, offset={enc.offset}\n')
        else:
            stream.write('    no encoding\n')
        return stream.getvalue()

    # pickling: the device objects are dropped and re-created, encodings travel as tuples (reference :182-220)
    def __getstate__(self):
        state = self.__dict__.copy()
        state['_num_ops'] = len(self._cppOp)
        state['_encoding'] = None if self._encoding is None else \
            [(e.min, e.max, e.delta, e.offset, e.bw) for e in self._encoding]
        for key in ('_cppOp', '_dev_params'):
            state.pop(key, None)
        return state

    def __setstate__(self, state):
        num_ops = state.pop('_num_ops')
        encoding = state.pop('_encoding')
        self.__dict__.update(state)
        self._cppOp = [AimetTensorQuantizer(MAP_QUANT_SCHEME_TO_PYMO[self._quant_scheme]) for _ in range(num_ops)]
        self._encoding = None if encoding is None else [libpymo.TfEncoding(*e) for e in encoding]
        self._dev_params = None

    @property
    def quant_scheme(self) -> QuantScheme:
        return self._quant_scheme

    @quant_scheme.setter
    def quant_scheme(self, quant_scheme: QuantScheme):
        # re-instantiates the analyzer objects, which also clears accumulated statistics (reference :222-247)
        self._quant_scheme = quant_scheme
        assert self._cppOp
        self._cppOp = [AimetTensorQuantizer(MAP_QUANT_SCHEME_TO_PYMO[quant_scheme]) for _ in self._cppOp]

    @property
    def encoding(self):
        return self._encoding

    @encoding.setter
    def encoding(self, encoding) -> None:
        if self._is_encoding_frozen:
            raise RuntimeError("Encoding can be set only when it is not frozen.")
        self._encoding = encoding
        self._dev_params = None

    @TensorQuantizer.encoding_min_max_fixed_vals.setter
    def encoding_min_max_fixed_vals(self, min_max_vals: Tuple[float, float]):
        assert isinstance(min_max_vals, tuple) and len(min_max_vals) == 2, 'Min max vals must be a tuple of two values'
        assert min_max_vals[0] < min_max_vals[1], f'Min value {min_max_vals[0]} is not less than max val ' \
                                                  f'{min_max_vals[1]}'
        if self.quant_scheme != QuantScheme.post_training_tf:
            self.quant_scheme = QuantScheme.post_training_tf
        self._encoding_min_max_fixed_vals = min_max_vals

    def _stats_tensor(self, tensor: torch.Tensor) -> torch.Tensor:
        if self.encoding_min_max_fixed_vals is not None:
            return torch.tensor(list(self.encoding_min_max_fixed_vals), dtype=torch.float32, device=tensor.device)
        return tensor

    def compute_encoding(self):
        """Compute the encoding(s) from the accumulated statistics; skipped for bitwidth 32 (reference :280-321)."""
        if self.enabled and not self._is_encoding_frozen:
            self._encoding = []
            self._dev_params = None
            if self.bitwidth == 32:
                self._encoding = None
                return
            for encoding, valid in self._compute_op_encodings():
                if not valid:
                    self.enabled = False
                else:
                    self._encoding.append(encoding)
            self.is_unsigned_symmetric = self.use_symmetric_encodings and self.use_unsigned_symmetric and \
                all(enc.min >= 0 and enc.max >= 0 for enc in self._encoding)
            assert not (not self.enabled and self._encoding), \
                'At least one encoding for a multi-encoding quantizer is invalid.'

    def _compute_op_encodings(self):
        return [op.getEncoding(self.bitwidth, self.use_symmetric_encodings, self.use_strict_symmetric,
                               self.use_unsigned_symmetric) for op in self._cppOp]

    def quantize_dequantize(self, tensor: torch.Tensor, round_mode: libpymo.RoundingMode) -> torch.Tensor:
        return QuantizeDequantize.apply(tensor, self, round_mode)

    def quantize(self, tensor: torch.Tensor, round_mode: libpymo.RoundingMode) -> torch.Tensor:
        return Quantize.apply(tensor, self, round_mode)

    def reset_encoding_stats(self):
        if not self._is_encoding_frozen:
            for op in self._cppOp:
                op.resetEncodingStats()
            self._encoding = None
            self._dev_params = None

    def get_stats_histogram(self) -> List[List]:
        if self._quant_scheme != QuantScheme.post_training_tf_enhanced:
            raise RuntimeError("get_stats_histogram() can be invoked only when quantization scheme is TF-Enhanced.")
        if not self._encoding:
            raise RuntimeError("get_stats_histogram() can be invoked only when encoding is computed.")
        return [op.getStatsHistogram() for op in self._cppOp]

    def freeze_encoding(self) -> None:
        if not self._encoding:
            raise RuntimeError("Encoding can be frozen only when it is not None.")
        self._is_encoding_frozen = True

    def set_percentile_value(self, percentile_value: float):
        for op in self._cppOp:
            op.setPercentileValue(percentile_value)


class StaticGridPerTensorQuantizer(StaticGridTensorQuantizer):
    """Per-tensor scale/offset."""

    def __init__(self, bitwidth, round_mode, quant_scheme, use_symmetric_encodings, enabled_by_default,
                 data_type=QuantizationDataType.int):
        super().__init__(bitwidth, round_mode, quant_scheme, use_symmetric_encodings, enabled_by_default, data_type)
        self._cppOp = [AimetTensorQuantizer(MAP_QUANT_SCHEME_TO_PYMO[quant_scheme])]
        self._dev_params = None

    @property
    def encoding(self) -> Union[None, libpymo.TfEncoding]:
        return self._encoding[0] if self._encoding else None

    @encoding.setter
    def encoding(self, encoding):
        if self._is_encoding_frozen:
            raise RuntimeError("Encoding can be set only when it is not frozen.")
        self._encoding = encoding if isinstance(encoding, list) and len(encoding) == 1 else [encoding]

    def update_encoding_stats(self, tensor: torch.Tensor):
        if self.enabled and not self._is_encoding_frozen:
            if self.bitwidth == 32:
                return
            self._cppOp[0].updateStats(self._stats_tensor(tensor), tensor.is_cuda)


class StaticGridPerChannelQuantizer(StaticGridTensorQuantizer):
    """Per-channel scale/offset along ``ch_axis``."""

    def __init__(self, bitwidth, round_mode, quant_scheme, use_symmetric_encodings, num_channels, enabled_by_default,
                 ch_axis: int = 0, data_type=QuantizationDataType.int):
        super().__init__(bitwidth, round_mode, quant_scheme, use_symmetric_encodings, enabled_by_default, data_type)
        self._cppOp = [AimetTensorQuantizer(MAP_QUANT_SCHEME_TO_PYMO[quant_scheme]) for _ in range(num_channels)]
        self._ch_axis = ch_axis
        self._dev_params = None      # (min, max, delta, offset, raw_min, raw_max) device vectors of the encoding
        self._tf_minmax = None       # fused per-channel running min/max for the TF scheme: device tensor [2, C]

    @property
    def channel_axis(self) -> int:
        return self._ch_axis

    def reset_encoding_stats(self):
        super().reset_encoding_stats()
        if not self._is_encoding_frozen:
            self._tf_minmax = None

    def update_encoding_stats(self, tensor: torch.Tensor):
        if self.enabled and not self._is_encoding_frozen:
            if self.bitwidth == 32:
                return
            if self.encoding_min_max_fixed_vals is not None:
                fixed = self._stats_tensor(tensor)
                for op in self._cppOp:
                    op.updateStats(fixed, fixed.is_cuda)
                return
            if tensor.dtype == torch.float16:
                tensor = tensor.to(torch.float32)
            if self._quant_scheme == QuantScheme.post_training_tf:
                # one fused pass: per-channel min and max of the whole tensor
                num_channel = tensor.shape[self._ch_axis]
                n_per_channel = functools.reduce(lambda a, b: a * b, tensor.shape[self._ch_axis + 1:], 1)
                mm = ops.minmax_per_channel(tensor, num_channel, n_per_channel)
                if self._tf_minmax is None:
                    self._tf_minmax = mm
                else:
                    self._tf_minmax = torch.stack((torch.minimum(self._tf_minmax[0], mm[0]),
                                                   torch.maximum(self._tf_minmax[1], mm[1])))
                return
            for channel_idx, op in enumerate(self._cppOp):
                tensor_slice = tensor.select(self._ch_axis, channel_idx).contiguous(
                    memory_format=torch.contiguous_format)
                op.updateStats(tensor_slice, tensor.is_cuda)

    def _compute_op_encodings(self):
        if self._tf_minmax is None:
            return super()._compute_op_encodings()
        # TfEncodingAnalyzer::computeEncoding per channel (DlQuantization/src/TfEncodingAnalyzer.cpp:80-101) on the
        # fused statistics: one small read-back, then the double-precision host recipe
        mm = self._tf_minmax.double().cpu()
        out = []
        for c in range(mm.shape[1]):
            lo, hi = min(0.0, float(mm[0, c])), max(0.0, float(mm[1, c]))
            hi = max(hi, lo + 0.01)
            e = ops.get_computed_encodings(self.bitwidth, lo, hi, self.use_symmetric_encodings,
                                           self.use_strict_symmetric, self.use_unsigned_symmetric)
            out.append((libpymo.TfEncoding(e.min, e.max, e.delta, e.offset, e.bw), True))
        return out

    def device_params(self, device):
        """Per-channel kernel parameters on `device`, built once per encoding."""
        if self._dev_params is None or self._dev_params[0].device != device:
            mn, mx, delta, offset = AimetTensorQuantizer.channelParams(device, self._encoding)
            raw = torch.tensor([[e.min for e in self._encoding], [e.max for e in self._encoding]],
                               dtype=torch.float32).to(device)
            self._dev_params = (mn, mx, delta, offset, raw[0].contiguous(), raw[1].contiguous())
        return self._dev_params


def _channel_geometry(tensor, ch_axis):
    sizes = [*tensor.shape, 1]
    num_channel = sizes[ch_axis]
    n_per_channel = functools.reduce(lambda x, y: x * y, sizes[ch_axis + 1:])
    return num_channel, n_per_channel


class QuantizeDequantize(torch.autograd.Function):
    """Quantize-dequantize with the straight-through gradient (reference :1098-1212)."""

    @staticmethod
    def _per_tensor_quantize_dequantize(tensor, tensor_quantizer, round_mode):
        # pylint: disable=protected-access
        return tensor_quantizer._cppOp[0].quantizeDequantize(tensor, tensor_quantizer.encoding, round_mode,
                                                             tensor.is_cuda)

    @staticmethod
    def _per_channel_quantize_dequantize(tensor, tensor_quantizer, round_mode):
        num_channel, n_per_channel = _channel_geometry(tensor, tensor_quantizer.channel_axis)
        mn, mx, delta, offset, _, _ = tensor_quantizer.device_params(tensor.device)
        dtype = tensor.dtype
        if dtype not in (torch.float32, torch.bfloat16):
            tensor = tensor.to(torch.float32)
        out = ops.qdq_per_channel(tensor, num_channel, n_per_channel, mn, mx, delta, offset,
                                  round_mode.value if isinstance(round_mode, libpymo.RoundingMode) else round_mode)
        return out.to(dtype)

    @staticmethod
    def forward(ctx, tensor, tensor_quantizer, round_mode):  # pylint: disable=arguments-differ
        if tensor_quantizer.enabled and tensor_quantizer.bitwidth != 32:
            if isinstance(tensor_quantizer, StaticGridPerChannelQuantizer):
                quantized = QuantizeDequantize._per_channel_quantize_dequantize(tensor, tensor_quantizer, round_mode)
            else:
                dtype = tensor.dtype
                quantized = QuantizeDequantize._per_tensor_quantize_dequantize(tensor, tensor_quantizer,
                                                                               round_mode).to(dtype)
            ctx.save_for_backward(tensor)
        else:
            quantized = tensor
        ctx.tensor_quantizer = tensor_quantizer
        return quantized

    @staticmethod
    def backward(ctx, output_grad):  # pylint: disable=arguments-differ
        q = ctx.tensor_quantizer
        if q.enabled and q.data_type == QuantizationDataType.int and q.bitwidth != 32:
            tensor, = ctx.saved_tensors
            if isinstance(q, StaticGridPerChannelQuantizer):
                _, _, _, _, raw_min, raw_max = q.device_params(tensor.device)
                grad = grad_fn.compute_dloss_by_dx(tensor, output_grad, raw_min, raw_max, q.channel_axis)
            else:
                grad = grad_fn.compute_dloss_by_dx(tensor, output_grad, q.encoding.min, q.encoding.max)
        else:
            grad = output_grad
        return grad, None, None


class Quantize(torch.autograd.Function):
    """Quantize only: float-valued grid indices, signed range by default (reference :1216-1277)."""

    @staticmethod
    def forward(ctx, tensor, tensor_quantizer, round_mode):  # pylint: disable=arguments-differ
        assert tensor_quantizer.enabled, 'Tensor quantizer must be enabled to perform quantize only.'
        assert tensor_quantizer.data_type == QuantizationDataType.int
        assert tensor_quantizer.bitwidth != 32, 'Tensor quantizer bitwidth must be < 32 to perform quantize only.'
        assert tensor_quantizer.encoding is not None, 'Tensor quantizer encoding must be valid.'
        shift_to_signed = not (tensor_quantizer.use_symmetric_encodings and tensor_quantizer.use_unsigned_symmetric)
        # pylint: disable=protected-access
        if isinstance(tensor_quantizer, StaticGridPerChannelQuantizer):
            slices = []
            for index, op in enumerate(tensor_quantizer._cppOp):
                tensor_slice = tensor.select(tensor_quantizer._ch_axis, index).contiguous()
                slices.append(op.quantize(tensor_slice, tensor_quantizer._encoding[index], round_mode,
                                          tensor.is_cuda, shift_to_signed))
            return torch.stack(tuple(slices), dim=tensor_quantizer._ch_axis)
        return tensor_quantizer._cppOp[0].quantize(tensor, tensor_quantizer.encoding, round_mode, tensor.is_cuda,
                                                   shift_to_signed)

    @staticmethod
    def backward(ctx, _output_grad):  # pylint: disable=arguments-differ
        raise AssertionError('Backward pass for quantize only not implemented')
