"""Quantization wrappers of the v1 path.

Mirrors TrainingExtensions/torch/src/python/aimet_torch/v1/qc_quantize_op.py: QcQuantizeOpMode (:63-70),
tensor_quantizer_factory (:80-112), QcQuantizeWrapper (:198-496), StaticGridQuantWrapper (:679-924) and
SteGatingFuncForParameters (:1314-1366).  The wrapper decides *which* tensors are quantized and when
(ANALYSIS = update statistics, ACTIVE = quantize-dequantize); the arithmetic is in the HIP kernels.

One mechanical difference: the original parameters are kept by reference and swapped back after the wrapped module
has run, instead of cloned and copied back (two fewer passes over every weight per forward); at backward time the
module's parameters hold the original values in both designs.
"""
import os
from enum import Enum
from typing import List, Tuple

import torch
from torch import nn

from ..common import libpymo
from ..common.defs import QuantizationDataType, QuantScheme
from . import quantsim_straight_through_grad as ste
from .tensor_quantizer import StaticGridPerChannelQuantizer, StaticGridPerTensorQuantizer


class QcQuantizeOpMode(Enum):
    """Mode for the quantization ops."""
    PASSTHROUGH = 1
    ANALYSIS = 2
    ACTIVE = 3
    LEARN_ENCODINGS = 4


QUANTIZER_TYPE_INPUT = 'input'
QUANTIZER_TYPE_OUTPUT = 'output'
TF_ENHANCED_USE_DOWNSAMPLING = bool(int(os.environ.get("AIMET_TFE_USE_DOWNSAMPLING", "0")))
TF_ENHANCED_OFFSET_FACTOR = 0
TF_ENHANCED_STRIDE_FACTOR = 2

MAP_ROUND_MODE = {'nearest': libpymo.RoundingMode.ROUND_NEAREST, 'stochastic': libpymo.RoundingMode.ROUND_STOCHASTIC}


def _to_round_mode(round_mode):
    return MAP_ROUND_MODE[round_mode] if isinstance(round_mode, str) else round_mode


def tensor_quantizer_factory(bitwidth: int, round_mode, quant_scheme: QuantScheme, use_symmetric_encodings: bool,
                             enabled_by_default: bool, data_type: QuantizationDataType = QuantizationDataType.int):
    """Instantiates the tensor quantizer for `quant_scheme` (post-training schemes; range learning is not built)."""
    if quant_scheme in (QuantScheme.post_training_tf_enhanced, QuantScheme.post_training_tf):
        return StaticGridPerTensorQuantizer(bitwidth, _to_round_mode(round_mode), quant_scheme,
                                            use_symmetric_encodings, enabled_by_default, data_type=data_type)
    raise AssertionError("Unsupported quant_scheme: " + str(quant_scheme))


class QcQuantizeWrapper(nn.Module):
    """Base class of the quantization wrappers: owns input / parameter / output quantizers of one module."""

    # pylint: disable=too-many-arguments
    def __init__(self, module_to_wrap: nn.Module, weight_bw: int, activation_bw: int, round_mode,
                 quant_scheme: QuantScheme, is_output_quantized=True, is_symmetric=False, num_inputs=1,
                 num_outputs=1, data_type: QuantizationDataType = QuantizationDataType.int):
        super().__init__()
        self.output_quantizers = [tensor_quantizer_factory(activation_bw, round_mode, quant_scheme, is_symmetric,
                                                           enabled_by_default=is_output_quantized,
                                                           data_type=data_type) for _ in range(num_outputs)]
        self._mode = QcQuantizeOpMode.ANALYSIS
        self._module_to_wrap = module_to_wrap
        self.param_quantizers = {}
        for name, _ in module_to_wrap.named_parameters():
            self.param_quantizers[name] = tensor_quantizer_factory(weight_bw, round_mode, quant_scheme, is_symmetric,
                                                                   enabled_by_default=True, data_type=data_type)
        self.input_quantizers = [tensor_quantizer_factory(activation_bw, round_mode, quant_scheme, is_symmetric,
                                                          enabled_by_default=False, data_type=data_type)
                                 for _ in range(num_inputs)]
        self.supported_kernels = {}

    def get_named_parameters(self):
        yield from self._module_to_wrap.named_parameters()

    def __getattr__(self, name):
        try:
            return super().__getattr__(name)
        except AttributeError:
            return getattr(self._module_to_wrap, name)

    def get_original_module(self) -> nn.Module:
        return self._module_to_wrap

    def set_output_bw(self, output_bw: int):
        self.output_quantizers[0].bitwidth = output_bw

    def set_mode(self, mode):
        self._mode = mode

    def enable_param_quantizers(self, enabled: bool, param_name_to_exclude: Tuple[str] = ("bias",)) -> None:
        param_name_to_exclude = param_name_to_exclude or ()
        for name, quantizer in self.param_quantizers.items():
            if name not in param_name_to_exclude:
                quantizer.enabled = enabled

    def enable_input_quantizers(self, enabled: bool) -> None:
        for quantizer in self.input_quantizers:
            quantizer.enabled = enabled

    def enable_output_quantizers(self, enabled: bool) -> None:
        for quantizer in self.output_quantizers:
            quantizer.enabled = enabled

    def enable_activation_quantizers(self, enabled: bool) -> None:
        self.enable_input_quantizers(enabled)
        self.enable_output_quantizers(enabled)

    def reset_encodings(self):
        for quantizer in self.param_quantizers.values():
            quantizer.reset_encoding_stats()
        for quantizer in self.output_quantizers:
            quantizer.reset_encoding_stats()
        for quantizer in self.input_quantizers:
            quantizer.reset_encoding_stats()

    def should_perform_quant_dequant(self, tensor: torch.Tensor, tensor_quantizer) -> bool:
        """Only floating point tensors with an enabled quantizer are quantized (reference :452-468)."""
        return tensor_quantizer.enabled and tensor.dtype in (torch.float32, torch.float16, torch.bfloat16)


class SteGatingFuncForParameters(torch.autograd.Function):
    """Identity in forward; in backward, masks each quantized parameter's .grad to its encoding range."""

    @staticmethod
    def forward(ctx, quant_wrapper_ref, *quantized_inputs):  # pylint: disable=arguments-differ
        ctx.quantization_wrapper_ref = quant_wrapper_ref
        return quantized_inputs

    @staticmethod
    def backward(ctx, *output_grad):  # pylint: disable=arguments-differ
        wrapper = ctx.quantization_wrapper_ref
        for name, param in wrapper.get_named_parameters():
            quantizer = wrapper.param_quantizers[name]
            if quantizer.bitwidth == 32 or quantizer.data_type == QuantizationDataType.float:
                continue
            if quantizer.enabled and param.grad is not None:
                if isinstance(quantizer.encoding, list):
                    _, _, _, _, raw_min, raw_max = quantizer.device_params(param.device)
                    # pylint: disable=protected-access
                    param.grad = ste.compute_dloss_by_dx(param, param.grad, raw_min, raw_max, quantizer._ch_axis)
                else:
                    param.grad = ste.compute_dloss_by_dx(param, param.grad, quantizer.encoding.min,
                                                         quantizer.encoding.max)
        return (None, *output_grad)


class StaticGridQuantWrapper(QcQuantizeWrapper):
    """Wrapper for post-training (static grid) quantization simulation."""

    def forward(self, *inputs, **kwargs):
        quantized_inputs = self._quantize_activation(self.input_quantizers, list(inputs))
        shadow_params = self._quantize_dequantize_params()
        if torch.is_grad_enabled():
            quantized_inputs = SteGatingFuncForParameters.apply(self, *quantized_inputs)
            # the custom function returns its inputs as they are; clone so that an in-place op of the wrapped module
            # cannot corrupt the gradient bookkeeping of that view.  Without autograd there is nothing to gate and
            # nothing to protect: no extra pass over the activations.
            quantized_inputs = [inp.clone() if isinstance(inp, torch.Tensor) else inp for inp in quantized_inputs]
        wrapped_output = self._module_to_wrap(*quantized_inputs, **kwargs)
        self._restore_shadow_params(shadow_params)
        if not isinstance(wrapped_output, (List, Tuple)):
            wrapped_output = [wrapped_output]
        output = self._quantize_activation(self.output_quantizers, list(wrapped_output))
        return output[0] if len(output) == 1 else output

    def _restore_shadow_params(self, shadow_params):
        for name, param in self.get_named_parameters():
            param.data = shadow_params[name]

    def _quantize_dequantize_params(self):
        shadow_params = {}
        for name, param in self.get_named_parameters():
            shadow_params[name] = param.data
            quantizer = self.param_quantizers[name]
            if quantizer.enabled and quantizer.bitwidth != 32:
                # in training mode the parameter encodings are recomputed in every pass
                if self._module_to_wrap.training or quantizer.encoding is None:
                    quantizer.reset_encoding_stats()
                    quantizer.update_encoding_stats(param.data)
                    quantizer.compute_encoding()
                round_mode = quantizer.round_mode if self.training else libpymo.RoundingMode.ROUND_NEAREST
                param.data = quantizer.quantize_dequantize(param.data, round_mode)
        return shadow_params

    def compute_weight_encodings(self):
        return self.param_quantizers['weight'].encoding if 'weight' in self.param_quantizers else None

    def compute_encoding(self):
        for quantizer in self.input_quantizers:
            quantizer.compute_encoding()
        for quantizer in self.param_quantizers.values():
            quantizer.compute_encoding()
        for quantizer in self.output_quantizers:
            quantizer.compute_encoding()

    def _quantize_activation(self, tensor_quantizers, tensors_to_quantize):
        def inner(tensor, index):
            if isinstance(tensor, (List, Tuple)):
                return [inner(t, index) for t in tensor]
            if not isinstance(tensor, torch.Tensor):
                return tensor
            quantizer = tensor_quantizers[index]
            if not self.should_perform_quant_dequant(tensor, quantizer):
                return tensor
            if self._mode is QcQuantizeOpMode.ANALYSIS and not quantizer.is_encoding_frozen:
                if TF_ENHANCED_USE_DOWNSAMPLING and quantizer.quant_scheme == QuantScheme.post_training_tf_enhanced:
                    flat = tensor.reshape(-1)
                    quantizer.update_encoding_stats(
                        flat[TF_ENHANCED_OFFSET_FACTOR::TF_ENHANCED_STRIDE_FACTOR].contiguous())
                else:
                    quantizer.update_encoding_stats(tensor)
                return tensor
            if self._mode is QcQuantizeOpMode.ACTIVE or \
                    (self._mode is QcQuantizeOpMode.ANALYSIS and quantizer.is_encoding_frozen):
                round_mode = quantizer.round_mode if self.training else libpymo.RoundingMode.ROUND_NEAREST
                return quantizer.quantize_dequantize(tensor, round_mode)
            return tensor

        outputs = []
        for index, tensor in enumerate(tensors_to_quantize):
            assert len(tensor_quantizers) > index, f"Not enough tensor quantizers ({len(tensor_quantizers)}) allocated"
            outputs.append(inner(tensor, index))
        return outputs

    def enable_per_channel_quantization(self):
        """Changes all parameter quantizers (if any) to per-channel mode (axis 0; axis 1 for transposed convs)."""
        new_param_quant_dict = {}
        for param_name, param in self._module_to_wrap.named_parameters():
            q = self.param_quantizers[param_name]
            channel_axis = 0
            if isinstance(self._module_to_wrap, (nn.ConvTranspose1d, nn.ConvTranspose2d, nn.ConvTranspose3d)) \
                    and len(param.shape) > 1:
                channel_axis = 1
            pc = StaticGridPerChannelQuantizer(q.bitwidth, q.round_mode, q.quant_scheme, q.use_symmetric_encodings,
                                               num_channels=param.shape[channel_axis], enabled_by_default=q.enabled,
                                               ch_axis=channel_axis, data_type=q.data_type)
            pc.use_strict_symmetric = q.use_strict_symmetric
            pc.use_unsigned_symmetric = q.use_unsigned_symmetric
            new_param_quant_dict[param_name] = pc
        self.param_quantizers = new_param_quant_dict
