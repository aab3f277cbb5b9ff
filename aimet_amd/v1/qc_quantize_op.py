"""Quantization wrappers of the v1 path.

Mirrors TrainingExtensions/torch/src/python/aimet_torch/v1/qc_quantize_op.py: QcQuantizeOpMode (:63-70),
tensor_quantizer_factory (:80-112), QcQuantizeWrapper (:198-496), StaticGridQuantWrapper (:679-924),
LearnedGridQuantWrapper (:947-1196), SteGatingFuncForParameters (:1314-1366) and FusedQdqLinear (:1446-1504).  The
wrapper decides *which* tensors are quantized and when (ANALYSIS = update statistics, ACTIVE = quantize-dequantize);
the arithmetic is in the HIP kernels.

One mechanical difference: the original parameters are kept by reference and swapped back after the wrapped module
has run, instead of cloned and copied back (two fewer passes over every weight per forward); at backward time the
module's parameters hold the original values in both designs.
"""
import os
from enum import Enum
from typing import List, Tuple

import torch
from torch import nn

from .. import ops
from ..common import libpymo
from ..common.defs import QuantizationDataType, QuantScheme
from ..utils import (compute_partial_encoding, create_encoding_dict, create_encoding_from_dict,
                     get_per_channel_quantizer_from_per_tensor, get_per_tensor_quantizer_from_per_channel,
                     validate_is_symmetric_flag)
from . import quantsim_straight_through_grad as ste
from .tensor_quantizer import (LearnedGridTensorQuantizer, StaticGridPerChannelQuantizer,
                               StaticGridPerTensorQuantizer, set_encoding_min_max_gating_threshold)


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
    """Instantiates the tensor quantizer for `quant_scheme`: static grid for the post-training schemes, learned grid
    for the range-learning schemes (reference :80-112)."""
    if quant_scheme in (QuantScheme.post_training_tf_enhanced, QuantScheme.post_training_tf,
                        QuantScheme.post_training_percentile):
        return StaticGridPerTensorQuantizer(bitwidth, _to_round_mode(round_mode), quant_scheme,
                                            use_symmetric_encodings, enabled_by_default, data_type=data_type)
    if quant_scheme in (QuantScheme.training_range_learning_with_tf_init,
                        QuantScheme.training_range_learning_with_tf_enhanced_init):
        return LearnedGridTensorQuantizer(bitwidth, _to_round_mode(round_mode), quant_scheme,
                                          use_symmetric_encodings, enabled_by_default, data_type)
    raise AssertionError("Unsupported quant_scheme: " + str(quant_scheme))


class QcQuantizeStandAloneBase(nn.Module):
    """A quantization op that stands by itself in a model: one output quantizer applied to whatever tensors pass
    through, with the wrappers' ANALYSIS / ACTIVE / PASSTHROUGH modes (reference :113-189)."""

    def __init__(self, activation_bw, round_mode, quant_scheme, is_symmetric, data_type=QuantizationDataType.int):
        super().__init__()
        self.output_quantizers = [tensor_quantizer_factory(activation_bw, round_mode, quant_scheme, is_symmetric,
                                                           enabled_by_default=True, data_type=data_type)]
        self._mode = QcQuantizeOpMode.ANALYSIS

    def forward(self, *inputs):
        raise NotImplementedError

    def set_output_bw(self, output_bw: int):
        self.output_quantizers[0].bitwidth = output_bw

    def set_mode(self, mode):
        self._mode = mode

    def _quantize_activation(self, tensor_quantizers, tensors_to_quantize):
        outputs = []
        for index, tensor in enumerate(tensors_to_quantize):
            if self._mode is QcQuantizeOpMode.ANALYSIS:
                tensor_quantizers[index].update_encoding_stats(tensor)
            elif self._mode is QcQuantizeOpMode.ACTIVE:
                # outside training only nearest rounding is used
                round_mode = tensor_quantizers[index].round_mode if self.training else \
                    libpymo.RoundingMode.ROUND_NEAREST
                tensor = tensor_quantizers[index].quantize_dequantize(tensor, round_mode)
            outputs.append(tensor)
        return outputs[0] if len(outputs) == 1 else outputs


class QcQuantizeStandalone(QcQuantizeStandAloneBase):
    """Quantizes its inputs (reference :1290-1310)."""

    def forward(self, *inputs):
        return self._quantize_activation(self.output_quantizers, list(inputs))

    def compute_encoding(self):
        self.output_quantizers[0].compute_encoding()


def get_encoding_by_quantizer(quantizer):
    """The encoding a quantizer is exported with: learned-grid quantizers report the one their quant scheme means
    (reference :1507-1519)."""
    if isinstance(quantizer, LearnedGridTensorQuantizer):
        return quantizer.get_effective_encoding()
    return quantizer.encoding


def export_quantizer_encoding(quantizer):
    """List of encoding dictionaries of an enabled quantizer, else None (reference :1522-1538)."""
    if not quantizer.enabled:
        return None
    encoding = get_encoding_by_quantizer(quantizer)
    if isinstance(encoding, list):
        return [create_encoding_dict(enc, quantizer, False) for enc in encoding]
    entry = create_encoding_dict(encoding, quantizer, False)
    return [entry] if entry else None


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
        module = self._module_to_wrap
        if not module._modules:                     # pylint: disable=protected-access
            # a leaf module: its own parameter table, without named_parameters' walk over the module tree (this runs
            # several times per forward pass of every wrapper)
            return [(name, p) for name, p in module._parameters.items() if p is not None]  # pylint: disable=protected-access
        return list(module.named_parameters())

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

    # ------------------------------------------------------------------------------- encodings in / out
    def export_param_encodings(self):
        """{parameter name: list of encoding dictionaries, or None} (reference :481-485)."""
        return {name: export_quantizer_encoding(q) for name, q in self.param_quantizers.items()}

    def export_output_encodings(self):
        return [export_quantizer_encoding(q) for q in self.output_quantizers]

    def export_input_encodings(self):
        return [export_quantizer_encoding(q) for q in self.input_quantizers]

    def set_param_encoding(self, module_name: str, param_encodings: dict, ignore_when_quantizer_disabled: bool = False,
                           disable_quantizer_without_encoding: bool = True):
        """Sets the parameter encodings found under '<module_name>.<parameter>' (reference :399-420)."""
        mine = {name: param_encodings[f'{module_name}.{name}'] for name in self.param_quantizers
                if f'{module_name}.{name}' in param_encodings}
        self.import_param_encodings(mine, strict=not ignore_when_quantizer_disabled,
                                    partial=not disable_quantizer_without_encoding, requires_grad=None,
                                    allow_overwrite=None)

    def set_activation_encoding(self, module_name: str, activation_encodings: dict,
                                ignore_when_quantizer_disabled: bool = False,
                                disable_quantizer_without_encoding: bool = True):
        """Sets input / output encodings found under activation_encodings[module_name] (reference :363-397)."""
        entry = activation_encodings.get(module_name, {})
        for kind, fn in (('input', self.import_input_encodings), ('output', self.import_output_encodings)):
            fn(entry.get(kind, {}), strict=not ignore_when_quantizer_disabled,
               partial=not disable_quantizer_without_encoding, requires_grad=None, allow_overwrite=None)

    def freeze_param_encoding(self, module_name: str, param_encodings: dict):
        for name, quantizer in self.param_quantizers.items():
            if f'{module_name}.{name}' in param_encodings and quantizer.enabled:
                quantizer.freeze_encoding()

    def freeze_activation_encoding(self, name: str, activation_encoding: dict):
        for input_quantizer, output_quantizer in zip(self.input_quantizers, self.output_quantizers):
            if name in activation_encoding:
                if QUANTIZER_TYPE_INPUT in activation_encoding[name] and input_quantizer.enabled:
                    input_quantizer.freeze_encoding()
                if QUANTIZER_TYPE_OUTPUT in activation_encoding[name] and output_quantizer.enabled:
                    output_quantizer.freeze_encoding()

    @staticmethod
    def _apply_int_encoding(quantizer, dicts, strict: bool):
        """Symmetry flags, bitwidth and the (completed) encodings of an 'int' entry onto one quantizer."""
        validate_is_symmetric_flag(quantizer, dicts[0], strict)
        is_symmetric = dicts[0]['is_symmetric'] == 'True'
        quantizer.use_symmetric_encodings = is_symmetric
        quantizer.use_unsigned_symmetric = quantizer.use_unsigned_symmetric if is_symmetric else False
        quantizer.use_strict_symmetric = quantizer.use_strict_symmetric if is_symmetric else False
        dicts = [compute_partial_encoding(quantizer, dict(d)) for d in dicts]
        quantizer.bitwidth = dicts[0]['bitwidth']
        encodings = [create_encoding_from_dict(d) for d in dicts]
        per_channel = isinstance(quantizer, StaticGridPerChannelQuantizer) or \
            (isinstance(quantizer, LearnedGridTensorQuantizer) and len(encodings) > 1)
        quantizer.encoding = encodings if per_channel else encodings[0]
        quantizer.data_type = QuantizationDataType.int

    @staticmethod
    def _finish_import(quantizer, requires_grad, allow_overwrite):
        if requires_grad is not None and isinstance(quantizer, LearnedGridTensorQuantizer) and quantizer.wrapper_ref:
            getattr(quantizer.wrapper_ref, quantizer.name + '_encoding_min').requires_grad_(requires_grad)
            getattr(quantizer.wrapper_ref, quantizer.name + '_encoding_max').requires_grad_(requires_grad)
        if allow_overwrite is not None and not allow_overwrite and quantizer.encoding is not None:
            quantizer.freeze_encoding()

    def import_param_encodings(self, encodings, strict: bool, partial: bool, requires_grad, allow_overwrite):
        """Imports {'parameter name': [dict, ...]} (reference :499-585).  strict: raise on a mismatch between the
        encodings and the quantizers instead of adapting; partial: leave quantizers without an entry alone instead
        of disabling them; allow_overwrite False freezes what was imported."""
        # pylint: disable=protected-access
        for name, quantizer in list(self.param_quantizers.items()):
            if quantizer._is_encoding_frozen:
                continue
            encoding = encodings.get(name, None)
            if not encoding:
                if not partial:
                    quantizer.enabled = False
                continue
            if not quantizer.enabled:
                if strict:
                    raise RuntimeError("The quantsim passed for loading encodings does not have the same "
                                       "configuration as the quantsim which was used to export the encodings")
                continue
            if isinstance(quantizer, StaticGridPerChannelQuantizer) and len(quantizer._cppOp) != len(encoding):
                assert len(encoding) == 1, (f'Number of Per Channel encodings provided ({len(encoding)}) is not same '
                                            f'as number of channels ({len(quantizer._cppOp)})')
                if strict:
                    raise ValueError(f"Invalid PerChannel encodings for {name}, the quantizer is a "
                                     f"PerChannelQuantizer. To avoid this, disable per_channel_quantization")
                quantizer = get_per_tensor_quantizer_from_per_channel(quantizer)
                self.param_quantizers[name] = quantizer
            elif isinstance(quantizer, StaticGridPerTensorQuantizer) and len(encoding) != 1:
                if strict:
                    raise ValueError(f"Invalid PerTensor encodings for {name}, the quantizer is a "
                                     f"PerTensorQuantizer. To avoid this, enable per_channel_quantization")
                quantizer = get_per_channel_quantizer_from_per_tensor(quantizer, self.get_original_module())
                assert len(quantizer._cppOp) == len(encoding), \
                    f'Number of per channel encodings ({len(encoding)}) should match the number of output channels'
                self.param_quantizers[name] = quantizer
            if encoding[0]['dtype'] == 'int':
                self._apply_int_encoding(quantizer, encoding, strict)
            elif encoding[0]['dtype'] == 'float':
                # a float entry carries no range: the quantizer casts to the float type of that many bits
                quantizer.bitwidth = encoding[0]['bitwidth']
                quantizer.data_type = QuantizationDataType.float
            else:
                raise RuntimeError("Data type does not match int or float in encodings file")
            self._finish_import(quantizer, requires_grad, allow_overwrite)

    def import_output_encodings(self, encodings, strict: bool, partial: bool, requires_grad, allow_overwrite):
        """Imports {'0': dict, '1': dict, ...} for the output quantizers (reference :588-676)."""
        self._import_encoding(encodings, self.output_quantizers, strict, partial, requires_grad, allow_overwrite)

    def import_input_encodings(self, encodings, strict: bool, partial: bool, requires_grad, allow_overwrite):
        self._import_encoding(encodings, self.input_quantizers, strict, partial, requires_grad, allow_overwrite)

    def _import_encoding(self, encodings, quantizers, strict, partial, requires_grad, allow_overwrite):
        for i, quantizer in enumerate(quantizers):
            if quantizer._is_encoding_frozen:  # pylint: disable=protected-access
                continue
            encoding = encodings.get(str(i), None)
            if not encoding:
                if not partial:
                    quantizer.enabled = False
                continue
            if not quantizer.enabled:
                if not strict:
                    continue
                raise RuntimeError("The quantsim passed for loading encodings does not have the same "
                                   "configuration as the quantsim which was used to export the encodings")
            if encoding['dtype'] == 'int':
                self._apply_int_encoding(quantizer, [encoding], strict)
            elif encoding['dtype'] == 'float':
                quantizer.bitwidth = encoding['bitwidth']
                quantizer.data_type = QuantizationDataType.float
            else:
                raise RuntimeError("Unrecognized encodings datatype")
            self._finish_import(quantizer, requires_grad, allow_overwrite)

    def enable_per_channel_quantization(self):
        """Changes the parameter quantizers to per-channel mode where the wrapper type supports it (static grid);
        a no-op otherwise (reference :355-361)."""

    def should_perform_quant_dequant(self, tensor: torch.Tensor, tensor_quantizer) -> bool:
        """Only floating point tensors with an enabled quantizer are quantized.  A quantizer that meets anything else,
        or a constant of one element, is switched off for good (reference :452-472)."""
        if not tensor_quantizer.enabled:
            return False
        if tensor.dtype not in (torch.float32, torch.float16, torch.bfloat16) or \
                (tensor_quantizer.is_const and tensor.numel() == 1):
            tensor_quantizer.enabled = False
            return False
        return True


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
                if isinstance(quantizer, StaticGridPerChannelQuantizer):
                    # (the bounds as device vectors: the per-channel encoding list is not needed on the host)
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
        if self._relu_is_absorbed(quantized_inputs, kwargs):
            wrapped_output = quantized_inputs[0]
        else:
            wrapped_output = self._module_to_wrap(*quantized_inputs, **kwargs)
        self._restore_shadow_params(shadow_params)
        if not isinstance(wrapped_output, (list, tuple)):
            wrapped_output = [wrapped_output]
        output = self._quantize_activation(self.output_quantizers, list(wrapped_output))
        return output[0] if len(output) == 1 else output

    def _relu_is_absorbed(self, inputs, kwargs) -> bool:
        """True when running the wrapped nn.ReLU would not change the wrapper's result, so its pass over the
        activations (one read and one write of the whole tensor, as much traffic as the quantizer itself) can be left
        out.  Quantize-dequantize first clamps to [encoding.min, encoding.max]; with encoding.min == 0 that clamp
        already maps every negative input to 0, NaN to encoding.max and leaves the rest alone, exactly as
        clamp(relu(x)) does, so QDQ(x) == QDQ(relu(x)) element for element.  Only taken without autograd (the
        straight-through mask of the pre-activation differs at x == 0) and for a ReLU that is not in-place (an
        in-place ReLU also rewrites its input, which other readers of that tensor may rely on)."""
        module = self._module_to_wrap
        if type(module) is not nn.ReLU or module.inplace or kwargs or torch.is_grad_enabled():  # pylint: disable=unidiomatic-typecheck
            return False
        if self._mode is not QcQuantizeOpMode.ACTIVE or len(inputs) != 1 or len(self.output_quantizers) != 1:
            return False
        tensor, quantizer = inputs[0], self.output_quantizers[0]
        if not isinstance(tensor, torch.Tensor) or not self.should_perform_quant_dequant(tensor, quantizer):
            return False
        encoding = getattr(quantizer, 'encoding', None)
        return quantizer.bitwidth < 32 and quantizer.data_type == QuantizationDataType.int and \
            encoding is not None and not isinstance(encoding, (list, tuple)) and encoding.min == 0.0

    def _restore_shadow_params(self, shadow_params):
        for name, param in self.get_named_parameters():
            param.data = shadow_params[name]

    # Quantized parameters are kept between forwards while nothing they depend on has changed: the reference
    # quantize-dequantizes every parameter in every forward (reference :747-763), which for a model in evaluation mode
    # is the same computation on the same numbers every time.  A kept tensor is used again only for the same storage
    # (data pointer), the same version of the parameter (in-place operations on the parameter count it up), shape and
    # dtype, and the same encoding object with the same bounds.  Not seen: an in-place edit through a `param.data`
    # alias (`w.data.mul_(2)` leaves pointer and version alone) -- call invalidate_param_cache() after one, or set
    # StaticGridQuantWrapper.cache_quantized_params = False.
    cache_quantized_params = True

    @staticmethod
    def _encoding_stamp(quantizer):
        return quantizer.encoding_stamp()

    def _param_cache_key(self, param, quantizer):
        # (the stream is part of the key: a tensor kept by a forward on one stream is not handed to a forward on
        # another, which nothing would order after the launch that wrote it)
        stream = ops.current_stream_handle(param.device) if param.is_cuda else None
        return (param.data_ptr(), param._version, param.dtype, tuple(param.shape), quantizer.bitwidth,  # pylint: disable=protected-access
                quantizer.data_type, self._encoding_stamp(quantizer), stream)

    def _params_may_be_kept(self) -> bool:
        return StaticGridQuantWrapper.cache_quantized_params and not self.training and \
            not self._module_to_wrap.training

    def invalidate_param_cache(self):
        self.__dict__['_param_cache'] = {}

    def __getstate__(self):
        # what is kept between forwards is not part of a saved or copied wrapper
        state = self.__dict__.copy()
        state.pop('_param_cache', None)
        state.pop('_param_encodings_ahead', None)
        return state

    @staticmethod
    def _observe_param(quantizer, param):
        """The statistics of a parameter quantizer are those of the parameter as it is now (reference :769-777)."""
        quantizer.reset_encoding_stats()
        quantizer.update_encoding_stats(param.data)
        if quantizer.quant_scheme == QuantScheme.post_training_percentile:
            quantizer.set_percentile_value(100)

    @staticmethod
    def _param_identity(param):
        return (param.data_ptr(), param._version, tuple(param.shape), param.dtype)  # pylint: disable=protected-access

    def observe_params_ahead(self):
        """What the first forward after a reset does for every parameter that has no encoding yet (reference
        :769-777), taken out of that forward: the statistics of all parameters of a model are queued here, and the
        encodings are read back by compute_param_encodings_ahead() before the calibration batches occupy the device,
        instead of one wait per parameter in the middle of the first batch.  A parameter that is replaced or changed in
        place before its wrapper's next forward is observed again there, as the reference would see it.  Returns the
        quantizers that were fed."""
        fed = []
        if self._module_to_wrap.training:
            return fed                      # recomputed in every pass anyway
        ahead = self.__dict__.setdefault('_param_encodings_ahead', {})
        for name, param in self.get_named_parameters():
            quantizer = self.param_quantizers[name]
            if quantizer.enabled and quantizer.bitwidth != 32 and not quantizer.has_encoding() and param.is_cuda:
                self._observe_param(quantizer, param)
                ahead[name] = self._param_identity(param)
                fed.append(quantizer)
        return fed

    def drop_params_observed_in_vain(self):
        """A wrapper whose forward never ran since observe_params_ahead() would not have fed its parameter quantizers
        in the reference: their statistics go, so that compute_encoding() switches them off as it does there."""
        for name in self.__dict__.pop('_param_encodings_ahead', {}):
            self.param_quantizers[name].reset_encoding_stats()

    def _quantize_dequantize_params(self):
        shadow_params = {}
        keep = self._params_may_be_kept()
        cache = self.__dict__.setdefault('_param_cache', {})
        for name, param in self.get_named_parameters():
            shadow_params[name] = param.data
            quantizer = self.param_quantizers[name]
            if quantizer.enabled and quantizer.bitwidth != 32:
                # in training mode the parameter encodings are recomputed in every pass
                ahead = self.__dict__.get('_param_encodings_ahead')
                stale = ahead is not None and ahead.pop(name, None) not in (None, self._param_identity(param))
                if self._module_to_wrap.training or not quantizer.has_encoding() or stale:
                    self._observe_param(quantizer, param)
                    quantizer.compute_encoding()
                if keep and quantizer.has_encoding():
                    key = self._param_cache_key(param, quantizer)
                    kept = cache.get(name)
                    if kept is None or kept[0] != key:
                        kept = (key, quantizer.quantize_dequantize(param.data, libpymo.RoundingMode.ROUND_NEAREST))
                        cache[name] = kept
                    param.data = kept[1]
                    continue
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

    def set_percentile_value(self, percentile_value: float):
        """Percentile of the activation quantizers of this wrapper (reference :827-835); parameters are always
        calibrated at 100 (:775-776)."""
        for quantizer in list(self.input_quantizers) + list(self.output_quantizers):
            quantizer.set_percentile_value(percentile_value)

    def _quantize_activation(self, tensor_quantizers, tensors_to_quantize):
        def inner(tensor, index):
            if isinstance(tensor, (list, tuple)):
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


# ------------------------------------------------------------------------------------------------- range learning
_ENABLE_RECOMPUTE = False


class _Handle:
    """Undoes a temporary change when closed or when the `with` block ends."""

    def __init__(self, cleanup_fn):
        self._cleanup_fn, self._done = cleanup_fn, False

    def remove(self):
        if not self._done:
            self._cleanup_fn()
            self._done = True

    def __enter__(self):
        return self

    def __exit__(self, *_):
        self.remove()


def _set_enable_recompute(mode: bool) -> _Handle:
    global _ENABLE_RECOMPUTE  # pylint: disable=global-statement
    original = _ENABLE_RECOMPUTE

    def cleanup():
        global _ENABLE_RECOMPUTE  # pylint: disable=global-statement
        _ENABLE_RECOMPUTE = original
    _ENABLE_RECOMPUTE = mode
    return _Handle(cleanup)


def is_recompute_enabled() -> bool:
    """True if the quantize-dequantized weight of fused layers is recomputed in backward instead of kept."""
    return _ENABLE_RECOMPUTE


def enable_recompute() -> _Handle:
    return _set_enable_recompute(True)


def disable_recompute() -> _Handle:
    return _set_enable_recompute(False)


no_recompute = disable_recompute       # the reference's name (:1439-1443)


class LearnedGridQuantWrapper(QcQuantizeWrapper):
    """Wrapper whose enabled quantizers learn their encoding min / max (reference :947-1170).  The min / max of every
    quantizer are parameters of this module, named input<i>_encoding_min/max, output<i>_encoding_min/max and
    <param>_encoding_min/max; they stay None until an encoding is assigned."""

    # pylint: disable=too-many-arguments
    def __init__(self, module_to_wrap: nn.Module, weight_bw: int, activation_bw: int, round_mode,
                 quant_scheme: QuantScheme, device: torch.device, is_output_quantized: bool = True,
                 is_symmetric: bool = False, num_inputs=1, num_outputs=1,
                 data_type: QuantizationDataType = QuantizationDataType.int):
        if data_type != QuantizationDataType.int:
            raise ValueError('Only QuantizationDataType.int is supported for LearnedGridQuantWrapper')
        super().__init__(module_to_wrap, weight_bw, activation_bw, round_mode, quant_scheme, is_output_quantized,
                         is_symmetric, num_inputs, num_outputs, data_type)
        self.device = device
        self._initialize_trainable_parameters_and_tensor_quantizers(num_inputs, num_outputs)

    def _initialize_trainable_parameters_and_tensor_quantizers(self, num_inputs, num_outputs):
        def attach(quantizer, name):
            self.register_parameter(name + '_encoding_min', None)
            self.register_parameter(name + '_encoding_max', None)
            quantizer.name, quantizer.wrapper_ref, quantizer.device = name, self, self.device

        for index in range(num_inputs):
            attach(self.input_quantizers[index], 'input' + str(index))
        for index in range(num_outputs):
            attach(self.output_quantizers[index], 'output' + str(index))
        transposed = isinstance(self._module_to_wrap, (nn.ConvTranspose1d, nn.ConvTranspose2d, nn.ConvTranspose3d))
        for name, param in self.get_named_parameters():
            attach(self.param_quantizers[name], name)
            # pylint: disable=protected-access
            self.param_quantizers[name]._ch_axis = 1 if transposed and len(param.shape) > 1 else 0

    def _named_quantizers(self):
        for index, quantizer in enumerate(self.input_quantizers):
            yield 'input' + str(index), quantizer
        for index, quantizer in enumerate(self.output_quantizers):
            yield 'output' + str(index), quantizer
        for name, _ in self._module_to_wrap.named_parameters():
            yield name, self.param_quantizers[name]

    def apply_gating_logic(self):
        """Keeps every learned range ordered around zero before it is used (min <= 0 <= max, max > min)."""
        for name, quantizer in self._named_quantizers():
            if quantizer.enabled and quantizer.bitwidth != 32 and quantizer.data_type != QuantizationDataType.float:
                encoding_min = getattr(self, name + '_encoding_min')
                encoding_max = getattr(self, name + '_encoding_max')
                if ste.grid_in_one_launch(encoding_min, encoding_max):
                    # the same launch leaves delta / offset of the ordered range for the forward pass that follows
                    ste.gate_and_prepare_grid(quantizer, encoding_min, encoding_max)
                else:
                    set_encoding_min_max_gating_threshold(encoding_min, encoding_max)

    def forward(self, *inputs, **kwargs):
        self.apply_gating_logic()
        quantized_inputs = self._quantize_activation(list(inputs), self.input_quantizers, 'input')
        forward_fn = _default_forward
        if torch.is_grad_enabled() and is_recompute_enabled():
            forward_fn = _fused_forward_functions.get(type(self._module_to_wrap), _default_forward)
        wrapped_output = forward_fn(self, quantized_inputs, **kwargs)
        if not isinstance(wrapped_output, (list, tuple)):
            wrapped_output = [wrapped_output]
        output = self._quantize_activation(list(wrapped_output), self.output_quantizers, 'output')
        return output[0] if len(output) == 1 else output

    def _quantize_params(self) -> _Handle:
        """Puts the quantize-dequantized parameters in the wrapped module's place until the handle is closed.  The
        replacements are results of an autograd function, so gradients reach the original parameter and the
        encoding min / max."""
        params = self._module_to_wrap._parameters  # pylint: disable=protected-access
        originals = {}

        def cleanup():
            for name, original in originals.items():
                params[name] = original

        try:
            for name, _ in self.get_named_parameters():
                quantizer = self.param_quantizers[name]
                if not quantizer.enabled:
                    continue
                original = params[name]
                quantized = quantizer.quantize_dequantize(original, getattr(self, name + '_encoding_min'),
                                                          getattr(self, name + '_encoding_max'))
                originals[name] = original
                params[name] = quantized
            return _Handle(cleanup)
        except Exception:
            cleanup()
            raise

    def _quantize_activation(self, tensors_to_quantize, tensor_quantizers, type_of_quantizer: str) -> List:
        def inner(tensor, index):
            if isinstance(tensor, (list, tuple)):
                return [inner(t, index) for t in tensor]
            if not isinstance(tensor, torch.Tensor) or \
                    not self.should_perform_quant_dequant(tensor, tensor_quantizers[index]):
                return tensor
            encoding_min = getattr(self, type_of_quantizer + str(index) + '_encoding_min')
            encoding_max = getattr(self, type_of_quantizer + str(index) + '_encoding_max')
            return tensor_quantizers[index].quantize_dequantize(tensor, encoding_min, encoding_max)

        outputs = []
        for index, tensor in enumerate(tensors_to_quantize):
            assert len(tensor_quantizers) > index, f"Not enough tensor quantizers ({len(tensor_quantizers)}) allocated"
            outputs.append(inner(tensor, index))
        return outputs


def _default_forward(quant_wrapper: LearnedGridQuantWrapper, inputs, **kwargs):
    # pylint: disable=protected-access
    with quant_wrapper._quantize_params():
        return quant_wrapper._module_to_wrap(*inputs, **kwargs)


def _linear_forward_with_recompute(quant_wrapper: LearnedGridQuantWrapper, inputs, **kwargs):
    """nn.Linear without keeping the quantize-dequantized weight for backward (reference :1175-1196)."""
    # pylint: disable=protected-access
    if not quant_wrapper.param_quantizers['weight'].enabled or kwargs or len(inputs) != 1:
        return _default_forward(quant_wrapper, inputs, **kwargs)
    module = quant_wrapper._module_to_wrap
    return FusedQdqLinear.apply(inputs[0], module.weight, module.bias, quant_wrapper.weight_encoding_min,
                                quant_wrapper.weight_encoding_max, quant_wrapper.param_quantizers['weight'])


_fused_forward_functions = {nn.Linear: _linear_forward_with_recompute}


class FusedQdqLinear(torch.autograd.Function):
    """Linear layer on a range-learned weight that saves the original weight only: backward recomputes the
    quantize-dequantized weight for the input gradient (one kernel) and gets the weight gradient and the encoding
    gradients from one pass over (weight, dL/dWq) (reference :1446-1504)."""

    @staticmethod
    def forward(ctx, inp, weight, bias, weight_encoding_min, weight_encoding_max, weight_quantizer):
        # pylint: disable=arguments-differ
        ctx.save_for_backward(inp, weight, bias, weight_encoding_min.detach().clone(),
                              weight_encoding_max.detach().clone())
        ctx.weight_quantizer = weight_quantizer
        qdq_weight, _ = ste.learned_grid_forward(weight, weight_quantizer, weight_encoding_min, weight_encoding_max)
        return torch.nn.functional.linear(inp, qdq_weight, bias)

    @staticmethod
    def backward(ctx, grad):  # pylint: disable=arguments-differ
        inp, weight, bias, encoding_min, encoding_max = ctx.saved_tensors
        quantizer = ctx.weight_quantizer
        need_x, need_w, need_b, need_min, need_max = ctx.needs_input_grad[:5]
        dloss_by_dx = dloss_by_dw = dloss_by_db = dloss_by_dmin = dloss_by_dmax = None
        saved = None
        if need_x:
            qdq_weight, saved = ste.learned_grid_forward(weight, quantizer, encoding_min, encoding_max)
            dloss_by_dx = torch.matmul(grad, qdq_weight)
            del qdq_weight
        if need_w or need_min or need_max:
            if saved is None:
                delta, offset, _ = ste.get_computed_encodings(quantizer.bitwidth, encoding_min.float(),
                                                              encoding_max.float(),
                                                              quantizer.use_symmetric_encodings,
                                                              quantizer.use_strict_symmetric,
                                                              quantizer.is_unsigned_symmetric)
                saved = (delta, offset, ste._num_steps(quantizer),  # pylint: disable=protected-access
                         *ste._channel_geometry(weight, delta.numel(), quantizer.channel_axis))
            dloss_by_dwq = torch.matmul(grad.reshape(-1, grad.shape[-1]).t(), inp.reshape(-1, inp.shape[-1]))
            dloss_by_dw, dloss_by_dmin, dloss_by_dmax = ste.learned_grid_backward(
                weight, dloss_by_dwq, saved, encoding_min, encoding_max, quantizer.use_symmetric_encodings,
                need_w, need_min or need_max)
            if not need_w:
                dloss_by_dw = None
        if need_b and isinstance(bias, torch.Tensor):
            dloss_by_db = grad.reshape(-1, grad.shape[-1]).sum(dim=0)
        return dloss_by_dx, dloss_by_dw, dloss_by_db, dloss_by_dmin if need_min else None, \
            dloss_by_dmax if need_max else None, None
