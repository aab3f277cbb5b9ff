"""Quantized modules of the v2 path: a mixin that adds input / parameter / output quantizers to a torch module class.

Mirrors BaseQuantizationMixin of TrainingExtensions/torch/src/python/aimet_torch/v2/nn/base.py (:60-262:
__quant_init__, __call__, _patch_quantized_parameters, _compute_param_encodings, compute_param_encodings,
compute_encodings, implements, from_module) and the fake-quantization forward of
TrainingExtensions/torch/src/python/aimet_torch/v2/nn/fake_quant.py (quantize inputs, patch quantized parameters, run
the base class' forward, quantize outputs).  The quantizers are the HIP-backed QuantizeDequantize modules.
"""
import contextlib
import itertools
from typing import Type

import torch
from torch import nn

from ... import ops
from ..quantization.affine.quantizer import MinMaxQuantizer
from ..utils import _ContextManager, patch_attr


def _no_op(input):  # pylint: disable=redefined-builtin
    return input


_no_op.is_pass_through = True      # a quantizer calibrating behind this forward need not quantize the batch


class BaseQuantizationMixin:
    """Mixin that implements quantization on top of regular torch modules."""

    cls_to_qcls: dict = {}
    qcls_to_cls: dict = {}

    def __init__(self, *args, **kwargs):
        super().__init__(*args, **kwargs)
        self.__quant_init__()

    def __quant_init__(self):
        """All quantizers start as None: one input, one output, one per parameter of the base module."""
        self.param_quantizers = nn.ModuleDict({name: None for name, _ in self.named_parameters(recurse=False)})
        self.input_quantizers = nn.ModuleList([None])
        self.output_quantizers = nn.ModuleList([None])

    def __call__(self, *args, **kwargs):
        self._compute_param_encodings(overwrite=False)
        return super().__call__(*args, **kwargs)

    # Quantized parameters are kept between forwards of a module in evaluation mode without autograd while nothing they
    # depend on has changed (the reference quantizes every parameter in every forward, :205-213): the same parameter
    # object at the same version and address, the same min / max parameter objects at the same versions, the same
    # grid, and a quantizer whose forward is its class's own.  In-place edits through a `.data` alias move no version
    # counter: set `keep_quantized_parameters = False` on the module (or the class) around them.
    keep_quantized_parameters = True

    def __getstate__(self):
        # what is kept between forwards is not part of a saved or copied module
        state = self.__dict__.copy()
        state.pop('_kept_quantized_parameters', None)
        return state

    def _kept_parameter_key(self, param, quantizer):
        if not self.keep_quantized_parameters or self.training or torch.is_grad_enabled() or \
                not isinstance(quantizer, MinMaxQuantizer) or 'forward' in quantizer.__dict__:
            return None
        mn, mx = quantizer.min, quantizer.max
        # pylint: disable=protected-access
        # (the stream is part of the key: see StaticGridQuantWrapper._param_cache_key)
        stream = ops.current_stream_handle(param.device) if param.is_cuda else None
        return (stream, id(param), param._version, param.data_ptr(), param.dtype, tuple(param.shape), id(quantizer),
                id(mn), mn._version, id(mx), mx._version, quantizer.qmin, quantizer.qmax, quantizer.symmetric,
                quantizer.block_size)

    def _patch_quantized_parameters(self):
        stack = contextlib.ExitStack()
        kept = self.__dict__.setdefault('_kept_quantized_parameters', {})
        for param_name, param_quantizer in self.param_quantizers.items():
            if param_quantizer and param_quantizer.is_initialized():
                param = getattr(self, param_name)
                key = self._kept_parameter_key(param, param_quantizer)
                entry = kept.get(param_name) if key is not None else None
                if entry is not None and entry[0] == key and entry[1] is param:
                    quantized = entry[2]
                else:
                    quantized = param_quantizer(param)
                    if key is not None:
                        kept[param_name] = (key, param, quantized)
                    else:
                        kept.pop(param_name, None)
                stack.enter_context(patch_attr(self, param_name, quantized))
        return stack

    def _compute_param_encodings(self, overwrite: bool):
        for param_name, param_quantizer in self.param_quantizers.items():
            if not param_quantizer or not param_quantizer._allow_overwrite:  # pylint: disable=protected-access
                continue
            if not param_quantizer.is_initialized() or overwrite:
                param = getattr(self, param_name)
                if param is not None:
                    with patch_attr(param_quantizer, "forward", _no_op), param_quantizer.compute_encodings():
                        _ = param_quantizer(param)

    def compute_param_encodings(self):
        self._compute_param_encodings(overwrite=True)

    @contextlib.contextmanager
    def compute_encodings(self):
        """Every quantizer of the layer observes what passes through it and computes its encoding on exit; input and
        output quantizers are pass-through meanwhile (as in the v1 simulation)."""
        self._compute_param_encodings(overwrite=True)
        with contextlib.ExitStack() as stack:
            for quantizer in itertools.chain(self.input_quantizers, self.output_quantizers):
                if not isinstance(quantizer, MinMaxQuantizer) or not quantizer._allow_overwrite:  # pylint: disable=protected-access
                    continue
                stack.enter_context(patch_attr(quantizer, 'forward', _no_op))
                stack.enter_context(quantizer.compute_encodings())
            yield

    # ------------------------------------------------------------------------------- encodings in the exported format
    def export_param_encodings(self):
        """{parameter name: list of encoding dicts, or None without an initialised quantizer}"""
        return {name: (q.get_legacy_encodings() if q is not None else None)
                for name, q in self.param_quantizers.items()}

    def export_input_encodings(self):
        return [q.get_legacy_encodings() if q is not None else None for q in self.input_quantizers]

    def export_output_encodings(self):
        return [q.get_legacy_encodings() if q is not None else None for q in self.output_quantizers]

    @staticmethod
    def _import_into(slots, keys, what, encodings, strict, partial, requires_grad, allow_overwrite):
        """Common part of the three imports (reference aimet_torch/v2/nn/base.py:282-330, :332-380, :395-470 without
        vector encodings).  `slots` is the ModuleList / ModuleDict of quantizers and `keys` its (slot key, key in
        `encodings`) pairs.  A frozen quantizer is skipped; a slot without an entry is left alone when `partial`, else
        emptied; an entry for an empty slot raises when `strict`."""
        for slot, key in keys:
            quantizer = slots[slot]
            if quantizer is not None and not quantizer._allow_overwrite:              # pylint: disable=protected-access
                continue
            entry = encodings.get(key)
            if not entry:
                if not partial:
                    slots[slot] = None
                continue
            if quantizer is None:
                if strict:
                    raise RuntimeError(f"Failed to import {what} {key}: no quantizer present.")
                continue
            quantizer.set_legacy_encodings([entry] if isinstance(entry, dict) else entry)
            if requires_grad is not None:
                quantizer.requires_grad_(requires_grad)
            quantizer.allow_overwrite(allow_overwrite)

    def import_param_encodings(self, encodings, strict: bool, partial: bool, requires_grad, allow_overwrite: bool):
        """encodings: {parameter name: [dict per channel]}"""
        keys = [(name, name) for name in self.param_quantizers]
        self._import_into(self.param_quantizers, keys, "encoding for parameter", encodings, strict, partial,
                          requires_grad, allow_overwrite)

    def import_input_encodings(self, encodings, strict: bool, partial: bool, requires_grad, allow_overwrite: bool):
        """encodings: {'0': dict, '1': dict, ...} by input index"""
        keys = [(i, str(i)) for i in range(len(self.input_quantizers))]
        self._import_into(self.input_quantizers, keys, "input encoding at index", encodings, strict, partial,
                          requires_grad, allow_overwrite)

    def import_output_encodings(self, encodings, strict: bool, partial: bool, requires_grad, allow_overwrite: bool):
        """encodings: {'0': dict, '1': dict, ...} by output index"""
        keys = [(i, str(i)) for i in range(len(self.output_quantizers))]
        self._import_into(self.output_quantizers, keys, "output encoding at index", encodings, strict, partial,
                          requires_grad, allow_overwrite)

    def get_original_module(self) -> nn.Module:
        """A plain module of the base class sharing this module's parameters and buffers."""
        base_cls = type(self).qcls_to_cls[type(self)]
        module = base_cls.__new__(base_cls)
        module.__dict__ = {k: v for k, v in self.__dict__.items()}
        module._modules = {k: v for k, v in self._modules.items()
                           if k not in ('param_quantizers', 'input_quantizers', 'output_quantizers')}
        module._parameters = dict(self._parameters)
        module._buffers = dict(self._buffers)
        return module

    # Taking quantizers out: each call empties the named slots at once and returns an object that puts the former
    # quantizers back when used as a context manager (or as a decorator); ignored, the slots stay empty
    # (reference :505-575).
    def _remove_input_quantizers(self, indices=None):
        return _emptied(self.input_quantizers, range(len(self.input_quantizers)), indices, int)

    def _remove_output_quantizers(self, indices=None):
        return _emptied(self.output_quantizers, range(len(self.output_quantizers)), indices, int)

    def _remove_param_quantizers(self, keys=None):
        return _emptied(self.param_quantizers, self.param_quantizers.keys(), keys, str)

    def _remove_activation_quantizers(self):
        return _all_of(self._remove_output_quantizers(), self._remove_input_quantizers())

    def _remove_all_quantizers(self):
        return _all_of(self._remove_activation_quantizers(), self._remove_param_quantizers())

    @classmethod
    def implements(cls, module_cls):
        """Decorator registering the quantized definition of a base class."""
        def wrapper(quantized_cls):
            cls.cls_to_qcls[module_cls] = quantized_cls
            cls.qcls_to_cls[quantized_cls] = module_cls
            return quantized_cls
        return wrapper

    @classmethod
    def from_module(cls, module: nn.Module):
        """Quantized module with the attributes, parameters and buffers of `module` (shared, not copied)."""
        module_cls = type(module)
        qtzn_module_cls = cls.cls_to_qcls.get(module_cls, None)
        if not qtzn_module_cls:
            raise RuntimeError(f'The quantized module definition of {module_cls} is not registered. '
                               f'Please register the quantized module definition of {module_cls} '
                               f'using `@{cls.__name__}.implements({module_cls.__name__})` decorator.')
        qtzn_module = cls.__new__(qtzn_module_cls)
        qtzn_module.__dict__ = module.__dict__.copy()
        qtzn_module._modules = module._modules.copy()
        qtzn_module._parameters = module._parameters.copy()
        qtzn_module._buffers = module._buffers.copy()
        qtzn_module.__quant_init__()
        return qtzn_module


class QuantizationMixin(BaseQuantizationMixin):
    """Fake-quantization: quantize-dequantize inputs, parameters and outputs around the base class' forward."""

    cls_to_qcls = {}
    qcls_to_cls = {}

    def forward(self, *args, **kwargs):
        args = list(args)
        for i, quantizer in enumerate(self.input_quantizers):
            if quantizer and i < len(args) and isinstance(args[i], torch.Tensor) and args[i].is_floating_point():
                args[i] = quantizer(args[i])
        if self._relu_is_absorbed(args, kwargs):
            output = args[0]
        else:
            with self._patch_quantized_parameters():
                output = super().forward(*args, **kwargs)
        outputs = list(output) if isinstance(output, (tuple, list)) else [output]
        for i, quantizer in enumerate(self.output_quantizers):
            if quantizer and i < len(outputs) and isinstance(outputs[i], torch.Tensor) and \
                    outputs[i].is_floating_point():
                outputs[i] = quantizer(outputs[i])
        return type(output)(outputs) if isinstance(output, (tuple, list)) else outputs[0]

    def _relu_is_absorbed(self, args, kwargs) -> bool:
        """True when running the ReLU would not change this module's result, so its pass over the activations (as
        much traffic as the quantizer's) is left out: the output quantizer's grid starts exactly at zero, and
        quantize-dequantize then maps every negative input to zero and leaves NaN a NaN, as it does after the ReLU --
        identical element for element.  Only without autograd (the straight-through mask of the pre-activation
        differs at zero) and for a ReLU that is not in-place (an in-place one also rewrites its input, which other
        readers of that tensor may rely on)."""
        if type(self).qcls_to_cls.get(type(self)) is not nn.ReLU or self.inplace or kwargs or \
                torch.is_grad_enabled() or len(args) != 1 or len(self.output_quantizers) != 1:
            return False
        quantizer, tensor = self.output_quantizers[0], args[0]
        if type(quantizer).__name__ != 'QuantizeDequantize' or 'forward' in quantizer.__dict__ or \
                not isinstance(tensor, torch.Tensor) or not tensor.is_floating_point() or not tensor.is_cuda:
            return False
        return quantizer.is_initialized() and quantizer.lower_bound_is_zero()

    @classmethod
    def wrap(cls, module_cls: Type[nn.Module]):
        """Creates (and registers) the quantized class of a single-input, single-output module class."""
        if module_cls in cls.cls_to_qcls:
            return cls.cls_to_qcls[module_cls]
        quantized_cls = type(f"Quantized{module_cls.__name__}", (cls, module_cls), {"_wrapped_by": (cls, module_cls)})
        return cls.implements(module_cls)(quantized_cls)

    def __reduce_ex__(self, protocol):
        # A class that wrap() made has no name to import it by: pickles (and copies) name the mixin and the base class
        # instead, and the class is made again where they are loaded.
        made_by = type(self).__dict__.get("_wrapped_by")
        if made_by is None:
            return super().__reduce_ex__(protocol)
        return _rebuild_wrapped, made_by, self.__getstate__()


def _emptied(slots, every_key, keys, one_key_type):
    """Sets slots[key] = None for the keys named (one key, several, or None for all of them)."""
    if keys is None:
        keys = every_key
    elif isinstance(keys, one_key_type):
        keys = (keys,)
    keys = list(keys)
    former = [(key, slots[key]) for key in keys]                    # a bad key raises before anything is changed

    def put_back():
        for key, quantizer in former:
            slots[key] = quantizer
    for key in keys:
        slots[key] = None
    return _ContextManager(action=lambda: None, cleanup=put_back)


def _all_of(*undo):
    return _ContextManager(action=lambda: None, cleanup=lambda: [u._cleanup() for u in undo])  # pylint: disable=protected-access


def _rebuild_wrapped(mixin_cls, module_cls):
    quantized_cls = mixin_cls.wrap(module_cls)
    return quantized_cls.__new__(quantized_cls)


for _cls in (nn.Linear, nn.Conv1d, nn.Conv2d, nn.Conv3d, nn.ConvTranspose1d, nn.ConvTranspose2d, nn.ConvTranspose3d,
             nn.ReLU, nn.ReLU6, nn.Sigmoid, nn.Tanh, nn.Hardtanh, nn.MaxPool2d, nn.AvgPool2d, nn.AdaptiveAvgPool2d,
             nn.Flatten, nn.Dropout, nn.BatchNorm2d, nn.LayerNorm, nn.GELU, nn.SiLU, nn.Softmax):
    QuantizationMixin.wrap(_cls)

QuantizedLinear = QuantizationMixin.cls_to_qcls[nn.Linear]
QuantizedConv2d = QuantizationMixin.cls_to_qcls[nn.Conv2d]
QuantizedConvTranspose2d = QuantizationMixin.cls_to_qcls[nn.ConvTranspose2d]
QuantizedReLU = QuantizationMixin.cls_to_qcls[nn.ReLU]
