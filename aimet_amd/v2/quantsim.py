"""Minimal v2 QuantizationSimModel: every supported leaf module becomes a quantized module with QuantizeDequantize
quantizers (reference: TrainingExtensions/torch/src/python/aimet_torch/v2/quantsim/quantsim.py, which builds on the v1
configurator; here only the defaults are implemented: symmetric parameter quantizers for weights, asymmetric output
quantizers for every layer, an input quantizer for the model inputs, per-tensor or per-output-channel weights).
"""
import copy
from typing import Tuple, Union

import torch
from torch import nn

from ..common.defs import QuantScheme
from .nn import BaseQuantizationMixin, QuantizationMixin
from .quantization.affine import QuantizeDequantize
from .quantization.encoding_analyzer import MinMaxEncodingAnalyzer, SqnrEncodingAnalyzer


def _analyzer(quant_scheme: QuantScheme, shape):
    if quant_scheme == QuantScheme.post_training_tf:
        return MinMaxEncodingAnalyzer(shape)
    if quant_scheme == QuantScheme.post_training_tf_enhanced:
        return SqnrEncodingAnalyzer(shape)
    raise ValueError(f"quant_scheme {quant_scheme} is not implemented (tf and tf_enhanced are)")


class QuantizationSimModel:
    """Replaces the supported leaf modules of a copy of `model` by their quantized counterparts."""

    def __init__(self, model: nn.Module, dummy_input: Union[torch.Tensor, Tuple] = None,
                 quant_scheme: Union[str, QuantScheme] = QuantScheme.post_training_tf_enhanced,
                 default_output_bw: int = 8, default_param_bw: int = 8, in_place: bool = False,
                 per_channel_quantization: bool = False, config_file: str = None):
        if config_file is not None:
            raise NotImplementedError("configuration files are implemented by the v1 QuantizationSimModel only")
        if isinstance(quant_scheme, str):
            quant_scheme = {'tf': QuantScheme.post_training_tf,
                            'tf_enhanced': QuantScheme.post_training_tf_enhanced}[quant_scheme]
        self._quant_scheme = quant_scheme
        self.model = model if in_place else copy.deepcopy(model)
        first_param = next(self.model.parameters(), None)
        self._device = first_param.device if first_param is not None else torch.device("cuda")
        self._convert(self.model, default_output_bw, default_param_bw, per_channel_quantization)
        first = next((m for m in self.model.modules() if isinstance(m, BaseQuantizationMixin)), None)
        if first is not None:
            first.input_quantizers[0] = self._make((), default_output_bw, False, first)

    def _make(self, shape, bitwidth, symmetric, like: nn.Module):
        q = QuantizeDequantize(shape, bitwidth=bitwidth, symmetric=symmetric,
                               encoding_analyzer=_analyzer(self._quant_scheme, shape))
        param = next(like.parameters(), None)
        return q.to(param.device if param is not None else self._device)

    def _convert(self, module: nn.Module, output_bw: int, param_bw: int, per_channel: bool):
        for name, child in list(module.named_children()):
            if type(child) in QuantizationMixin.cls_to_qcls and not list(child.children()):
                q = QuantizationMixin.from_module(child)
                for pname, param in child.named_parameters(recurse=False):
                    if pname != 'weight':
                        continue            # biases are not quantized by default
                    shape = ()
                    if per_channel and param.dim() > 1:
                        axis = 1 if isinstance(child, (nn.ConvTranspose1d, nn.ConvTranspose2d,
                                                       nn.ConvTranspose3d)) else 0
                        shape = tuple(d if a == axis else 1 for a, d in enumerate(param.shape))
                    q.param_quantizers[pname] = self._make(shape, param_bw, True, child)
                if not isinstance(child, (nn.Flatten, nn.Dropout)):
                    q.output_quantizers[0] = self._make((), output_bw, False, child)
                setattr(module, name, q)
            else:
                self._convert(child, output_bw, param_bw, per_channel)

    def qmodules(self):
        for name, module in self.model.named_modules():
            if isinstance(module, BaseQuantizationMixin):
                yield name, module

    def compute_encodings(self, forward_pass_callback, forward_pass_callback_args):
        """Runs the callback with every quantizer observing, then fixes the encodings."""
        import contextlib
        with contextlib.ExitStack() as stack:
            for _, module in self.qmodules():
                stack.enter_context(module.compute_encodings())
            was_training = self.model.training
            self.model.eval()
            try:
                with torch.no_grad():
                    forward_pass_callback(self.model, forward_pass_callback_args)
            finally:
                self.model.train(was_training)
