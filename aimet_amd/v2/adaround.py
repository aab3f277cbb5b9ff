"""AdaRound on the v2 quantized modules.

Mirrors TrainingExtensions/torch/src/python/aimet_torch/v2/adaround.py: the Adaround class with the v2 overrides
(_get_quantsim :60-65, _get_adaround_wrapper :67-69, _remove_quantization_wrappers :71-77, _get_quant_wrapper :79-95,
_compute_param_encodings :97-114, _validate_quant_module_for_adaround :116-119,
_check_input_output_quantizers_for_adaround :121-126, _get_lowest_weight_bw :128-140) and AdaroundWrapper (:142-191):
delta / offset come from the weight quantizer's scale / offset and a signed quantizer uses the signed integer grid
[-2^(bw-1), 2^(bw-1) - 1].  The optimisation loop and its kernels are those of the v1 path.
"""
import contextlib
import itertools
from typing import Tuple, Union

import torch
from torch import nn

from ..common.defs import QuantScheme
from ..v1.adaround.adaround_weight import Adaround as V1Adaround, AdaroundParameters as V1AdaroundParameters
from ..v1.adaround.adaround_weight import AdaroundSupportedModules
from ..v1.adaround.adaround_wrapper import AdaroundWrapper as V1AdaroundWrapper
from .nn import BaseQuantizationMixin
from .quantization.affine.quantizer import MinMaxQuantizer
from .quantsim import QuantizationSimModel


class AdaroundWrapper(V1AdaroundWrapper):
    """AdaRound wrapper of a v2 quantized module."""

    def __init__(self, module: BaseQuantizationMixin):  # pylint: disable=super-init-not-called
        torch.nn.Module.__init__(self)
        assert self.weight_name in module.param_quantizers
        self.module_to_wrap = module
        self._init_param()

    def forward(self, *args, **kwargs):
        """Runs the quantized module with its weight replaced by the adarounded weight."""
        if not self._is_weight_quantizer_enabled():
            return self.module_to_wrap(*args, **kwargs)
        param = getattr(self.module_to_wrap, self.weight_name)
        saved = param.data
        with self._disable_weight_quantizer():
            param.data = self.apply_adaround(saved).detach()
            try:
                return self.module_to_wrap(*args, **kwargs)
            finally:
                param.data = saved

    @contextlib.contextmanager
    def _disable_weight_quantizer(self):
        weight_quantizer = self.module_to_wrap.param_quantizers[self.weight_name]
        self.module_to_wrap.param_quantizers[self.weight_name] = None
        try:
            yield
        finally:
            self.module_to_wrap.param_quantizers[self.weight_name] = weight_quantizer

    def _is_weight_quantizer_enabled(self) -> bool:
        return bool(self.module_to_wrap.param_quantizers[self.weight_name])

    def get_original_module(self) -> torch.nn.Module:
        return self.module_to_wrap

    def _get_weight_quantizer_channel_axis(self) -> int:
        quantizer = self.module_to_wrap.param_quantizers[self.weight_name]
        shape = quantizer.shape
        padded = (1,) * (self.weight.dim() - len(shape)) + tuple(shape)
        for idx, dim in enumerate(padded):
            if dim != 1:
                return idx
        return 0

    def _get_weight_quantizer_delta_and_offset(self) -> Tuple[torch.Tensor, torch.Tensor]:
        quantizer = self.module_to_wrap.param_quantizers[self.weight_name]
        with torch.no_grad():
            scale = quantizer.get_scale().detach().to(torch.float32).reshape(-1)
            offset = quantizer.get_offset().detach().to(torch.float32).reshape(-1)
        return scale, offset

    def _get_weight_quantizer_bitwidth(self) -> int:
        return self.module_to_wrap.param_quantizers[self.weight_name].bitwidth

    def _init_param(self):
        super()._init_param()
        quantizer = self.module_to_wrap.param_quantizers[self.weight_name]
        if quantizer.signed:
            self.clip_max = 2 ** (self.bitwidth - 1) - 1
            self.clip_min = - 2 ** (self.bitwidth - 1)


class AdaroundParameters(V1AdaroundParameters):
    """Configuration parameters for Adaround."""


class Adaround(V1Adaround):
    """Weight-rounding mechanism for post-training quantization, on the v2 quantized modules."""

    @staticmethod
    def _get_quantsim(model: nn.Module, dummy_input, quant_scheme: QuantScheme, default_param_bw: int,
                      config_file: str):
        return QuantizationSimModel(model, dummy_input=dummy_input, quant_scheme=quant_scheme,
                                    default_param_bw=default_param_bw, config_file=config_file)

    @staticmethod
    def _get_adaround_wrapper(quant_module: BaseQuantizationMixin):
        return AdaroundWrapper(quant_module)

    @classmethod
    def _remove_quantization_wrappers(cls, module: nn.Module):
        for module_name, module_ref in module.named_children():
            if isinstance(module_ref, BaseQuantizationMixin):
                setattr(module, module_name, module_ref.get_original_module())
            else:
                cls._remove_quantization_wrappers(module_ref)

    @staticmethod
    def _get_quant_wrapper(quant_sim_model: nn.Module, module_name: str) -> Union[BaseQuantizationMixin, None]:
        for name, module in quant_sim_model.named_modules():
            if name == module_name and isinstance(module, BaseQuantizationMixin):
                return module
        return None

    @staticmethod
    def _compute_param_encodings(quant_sim: QuantizationSimModel):
        for quant_module in quant_sim.model.modules():
            if isinstance(quant_module, BaseQuantizationMixin):
                # AdaRound requires input and output quantizers to be disabled
                quant_module.input_quantizers = nn.ModuleList([None for _ in quant_module.input_quantizers])
                quant_module.output_quantizers = nn.ModuleList([None for _ in quant_module.output_quantizers])
                for name, param_quantizer in quant_module.param_quantizers.items():
                    if not param_quantizer:
                        continue
                    with param_quantizer.compute_encodings():
                        _ = param_quantizer(getattr(quant_module, name))

    @staticmethod
    def _validate_quant_module_for_adaround(quant_module: BaseQuantizationMixin):
        assert quant_module.param_quantizers['weight'], '%s does not have weight parameter.' % quant_module
        assert quant_module.param_quantizers['weight'].is_initialized(), '%s encoding needs to be set.' % quant_module

    @staticmethod
    def _check_input_output_quantizers_for_adaround(quant_model: nn.Module):
        for module in quant_model.modules():
            if isinstance(module, BaseQuantizationMixin):
                for quantizer in itertools.chain(module.input_quantizers, module.output_quantizers):
                    assert quantizer is None

    @staticmethod
    def _get_lowest_weight_bw(quant_model: nn.Module):
        return min(quantizer.bitwidth for module in quant_model.modules() if isinstance(module, BaseQuantizationMixin)
                   for quantizer in module.param_quantizers.values() if isinstance(quantizer, MinMaxQuantizer))

    @classmethod
    def _export_encodings_to_json(cls, path: str, filename_prefix: str, quant_sim: QuantizationSimModel):
        import json
        import os
        param_encodings = {}
        for name, quant_module in quant_sim.model.named_modules():
            if isinstance(quant_module, BaseQuantizationMixin) and isinstance(quant_module, AdaroundSupportedModules):
                quantizer = quant_module.param_quantizers['weight'] if 'weight' in quant_module.param_quantizers \
                    else None
                if quantizer is not None and quantizer.is_initialized():
                    param_encodings[name + '.weight'] = quantizer.get_legacy_encodings()
        os.makedirs(os.path.abspath(path), exist_ok=True)
        with open(os.path.join(path, filename_prefix + '.encodings'), 'w') as encoding_fp:
            json.dump({'param_encodings': param_encodings}, encoding_fp, sort_keys=True, indent=4)
