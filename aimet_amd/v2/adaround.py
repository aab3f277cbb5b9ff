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
import json
import os
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


def _quantized_modules(root: nn.Module):
    """Every v2 quantized module below (and including) `root`."""
    return (m for m in root.modules() if isinstance(m, BaseQuantizationMixin))


class AdaroundWrapper(V1AdaroundWrapper):
    """AdaRound wrapper of a v2 quantized module: the grid comes from the weight quantizer's scale / offset."""

    def __init__(self, module: BaseQuantizationMixin):  # pylint: disable=super-init-not-called
        torch.nn.Module.__init__(self)
        assert self.weight_name in module.param_quantizers
        self.module_to_wrap = module
        self._init_param()

    # the weight quantizer of the wrapped module, wherever a hook below needs it
    @property
    def _weight_quantizer(self):
        return self.module_to_wrap.param_quantizers[self.weight_name]

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
        slots, parked = self.module_to_wrap.param_quantizers, self._weight_quantizer
        slots[self.weight_name] = None
        try:
            yield
        finally:
            slots[self.weight_name] = parked

    def _is_weight_quantizer_enabled(self) -> bool:
        return self._weight_quantizer is not None

    def get_original_module(self) -> torch.nn.Module:
        """The quantized module itself: there is no separate wrapped module in v2."""
        return self.module_to_wrap

    def _get_weight_quantizer_channel_axis(self) -> int:
        # the quantizer's shape broadcasts against the weight from the right; the first axis along which it has more
        # than one entry is the channel axis (0 for a per-tensor quantizer)
        lead = self.weight.dim() - len(self._weight_quantizer.shape)
        return next((lead + axis for axis, size in enumerate(self._weight_quantizer.shape) if size != 1), 0)

    def _get_weight_quantizer_delta_and_offset(self) -> Tuple[torch.Tensor, torch.Tensor]:
        with torch.no_grad():
            flat = [t.detach().to(torch.float32).reshape(-1)
                    for t in (self._weight_quantizer.get_scale(), self._weight_quantizer.get_offset())]
        return flat[0], flat[1]

    def _get_weight_quantizer_bitwidth(self) -> int:
        return self._weight_quantizer.bitwidth

    def _init_param(self):
        super()._init_param()
        if self._weight_quantizer.signed:
            # signed integer grid [-2^(bw-1), 2^(bw-1) - 1] instead of v1's [0, 2^bw - 1]
            half = 2 ** (self.bitwidth - 1)
            self.clip_min, self.clip_max = -half, half - 1


class AdaroundParameters(V1AdaroundParameters):
    """Configuration parameters for Adaround."""


class Adaround(V1Adaround):
    """Weight-rounding mechanism for post-training quantization, on the v2 quantized modules."""

    @staticmethod
    def _get_quantsim(model: nn.Module, dummy_input, quant_scheme: QuantScheme, default_param_bw: int,
                      config_file: str):
        return QuantizationSimModel(model, dummy_input, quant_scheme, default_param_bw=default_param_bw,
                                    config_file=config_file)

    @staticmethod
    def _get_adaround_wrapper(quant_module: BaseQuantizationMixin):
        return AdaroundWrapper(quant_module)

    @classmethod
    def _remove_quantization_wrappers(cls, module: nn.Module):
        for child_name, child in list(module.named_children()):
            if not isinstance(child, BaseQuantizationMixin):
                cls._remove_quantization_wrappers(child)
                continue
            setattr(module, child_name, child.get_original_module())

    @staticmethod
    def _get_quant_wrapper(quant_sim_model: nn.Module, module_name: str) -> Union[BaseQuantizationMixin, None]:
        found = dict(quant_sim_model.named_modules()).get(module_name)
        return found if isinstance(found, BaseQuantizationMixin) else None

    @staticmethod
    def _supported_wrappers(quant_sim_model: nn.Module):
        return ((n, m) for n, m in quant_sim_model.named_modules()
                if isinstance(m, BaseQuantizationMixin) and isinstance(m, AdaroundSupportedModules))

    @staticmethod
    def _compute_param_encodings(quant_sim: QuantizationSimModel):
        for quantized in _quantized_modules(quant_sim.model):
            # only parameters are quantized while AdaRound runs: activation quantizers are taken out
            quantized.input_quantizers = nn.ModuleList([None] * len(quantized.input_quantizers))
            quantized.output_quantizers = nn.ModuleList([None] * len(quantized.output_quantizers))
            for param_name, quantizer in quantized.param_quantizers.items():
                if quantizer is not None:
                    with quantizer.compute_encodings():
                        quantizer(getattr(quantized, param_name))

    @staticmethod
    def _validate_quant_module_for_adaround(quant_module: BaseQuantizationMixin):
        weight_quantizer = quant_module.param_quantizers['weight']
        assert weight_quantizer, f'{quant_module} does not have weight parameter.'
        assert weight_quantizer.is_initialized(), f'{quant_module} encoding needs to be set.'

    @staticmethod
    def _check_input_output_quantizers_for_adaround(quant_model: nn.Module):
        leftover = [q for m in _quantized_modules(quant_model)
                    for q in itertools.chain(m.input_quantizers, m.output_quantizers) if q is not None]
        assert not leftover

    @staticmethod
    def _get_lowest_weight_bw(quant_model: nn.Module):
        return min(quantizer.bitwidth for module in _quantized_modules(quant_model)
                   for quantizer in module.param_quantizers.values() if isinstance(quantizer, MinMaxQuantizer))

    @classmethod
    def _export_encodings_to_json(cls, path: str, filename_prefix: str, quant_sim: QuantizationSimModel):
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
