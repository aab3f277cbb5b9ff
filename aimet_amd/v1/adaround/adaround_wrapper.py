"""AdaRound wrapper of a quantization wrapper.

Mirrors TrainingExtensions/torch/src/python/aimet_torch/v1/adaround/adaround_wrapper.py (AdaroundWrapper :92-224):
same attributes (alpha, use_soft_rounding, clip_min / clip_max, bitwidth, broadcasted_delta / broadcasted_offset,
weight) and the same apply_adaround arithmetic, computed by one HIP kernel instead of about ten ATen kernels.
apply_adaround is differentiable w.r.t. alpha through a custom autograd function whose backward is one kernel as
well.
"""
import contextlib
from typing import Tuple

import torch

from ... import ops
from ...common.AimetTensorQuantizer import AimetTensorQuantizer
from ..qc_quantize_op import QcQuantizeWrapper
from ..quantsim_straight_through_grad import broadcast_to_tensor
from ..tensor_quantizer import StaticGridPerChannelQuantizer


class _ApplyAdaround(torch.autograd.Function):
    """W' = (clamp(floor(W / delta) + h(alpha) - offset, clip_min, clip_max) + offset) * delta."""

    @staticmethod
    def forward(ctx, weight, alpha, wrapper):  # pylint: disable=arguments-differ
        ctx.wrapper = wrapper
        ctx.save_for_backward(weight, alpha)
        return ops.adaround_soft_round(weight, alpha, wrapper.num_channel, wrapper.n_per_channel, wrapper.delta,
                                       wrapper.offset, wrapper.clip_min, wrapper.clip_max,
                                       wrapper.use_soft_rounding)

    @staticmethod
    def backward(ctx, grad_out):  # pylint: disable=arguments-differ
        weight, alpha = ctx.saved_tensors
        w = ctx.wrapper
        if not w.use_soft_rounding:
            return None, torch.zeros_like(alpha), None
        grad = ops.adaround_bwd(weight, grad_out.contiguous(), alpha, w.num_channel, w.n_per_channel, w.delta,
                                w.offset, w.clip_min, w.clip_max)
        return None, grad, None


class AdaroundWrapper(torch.nn.Module):
    """Holds the rounding parameter alpha of one quantized module's weight."""

    weight_name = 'weight'

    def __init__(self, module: QcQuantizeWrapper):
        super().__init__()
        assert self.weight_name in module.param_quantizers
        self.module_to_wrap = module
        self._init_param()

    def forward(self, *args, **kwargs):
        """Runs the wrapped module with its weight replaced by the adarounded weight."""
        original_module = self.get_original_module()
        param = getattr(original_module, self.weight_name)
        if not self._is_weight_quantizer_enabled():
            return self.module_to_wrap.forward(*args, **kwargs)
        saved = param.data
        with self._disable_weight_quantizer():
            param.data = self.apply_adaround(saved).detach()
            try:
                return self.module_to_wrap.forward(*args, **kwargs)
            finally:
                param.data = saved

    def get_original_module(self) -> torch.nn.Module:
        # pylint: disable=protected-access
        return self.module_to_wrap._module_to_wrap

    @property
    def weight(self) -> torch.Tensor:
        return getattr(self.get_original_module(), self.weight_name)

    def apply_adaround(self, tensor: torch.Tensor) -> torch.Tensor:
        """Adarounds `tensor` (the weight); float32 arithmetic, result in the dtype of `tensor`."""
        input_dtype = tensor.dtype
        if not tensor.is_cuda:
            raise RuntimeError("AdaroundWrapper.apply_adaround (aimet_amd) computes on the GPU only")
        weight = tensor.detach().to(torch.float32).contiguous()
        alpha = self.alpha if self.alpha.device == tensor.device else self.alpha.to(tensor.device)
        out = _ApplyAdaround.apply(weight, alpha, self)
        return out.to(input_dtype)

    @contextlib.contextmanager
    def _disable_weight_quantizer(self):
        weight_quantizer = self.module_to_wrap.param_quantizers[self.weight_name]
        is_enabled = weight_quantizer.enabled
        weight_quantizer.enabled = False
        try:
            yield
        finally:
            weight_quantizer.enabled = is_enabled

    def _is_weight_quantizer_enabled(self) -> bool:
        return self.module_to_wrap.param_quantizers[self.weight_name].enabled

    def _get_weight_quantizer_channel_axis(self) -> int:
        quantizer = self.module_to_wrap.param_quantizers[self.weight_name]
        if isinstance(quantizer, StaticGridPerChannelQuantizer):
            return quantizer._ch_axis  # pylint: disable=protected-access
        return 0

    def _get_weight_quantizer_delta_and_offset(self) -> Tuple[torch.Tensor, torch.Tensor]:
        """float32 device vectors (one entry per channel, or one entry for a per-tensor encoding)."""
        quantizer = self.module_to_wrap.param_quantizers[self.weight_name]
        device = self.weight.device
        if isinstance(quantizer.encoding, list):
            return AimetTensorQuantizer.makeDeltaOffsetTensor(device, quantizer.encoding)
        vec = torch.tensor([quantizer.encoding.delta, quantizer.encoding.offset], dtype=torch.float32).to(device)
        return vec[0:1], vec[1:2]

    def _get_weight_quantizer_bitwidth(self) -> int:
        return self.module_to_wrap.param_quantizers[self.weight_name].bitwidth

    def _init_param(self):
        weight = self.weight
        delta, offset = self._get_weight_quantizer_delta_and_offset()
        self.delta, self.offset = delta.contiguous(), offset.contiguous()
        ch_axis = self._get_weight_quantizer_channel_axis()
        if self.delta.numel() == 1:
            self.num_channel, self.n_per_channel = 1, max(1, weight.numel())
        else:
            sizes = list(weight.shape) + [1]
            self.num_channel = sizes[ch_axis]
            self.n_per_channel = 1
            for s in sizes[ch_axis + 1:]:
                self.n_per_channel *= s
            assert self.delta.numel() == self.num_channel
        self.broadcasted_delta = broadcast_to_tensor(weight, self.delta, ch_axis)
        self.broadcasted_offset = broadcast_to_tensor(weight, self.offset, ch_axis)
        self.alpha = self._generate_alpha_parameter(weight)
        self.bitwidth = self._get_weight_quantizer_bitwidth()
        self.use_soft_rounding = True
        self.clip_max = 2 ** self.bitwidth - 1
        self.clip_min = 0

    def _generate_alpha_parameter(self, tensor: torch.Tensor) -> torch.nn.Parameter:
        """alpha = -log((zeta - gamma) / (frac(w / delta) - gamma) - 1), float32 whatever the weight's dtype."""
        if not tensor.is_cuda:
            raise RuntimeError("AdaroundWrapper (aimet_amd) needs the module on the GPU")
        alpha = ops.adaround_init_alpha(tensor.detach().to(torch.float32).contiguous(), self.num_channel,
                                        self.n_per_channel, self.delta)
        return torch.nn.Parameter(alpha, requires_grad=True)
