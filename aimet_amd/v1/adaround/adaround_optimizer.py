"""Per-layer optimisation of the weight rounding.

Mirrors AdaroundOptimizer of TrainingExtensions/torch/src/python/aimet_torch/v1/adaround/adaround_optimizer.py
(adaround_module :66-113, _optimize_rounding :115-222, _compute_recons_metrics :224-251,
_compute_output_with_adarounded_weights :253-283).  Per iteration the reference runs apply_adaround's elementwise ops,
the layer, both losses, autograd through all of it and torch.optim.Adam -- some forty kernels over weight-shaped
tensors.  Here an iteration is: one soft-rounding kernel (W, alpha -> W'), the layer forward and its weight gradient
(torch, on W' as a leaf), and one fused kernel (dW', W, alpha, moments -> alpha, moments) that applies the chain rule
of the soft rounding, adds the rounding regulariser's gradient and performs the Adam update.  The batch indices are
drawn with torch.randperm on the host exactly as the reference draws them, so a seeded run visits the same batches.
"""
from typing import Any, Callable, Tuple, Union

import torch
import torch.nn.functional as functional

from ... import ops
from .activation_sampler import ActivationSampler
from .adaround_loss import AdaroundHyperParameters, AdaroundLoss
from .adaround_wrapper import AdaroundWrapper

BATCH_SIZE = 32
ADAM_LR, ADAM_BETAS, ADAM_EPS = 1e-3, (0.9, 0.999), 1e-8      # torch.optim.Adam defaults, as the reference uses


class AdaroundOptimizer:
    """Optimizes the weight rounding of a quantized wrapper module."""

    # Linear layers and 1x1 convolutions whose shape the MFMA-fused kernels take (out % 32 == 0, in % 128 == 0,
    # 32 / 64 / 128 / 256 rows per iteration, no activation or ReLU) use them; everything else runs soft-round kernel +
    # torch layer + fused backward/Adam kernel
    use_fused_linear = True
    # rows per iteration up to which the fused kernels are the faster path: on a [4096, 4096] layer they take 0.105 /
    # 0.136 / 0.188 / 0.321 ms per iteration at 32 / 64 / 128 / 256 rows against 0.170 / 0.186 / 0.236 / 0.289 ms for
    # the general path (the kernels themselves take up to 256)
    fused_rows_limit = 128
    use_int8_floor = True    # store floor(W / delta) as int8 / int16 for the fused Linear path when the grid allows it

    @classmethod
    def adaround_module(cls, module: torch.nn.Module, quant_module: AdaroundWrapper, orig_model: torch.nn.Module,
                        quant_model: torch.nn.Module, act_func: Union[torch.nn.Module, None], cached_dataset,
                        forward_fn: Callable[[torch.nn.Module, Any], Any], opt_params: AdaroundHyperParameters,
                        cached_quant_dataset=None):
        # pylint: disable=too-many-arguments
        assert isinstance(quant_module, AdaroundWrapper), '%s is not adaround wrapper module.' % quant_module
        cls._optimize_rounding(module, quant_module, orig_model, quant_model, act_func, cached_dataset, forward_fn,
                               opt_params, cached_quant_dataset)
        # after optimisation the layer uses hard rounding
        quant_module.use_soft_rounding = False

    @classmethod
    def _optimize_rounding(cls, module: torch.nn.Module, quant_module: AdaroundWrapper, orig_model: torch.nn.Module,
                           quant_model: torch.nn.Module, act_func: Union[torch.nn.Module, None], cached_dataset,
                           forward_fn: Callable[[torch.nn.Module, Any], Any], opt_params: AdaroundHyperParameters,
                           cached_quant_dataset=None):
        # pylint: disable=too-many-arguments, too-many-locals
        assert isinstance(quant_module, AdaroundWrapper), '%s is not adaround wrapper module.' % quant_module
        assert quant_module.use_soft_rounding, 'optimization should use soft rounding only.'
        assert quant_module.alpha is not None, 'alpha parameter should be initialized.'

        act_sampler = ActivationSampler(module, quant_module, orig_model, quant_model, forward_fn)
        all_inp_data, all_orig_out_data = act_sampler.sample_all_acts(cached_dataset, cached_quant_dataset)
        cls.optimize_rounding_on_cached_acts(quant_module, act_func, all_inp_data, all_orig_out_data, opt_params)

    @classmethod
    def optimize_rounding_on_cached_acts(cls, quant_module: AdaroundWrapper, act_func, all_inp_data: torch.Tensor,
                                         all_orig_out_data: torch.Tensor, opt_params: AdaroundHyperParameters,
                                         batches=None, first_iteration: int = 0):
        """The iteration loop over activations that are already resident on the GPU.

        `batches`: optional iterable of index tensors, one per iteration; by default opt_params.num_iterations batches
        of torch.randperm(N)[:BATCH_SIZE] drawn from torch's global host generator.
        Returns the Adam state (exp_avg, exp_avg_sq); alpha is updated in place and alpha.grad holds the last gradient.
        """
        # pylint: disable=too-many-arguments, too-many-locals
        qm = quant_module
        device = all_inp_data.device
        weight = qm.weight.detach().to(torch.float32).contiguous()
        alpha = qm.alpha.data
        exp_avg = torch.zeros_like(alpha)
        exp_avg_sq = torch.zeros_like(alpha)
        grad_alpha = torch.empty_like(alpha)
        if batches is None:
            n = all_inp_data.size(0)
            batches = [torch.randperm(n)[:BATCH_SIZE] for _ in range(opt_params.num_iterations)]
        else:
            batches = list(batches)
        if not batches:
            return exp_avg, exp_avg_sq

        def beta_of(iteration):
            if AdaroundLoss.in_warm_start(opt_params, iteration):
                return -1.0
            return AdaroundLoss._compute_beta(opt_params.num_iterations, iteration,  # pylint: disable=protected-access
                                              opt_params.beta_range, opt_params.warm_start)

        activation = cls._fused_activation_code(act_func)
        module = qm.get_original_module()
        rows = cls._fused_rows(module, weight, qm, all_inp_data, all_orig_out_data, batches) \
            if cls.use_fused_linear and activation is not None else None
        if rows is not None:
            # soft rounding fused into the MFMA GEMMs: three launches per iteration, nothing weight-shaped is
            # written except alpha and the Adam moments
            x_rows, y_rows, pixels = rows
            out_features, in_features = weight.shape[:2]
            as_matrix = lambda t: t.view(out_features, in_features)     # a 1x1 kernel is the same memory
            weight2, alpha2 = as_matrix(weight), as_matrix(alpha)
            # floor(W / delta) never changes during the optimisation: int8 where the grid allows it (up to 7 bits; a
            # quarter of the bytes), else int16, else float32 -- identical results in every form
            weight_floor = ops.adaround_floor_packed(weight2, qm.num_channel, qm.n_per_channel, qm.delta, qm.offset,
                                                     qm.clip_min, qm.clip_max) if cls.use_int8_floor else None
            if weight_floor is None:
                weight_floor = ops.adaround_floor(weight2, qm.num_channel, qm.n_per_channel, qm.delta)
            index = torch.stack(batches)
            # the kernels gather rows by these numbers; the reference's all_inp_data[indices] raises on a bad one
            num_samples = min(all_inp_data.size(0), all_orig_out_data.size(0))
            if index.numel() and (int(index.min()) < -num_samples or int(index.max()) >= num_samples):
                raise IndexError(f"batch index out of range for {num_samples} cached rows")
            index = torch.where(index < 0, index + num_samples, index)      # negative numbers count from the end
            if pixels > 1:
                # sample b owns rows b * pixels .. b * pixels + pixels - 1 of the channels-last copies
                index = (index.unsqueeze(-1) * pixels + torch.arange(pixels)).flatten(1)
            index = index.to(dtype=torch.int32, device=device).contiguous()
            batch_rows = index.size(1)
            bias = None if module.bias is None else module.bias.detach().to(torch.float32).contiguous()
            workspace = ops.adaround_linear_workspace(out_features, in_features, device, batch_rows)
            grad_out = torch.empty(batch_rows, out_features, dtype=torch.float32, device=device)
            moments = as_matrix(exp_avg), as_matrix(exp_avg_sq)
            for k in range(len(batches)):
                ops.adaround_linear_fwd(weight_floor, alpha2, x_rows, index[k], y_rows, bias,
                                        qm.num_channel, qm.delta, qm.offset, qm.clip_min, qm.clip_max, activation,
                                        workspace, grad_out)
                ops.adaround_linear_bwd_adam(weight_floor, grad_out, x_rows, index[k], alpha2, *moments,
                                             qm.num_channel, qm.delta, qm.offset, qm.clip_min, qm.clip_max,
                                             opt_params.reg_param, beta_of(first_iteration + k), ADAM_LR,
                                             ADAM_BETAS[0], ADAM_BETAS[1], ADAM_EPS, k + 1,
                                             grad_alpha=as_matrix(grad_alpha) if k == len(batches) - 1 else None)
            qm.alpha.grad = grad_alpha
            return exp_avg, exp_avg_sq

        # the batch indices of all iterations in one host-to-device copy (one copy per iteration waits for the device
        # every time); ragged batches (a caller's own) keep their own copies
        same_size = all(b.numel() == batches[0].numel() for b in batches)
        index_dev = torch.stack(batches).to(device) if same_size else None
        explicit = cls.use_explicit_gradient and activation is not None and cls._explicit_gradient_applies(module)
        for k, indices in enumerate(batches):
            indices = index_dev[k] if index_dev is not None else indices.to(device)
            inp_data = all_inp_data[indices]

            ada_weight = ops.adaround_soft_round(weight, alpha, qm.num_channel, qm.n_per_channel, qm.delta, qm.offset,
                                                 qm.clip_min, qm.clip_max, True)
            if explicit:
                grad_weight = cls._recon_loss_weight_gradient(module, inp_data, all_orig_out_data, indices, ada_weight,
                                                              activation)
            else:
                orig_out_data = all_orig_out_data[indices]
                ada_weight.requires_grad_(True)
                quant_out_data = cls._layer_output(module, inp_data, ada_weight)
                if act_func is not None:
                    orig_out_data = act_func(orig_out_data)
                    quant_out_data = act_func(quant_out_data)
                recon_loss = AdaroundLoss.compute_recon_loss(quant_out_data, orig_out_data)
                grad_weight, = torch.autograd.grad(recon_loss, ada_weight)
            ops.adaround_bwd_adam(weight, grad_weight.contiguous(), alpha, exp_avg, exp_avg_sq, qm.num_channel,
                                  qm.n_per_channel, qm.delta, qm.offset, qm.clip_min, qm.clip_max,
                                  opt_params.reg_param, beta_of(first_iteration + k), ADAM_LR, ADAM_BETAS[0],
                                  ADAM_BETAS[1], ADAM_EPS, k + 1,
                                  grad_alpha=grad_alpha if k == len(batches) - 1 else None)
        qm.alpha.grad = grad_alpha
        return exp_avg, exp_avg_sq

    # For Conv2d and Linear with no activation or ReLU the gradient of the reconstruction loss w.r.t. the soft-rounded
    # weight is written out -- dLoss/dout = 2 (act(out) - act(target)) act'(out) / (elements per channel), then the
    # layer's own weight-gradient routine -- instead of recorded and replayed by autograd: the same operations on the
    # same numbers (torch's backward of square / sum / mean / relu / convolution performs exactly these), without the
    # graph and the engine's hand-over, which at 32 samples per iteration cost more than the kernels.  False: autograd.
    # The reference can gather a layer's activations batch by batch inside the loop instead of once per layer, to save
    # host memory (:363-368); here they are always gathered once and stay on the GPU, whatever this says.
    is_activation_caching_enabled = True

    @staticmethod
    def enable_caching_acts_data() -> bool:
        return AdaroundOptimizer.is_activation_caching_enabled

    use_explicit_gradient = True
    # dLoss/dout of that written-out gradient by one kernel (False: the five tensor operations it stands for)
    use_fused_recon_gradient = True

    @staticmethod
    def _explicit_gradient_applies(module) -> bool:
        if isinstance(module, torch.nn.Linear):
            return True
        return isinstance(module, torch.nn.Conv2d) and isinstance(module.padding, tuple) and \
            module.padding_mode == 'zeros'

    @classmethod
    @torch.no_grad()
    def _recon_loss_weight_gradient(cls, module, inp_data, all_orig_out_data, indices, ada_weight, activation):
        out = cls._layer_output(module, inp_data, ada_weight)
        if cls.use_fused_recon_gradient and out.dtype == all_orig_out_data.dtype == torch.float32 and \
                all_orig_out_data.device == out.device and all_orig_out_data.is_contiguous() and \
                indices.dtype == torch.int64 and 0 < out.shape[0] <= 65535:
            # both activations, the difference, the loss's factor and relu's mask in one pass over the output; the
            # target rows are read where they lie in the cache
            grad_out = ops.adaround_recon_grad(out.contiguous(), all_orig_out_data, indices.contiguous(), activation)
        else:
            orig_out_data = all_orig_out_data[indices]
            if activation == 1:
                quant_act, orig_act = torch.relu(out), torch.relu(orig_out_data)
            else:
                quant_act, orig_act = out, orig_out_data
            # compute_recon_loss: squared error summed over dim 1, mean over the rest
            grad_out = (quant_act - orig_act) * (2.0 / (out.numel() // out.shape[1]))
            if activation == 1:
                grad_out = grad_out * (quant_act > 0)          # relu's backward: the gradient where its result is positive
        if isinstance(module, torch.nn.Linear):
            return grad_out.reshape(-1, grad_out.shape[-1]).t().mm(inp_data.reshape(-1, inp_data.shape[-1]))
        return torch.ops.aten.convolution_backward(
            grad_out, inp_data, ada_weight, None, list(module.stride), list(module.padding), list(module.dilation),
            False, [0, 0], module.groups, (False, True, False))[1]

    @staticmethod
    def _fused_activation_code(act_func):
        """0 / 1 for the activations the fused Linear kernels implement (none / ReLU), else None."""
        if act_func is None:
            return 0
        if isinstance(act_func, torch.nn.ReLU) or act_func in (torch.relu, functional.relu):
            return 1
        return None

    @staticmethod
    def _fused_rows(module, weight, qm, all_inp_data, all_orig_out_data, batches):
        """(x rows, target rows, rows per sample) when the MFMA-fused kernels take this layer, else None.

        They take a Linear layer on 2-D activations, and a Conv2d with a 1x1 kernel, unit stride, no padding and one
        group, which is the same contraction over the channels for every pixel (the reference calls functional.conv2d
        there, :268-272): its rows are the pixels, read from channels-last copies of the cached activations that are
        made once per layer.  The rows of an iteration -- batch entries times pixels -- must be 32, 64 or 128 (256, which
        the kernels also take, is faster through the general path: fused_rows_limit)."""
        if not batches or any(b.numel() != batches[0].numel() for b in batches):
            return None
        limit = AdaroundOptimizer.fused_rows_limit
        out_features, in_features = weight.shape[:2]
        per_channel_ok = qm.num_channel == 1 or (qm.num_channel == out_features and qm.n_per_channel == in_features)
        if not per_channel_ok or all_inp_data.dtype != torch.float32 or all_orig_out_data.dtype != torch.float32:
            return None
        if isinstance(module, torch.nn.Linear) and weight.dim() == 2:
            pixels = 1
            if all_inp_data.dim() != 2 or all_orig_out_data.dim() != 2:
                return None
            x_rows, y_rows = all_inp_data, all_orig_out_data
        elif isinstance(module, torch.nn.Conv2d) and weight.dim() == 4:
            one, zero = (1, 1), (0, 0)
            if tuple(weight.shape[2:]) != one or tuple(module.stride) != one or tuple(module.dilation) != one or \
                    module.groups != 1 or module.padding not in (zero, 0, 'valid') or \
                    all_inp_data.dim() != 4 or all_orig_out_data.dim() != 4 or \
                    all_inp_data.shape[2:] != all_orig_out_data.shape[2:]:
                return None
            pixels = all_inp_data.shape[2] * all_inp_data.shape[3]
            rows = batches[0].numel() * pixels
            if rows > limit or not ops.adaround_linear_supported(out_features, in_features, rows):
                return None             # before anything is copied
            x_rows = all_inp_data.permute(0, 2, 3, 1).reshape(-1, in_features).contiguous()
            y_rows = all_orig_out_data.permute(0, 2, 3, 1).reshape(-1, out_features).contiguous()
        else:
            return None
        if x_rows.size(1) != in_features or y_rows.size(1) != out_features:
            return None
        data_ok = all(t.stride(1) == 1 and t.stride(0) % 4 == 0 and t.data_ptr() % 16 == 0 for t in (x_rows, y_rows))
        rows = batches[0].numel() * pixels
        if data_ok and rows <= limit and ops.adaround_linear_supported(out_features, in_features, rows):
            return x_rows, y_rows, pixels
        return None

    @classmethod
    def _compute_recons_metrics(cls, quant_module: AdaroundWrapper, act_func, inp_data: torch.Tensor,
                                out_data: torch.Tensor) -> Tuple[float, float]:
        """MSE of the layer output under hard and under soft rounding: (recons_err_hard, recons_err_soft)."""
        with torch.no_grad():
            quant_module.use_soft_rounding = False
            out_data_hard = cls._compute_output_with_adarounded_weights(quant_module, inp_data)
            quant_module.use_soft_rounding = True
            out_data_soft = cls._compute_output_with_adarounded_weights(quant_module, inp_data)
            if act_func is not None:
                out_data = act_func(out_data)
                out_data_soft = act_func(out_data_soft)
                out_data_hard = act_func(out_data_hard)
            recons_err_soft = functional.mse_loss(out_data_soft, out_data)
            recons_err_hard = functional.mse_loss(out_data_hard, out_data)
        return float(recons_err_hard), float(recons_err_soft)

    @staticmethod
    def _layer_output(module: torch.nn.Module, inp_data: torch.Tensor, weight: torch.Tensor) -> torch.Tensor:
        if isinstance(module, torch.nn.Conv2d):
            return functional.conv2d(inp_data, weight, bias=module.bias, stride=module.stride,
                                     dilation=module.dilation, padding=module.padding, groups=module.groups)
        if isinstance(module, torch.nn.ConvTranspose2d):
            return functional.conv_transpose2d(inp_data, weight, bias=module.bias, stride=module.stride,
                                               padding=module.padding, output_padding=module.output_padding,
                                               groups=module.groups, dilation=module.dilation)
        if isinstance(module, torch.nn.Linear):
            return functional.linear(inp_data, weight, bias=module.bias)
        raise ValueError('AdaRound is not supported for the module: ', module)

    @classmethod
    def _compute_output_with_adarounded_weights(cls, quant_module: AdaroundWrapper, inp_data: torch.Tensor):
        """Output of the wrapped Conv2d / ConvTranspose2d / Linear computed with the adarounded weight."""
        module = quant_module.get_original_module()
        quant_module.to(inp_data.device)
        adarounded_weights = quant_module.apply_adaround(quant_module.weight)
        return cls._layer_output(module, inp_data, adarounded_weights)
