"""Sequential MSE: layer by layer, in forward order, pick for each output channel of a Linear / Conv2d weight the
clipping range -- among `num_candidates` equal fractions of the channel's own range -- whose quantized weight
reproduces the layer's output best, and freeze the weight quantizer there.

Same entry points, parameters and hooks as TrainingExtensions/torch/src/python/aimet_torch/v1/seq_mse.py (SeqMseParams
:84-99, SequentialMse.apply_seq_mse :106-167, apply_seq_mse_using_opt_sampling :169-241, run_seq_mse :243-293,
get_module_inp_acts :295-331, temporarily_disable_quantizers :333-394, compute_all_param_encodings :396-411,
get_per_channel_min_and_max :413-439, get_candidates :441-464, optimize_module :466-503, compute_param_encodings
:505-519, compute_outputs :521-555, compute_recon_loss :557-581, neg_sqnr :602-615).

What runs where: every candidate's encodings come from the TF analyzer kernels on the [channels, 2] tensor of its
(min, max) pairs, its quantized weight from the per-channel / per-tensor quantize-dequantize kernel, the two layer
outputs from the GEMM / convolution library; activations sampled for a layer stay on the device.  The float output of a
batch does not depend on the candidate and is computed once per batch instead of once per candidate and batch -- the
same operation on the same operands, so every loss is the reference's.
"""
import contextlib
import json
from dataclasses import dataclass
from typing import Callable, List, Optional, Tuple

import torch
import torch.nn.functional as functional

from .. import ops
from ..common import libpymo
from ..common.defs import QuantScheme
from ..utils import (CachedDataset, StopForwardException, change_tensor_device_placement, get_device,
                     get_ordered_list_of_modules, in_eval_mode)
from .adaround.activation_sampler import create_modulelist_for_group_modules, get_block_inputs, get_block_outputs
from .qc_quantize_op import QcQuantizeOpMode, QcQuantizeWrapper
from .quantsim import QuantizationSimModel

# module types whose weight encodings are searched
SUPPORTED_MODULES = (torch.nn.Linear, torch.nn.Conv2d)

# weights quantized to more bits than this are left alone: the search pays off on coarse grids
SUPPORTED_PARAM_BW = 4


def default_forward_fn(model, inputs):
    """model(*inputs); a lone tensor is one input."""
    if isinstance(inputs, torch.Tensor):
        inputs = [inputs]
    return model(*inputs)


@dataclass
class SeqMseParams:
    """num_batches: batches of the data loader to use.  num_candidates: fractions of a channel's range to try.
    inp_symmetry: which inputs feed the two layer outputs that are compared -- 'asym': float inputs into the float
    weight against quantized-model inputs into the quantized weight; 'symfp': float inputs into both; 'symqt':
    quantized-model inputs into both.  loss_fn: 'mse', 'l1' or 'sqnr'.  forward_fn(model, batch): runs the model on
    what the data loader yields."""
    num_batches: int
    num_candidates: int = 20
    inp_symmetry: str = 'symqt'
    loss_fn: str = 'mse'
    forward_fn: Callable = default_forward_fn


class SequentialMse:
    """Weight encodings by minimizing each layer's output error, one layer after the other."""

    # ---------------------------------------------------------------------------------------------- entry points
    @classmethod
    def apply_seq_mse(cls, model: torch.nn.Module, sim: QuantizationSimModel, data_loader, params: SeqMseParams,
                      modules_to_exclude: Optional[List[torch.nn.Module]] = None,
                      checkpoints_config: Optional[str] = None):
        """Finds and freezes the weight encodings of the supported modules of `sim` (built from `model`); everything
        else about `sim` is as before afterwards, so that `sim.compute_encodings` can follow for the activations and
        the remaining parameters.  `modules_to_exclude` names modules of `model`."""
        # pylint: disable=too-many-arguments, protected-access
        assert sim._quant_scheme in (QuantScheme.post_training_tf, QuantScheme.training_range_learning_with_tf_init), \
            "Use TF quant-scheme with sequential MSE."
        # while the search runs only the weights of supported modules are quantized
        with cls.temporarily_disable_quantizers(model, sim, modules_to_exclude):
            cls.compute_all_param_encodings(sim)
            batches = CachedDataset(data_loader, params.num_batches)
            if checkpoints_config:
                cls.apply_seq_mse_using_opt_sampling(checkpoints_config, model, sim, modules_to_exclude, batches, params,
                                                     None)
                return
            dummy_input = change_tensor_device_placement(next(iter(data_loader)), get_device(model))
            layers = cls._searched_layers(get_ordered_list_of_modules(model, dummy_input, fwd_func=params.forward_fn),
                                          modules_to_exclude)
            cls.run_seq_mse(layers, model, sim.model, params, params.forward_fn, batches, cached_quant_dataset=None)

    @classmethod
    def apply_seq_mse_using_opt_sampling(cls, checkpoints_config: str, model: torch.nn.Module,
                                         sim: QuantizationSimModel, modules_to_exclude, cached_dataset,
                                         params: SeqMseParams, tempdir: str):
        """The model as consecutive groups of modules (the sequential layout of an AdaRound checkpoints file): a
        layer's inputs are sampled by passes through its own group, fed from the kept outputs of the group before.
        Nothing may happen between two groups outside their modules."""
        # pylint: disable=too-many-arguments, too-many-locals
        with open(checkpoints_config, encoding='utf-8') as file:
            checkpoints = json.load(file)
        for key, what in (('grouped_modules', "a dictionary of grouped_modules in the file to define checkpoints"),
                          ('include_static_inputs', "a dictionary of include_static_inputs in the file to define "
                                                    "checkpoints"),
                          ('cache_on_cpu', "cache_on_cpu to determine whether to cache intermediate tensors on CPU")):
            assert key in checkpoints, f"Please provide {what}"
        groups = checkpoints['grouped_modules']
        cache_on_cpu = checkpoints['cache_on_cpu'] in (True, "True", "true")
        fp_inputs, quant_inputs = get_block_inputs(model, sim, next(iter(groups.values()))[0], cached_dataset,
                                                   cache_on_cpu, params.forward_fn, params.num_batches, tempdir)
        device = get_device(model)

        def through_the_group(group, x):
            for module in group:
                x = module(*x) if isinstance(x, (tuple, list)) else module(x)
            return x

        fp_groups, sim_groups = create_modulelist_for_group_modules(model, sim, groups)
        for index, (fp_group, sim_group, static) in enumerate(zip(fp_groups, sim_groups,
                                                                  checkpoints['include_static_inputs'])):
            first_inputs = change_tensor_device_placement(fp_inputs[0], device)
            layers = cls._searched_layers(get_ordered_list_of_modules(fp_group, first_inputs,
                                                                      fwd_func=through_the_group), modules_to_exclude)
            cls.run_seq_mse(layers, fp_group, sim_group, params, through_the_group, fp_inputs,
                            cached_quant_dataset=quant_inputs)
            if index < len(fp_groups) - 1:
                get_block_outputs(fp_group, sim_group, static, fp_inputs, quant_inputs, cache_on_cpu, through_the_group,
                                  device, tempdir)

    @staticmethod
    def _searched_layers(in_forward_order, modules_to_exclude) -> List[Tuple[str, torch.nn.Module]]:
        excluded = modules_to_exclude or []
        return [(name, module) for name, module in in_forward_order
                if isinstance(module, SUPPORTED_MODULES) and not any(module is other for other in excluded)]

    @classmethod
    def run_seq_mse(cls, fp32_modules: List[Tuple[str, torch.nn.Module]], model: torch.nn.Module,
                    quant_model: torch.nn.Module, params: SeqMseParams, forward_fn: Callable, cached_fp_dataset,
                    cached_quant_dataset=None):
        """The layers of `fp32_modules` in order; the quantized model's inputs to a layer already carry the frozen
        encodings of the layers before it."""
        # pylint: disable=too-many-arguments
        quantized = dict(quant_model.named_modules())
        if not cached_quant_dataset:
            cached_quant_dataset = cached_fp_dataset
        for name, fp32_module in fp32_modules:
            quant_module = quantized.get(name)
            if quant_module is None or cls._weight_bitwidth(quant_module) > SUPPORTED_PARAM_BW:
                continue
            from_float = lambda: cls.get_module_inp_acts(fp32_module, model, params, forward_fn, cached_fp_dataset)
            from_quantized = lambda: cls.get_module_inp_acts(quant_module, quant_model, params, forward_fn,
                                                             cached_quant_dataset)       # pylint: disable=cell-var-from-loop
            if params.inp_symmetry == "asym":
                cls.optimize_module(quant_module, from_float(), from_quantized(), params)
            elif params.inp_symmetry == "symfp":
                acts = from_float()
                cls.optimize_module(quant_module, acts, acts, params)
            elif params.inp_symmetry == "symqt":
                acts = from_quantized()
                cls.optimize_module(quant_module, acts, acts, params)
            else:
                raise ValueError(f"Invalid inp_symmetry: {params.inp_symmetry}")

    @staticmethod
    def _weight_bitwidth(quant_module) -> int:
        return quant_module.param_quantizers['weight'].bitwidth

    @staticmethod
    def get_module_inp_acts(module: torch.nn.Module, model: torch.nn.Module, params: SeqMseParams,
                            forward_fn: Callable, cached_dataset) -> torch.Tensor:
        """The first input of `module` for each of the first `num_batches` batches, stacked: [num_batches, ...].  Each
        pass stops at the module."""
        seen = []

        def keep_and_stop(_module, inputs, _output):
            if isinstance(inputs, tuple):
                seen.append(inputs[0])
            raise StopForwardException

        handle = module.register_forward_hook(keep_and_stop)
        device = get_device(model)
        try:
            batches = iter(cached_dataset)
            for _ in range(params.num_batches):
                batch = change_tensor_device_placement(next(batches), device)
                try:
                    with in_eval_mode(model), torch.no_grad():
                        forward_fn(model, batch)
                except StopForwardException:
                    pass
        finally:
            handle.remove()
        return torch.stack(seen)

    # --------------------------------------------------------------------------- what is quantized during the search
    @staticmethod
    def _get_quantizers_to_be_disabled(model: torch.nn.Module, sim: QuantizationSimModel, modules_to_exclude) -> List:
        """The enabled quantizers that must be off while the search runs: every activation quantizer, the parameter
        quantizers of unsupported module types, and those of the excluded modules."""
        # pylint: disable=protected-access
        float_modules = dict(model.named_modules())
        excluded = modules_to_exclude or []
        off = []
        for name, wrapper in sim.quant_wrappers():
            off += [q for q in (*wrapper.input_quantizers, *wrapper.output_quantizers) if q.enabled]
            searched = isinstance(wrapper._module_to_wrap, SUPPORTED_MODULES) and \
                not any(float_modules.get(name) is other for other in excluded)
            if not searched:
                off += [q for q in wrapper.param_quantizers.values() if q.enabled]
        return off

    @classmethod
    @contextlib.contextmanager
    def temporarily_disable_quantizers(cls, model: torch.nn.Module, sim: QuantizationSimModel, modules_to_exclude):
        """Inside the `with` only the weights (and biases, if configured) of searched modules are quantized."""
        off = cls._get_quantizers_to_be_disabled(model, sim, modules_to_exclude)
        for quantizer in off:
            quantizer.enabled = False
        try:
            yield
        finally:
            for quantizer in off:
                quantizer.enabled = True

    @staticmethod
    def compute_all_param_encodings(sim: QuantizationSimModel):
        """Every parameter quantizer's encoding from its parameter; wrappers go to ACTIVE mode, in which they
        quantize their parameters."""
        for _, wrapper in sim.quant_wrappers():
            for name, quantizer in wrapper.param_quantizers.items():
                quantizer.reset_encoding_stats()
                quantizer.update_encoding_stats(getattr(wrapper, name).data)
                quantizer.compute_encoding()
            wrapper.set_mode(QcQuantizeOpMode.ACTIVE)

    # ------------------------------------------------------------------------------------------------ one layer
    @classmethod
    def get_per_channel_min_and_max(cls, quant_module) -> Tuple[Optional[torch.Tensor], torch.Tensor]:
        """Per output channel: (min, max) of the weight, or (None, max |weight|) under a symmetric quantizer."""
        module = cls._get_original_module(quant_module)
        if isinstance(module, torch.nn.Conv2d):
            rows = module.weight.reshape(module.out_channels, -1)
        elif isinstance(module, torch.nn.Linear):
            rows = module.weight
        else:
            raise ValueError('Unsupported module: ', module)
        rows = rows.detach()
        if cls._is_symmetric_quantizer(quant_module.param_quantizers["weight"]):
            return None, rows.abs().max(dim=1)[0]
        return rows.min(dim=1)[0], rows.max(dim=1)[0]

    @staticmethod
    def get_candidates(num_candidates: int, per_channel_max: torch.Tensor,
                       per_channel_min: Optional[torch.Tensor]) -> List[Tuple[torch.Tensor, torch.Tensor]]:
        """(max, min) per channel for fractions 1/n, 2/n, ... n/n of the range; min = -max when no min is given."""
        candidates = []
        for step in range(1, num_candidates + 1):
            cand_max = (per_channel_max / num_candidates * step).clone().detach()
            cand_min = -cand_max if per_channel_min is None else \
                (per_channel_min / num_candidates * step).clone().detach()
            candidates.append((cand_max, cand_min))
        return candidates

    @classmethod
    def optimize_module(cls, quant_module, x: torch.Tensor, xq: torch.Tensor, params: SeqMseParams):
        """Tries every candidate on all batches (x, xq: [num_batches, ...] inputs for the float and for the quantized
        weight), keeps per channel the candidate of least summed loss, and freezes the weight quantizer on it."""
        # pylint: disable=too-many-locals
        per_channel_min, per_channel_max = cls.get_per_channel_min_and_max(quant_module)
        candidates = cls.get_candidates(params.num_candidates, per_channel_max, per_channel_min)
        quantizer = quant_module.param_quantizers['weight']
        module = cls._get_original_module(quant_module)
        w = quant_module.weight
        with torch.no_grad():
            float_outputs = [cls._layer_output(module, x[b], w) for b in range(params.num_batches)]
            total_loss = []
            for cand_max, cand_min in candidates:
                cls.compute_param_encodings(quantizer, cand_min, cand_max)
                wq = cls._get_quantized_weight(quant_module)
                loss = torch.zeros(len(cand_max), device=w.device)
                for b in range(params.num_batches):
                    loss += cls.compute_recon_loss(cls._layer_output(module, xq[b], wq), float_outputs[b], params)
                total_loss.append(loss)
        best = torch.stack(total_loss).min(0, keepdim=True)[1]
        best_max = torch.stack([cand_max for cand_max, _ in candidates]).gather(0, best)[0]
        best_min = torch.stack([cand_min for _, cand_min in candidates]).gather(0, best)[0]
        cls.compute_param_encodings(quantizer, best_min, best_max)
        cls._freeze_quantizer_encoding(quantizer)

    @staticmethod
    def compute_param_encodings(quantizer, x_min: torch.Tensor, x_max: torch.Tensor):
        """The quantizer's encodings as if it had observed a tensor whose channel c spans [x_min[c], x_max[c]]."""
        quantizer.reset_encoding_stats()
        quantizer.update_encoding_stats(torch.stack([x_min, x_max], dim=-1))
        quantizer.compute_encoding()

    @staticmethod
    def _layer_output(module: torch.nn.Module, inputs: torch.Tensor, weight: torch.Tensor) -> torch.Tensor:
        """The layer's product without its bias, channels last."""
        if isinstance(module, torch.nn.Linear):
            return functional.linear(inputs, weight)
        if isinstance(module, torch.nn.Conv2d):
            out = functional.conv2d(inputs, weight, stride=module.stride, dilation=module.dilation,
                                    padding=module.padding, groups=module.groups)
            return out.permute(0, 2, 3, 1)                          # [N, C, H, W] -> [N, H, W, C]
        raise ValueError('Unsupported module: ', module)

    @classmethod
    def compute_outputs(cls, quant_module, x: torch.Tensor, xq: torch.Tensor, w: torch.Tensor,
                        wq: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
        """(xq * wq, x * w) through the layer's operation, channels last."""
        # pylint: disable=too-many-arguments
        module = cls._get_original_module(quant_module)
        return cls._layer_output(module, xq, wq), cls._layer_output(module, x, w)

    @staticmethod
    def compute_recon_loss(xqwq: torch.Tensor, xw: torch.Tensor, params: SeqMseParams) -> torch.Tensor:
        """Per output channel: the loss summed over everything else."""
        try:
            loss_fn = {"mse": functional.mse_loss, "l1": functional.l1_loss, "sqnr": neg_sqnr}[params.loss_fn]
        except KeyError:
            raise ValueError(f"Invalid loss function: {params.loss_fn}") from None
        channels = xqwq.shape[-1]
        xqwq, xw = xqwq.reshape(-1, channels), xw.reshape(-1, channels)
        if xqwq.is_cuda and xqwq.dtype == xw.dtype == torch.float32 and xqwq.is_contiguous() and xw.is_contiguous():
            # one pass over the two outputs instead of a difference, a square and a sum
            rows = xqwq.shape[0]
            if params.loss_fn == "sqnr":
                noise, signal = ops.column_error(xqwq[None], xw[None], ops.COLUMN_ERROR_SQUARED_AND_SIGNAL)
                return (-10 * torch.log10((signal / rows) / (noise / rows + 1e-10)))[0]
            kind = ops.COLUMN_ERROR_SQUARED if params.loss_fn == "mse" else ops.COLUMN_ERROR_ABSOLUTE
            return ops.column_error(xqwq[None], xw[None], kind)[0]
        loss = loss_fn(xqwq, xw, reduction="none").sum(0)
        assert loss.size() == torch.Size([channels])
        return loss

    # ------------------------------------------------------------------- what differs between the v1 and v2 models
    @staticmethod
    def _is_symmetric_quantizer(quantizer) -> bool:
        return quantizer.use_symmetric_encodings

    @staticmethod
    def _freeze_quantizer_encoding(quantizer):
        return quantizer.freeze_encoding()

    @staticmethod
    def _get_quantized_weight(quant_module: QcQuantizeWrapper) -> torch.Tensor:
        return quant_module.param_quantizers['weight'].quantize_dequantize(quant_module.weight,
                                                                           libpymo.RoundingMode.ROUND_NEAREST)

    @staticmethod
    def _get_original_module(quant_module: QcQuantizeWrapper) -> torch.nn.Module:
        return quant_module._module_to_wrap                         # pylint: disable=protected-access


def neg_sqnr(pred: torch.Tensor, target: torch.Tensor, eps=1e-10, reduction="none"):
    """Minus the signal-to-quantization-noise ratio in dB per column (one row of output: the sum over rows that the
    caller takes leaves it as it is)."""
    # pylint: disable=unused-argument
    noise = torch.mean((target - pred) ** 2, 0, keepdim=True) + eps
    signal = torch.mean(target ** 2, 0, keepdim=True)
    return -10 * torch.log10(signal / noise)


# module-level names, as the reference offers them
apply_seq_mse = SequentialMse.apply_seq_mse
get_candidates = SequentialMse.get_candidates
optimize_module = SequentialMse.optimize_module
