"""Collects, for one layer, the input the weight-quantized model feeds it and the output the original model produces.

Mirrors ActivationSampler of TrainingExtensions/torch/src/python/aimet_torch/v1/adaround/activation_sampler.py
(:175-264).  Activations are gathered into tensors on the model's device and stay there: one GPU's memory holds the
reference's whole default sample (2000 images) for any layer, so there is no CPU staging and no per-iteration
host-to-device copy.
"""
from typing import Any, Callable, List, Tuple, Union

import torch

from ... import utils


class ActivationSampler:
    """Input of `quant_module` in `quant_model` and output of `orig_module` in `orig_model` for the same model input."""

    def __init__(self, orig_module: torch.nn.Module, quant_module: torch.nn.Module, orig_model: torch.nn.Module,
                 quant_model: torch.nn.Module, forward_fn: Callable[[torch.nn.Module, Any], Any]):
        self._orig_module_collector = utils.ModuleData(orig_model, orig_module, forward_fn)
        self._quant_module_collector = utils.ModuleData(quant_model, quant_module, forward_fn)

    def sample_acts(self, model_inputs: Union[torch.Tensor, List, Tuple], collect_input=True, collect_output=True) \
            -> Tuple[torch.Tensor, torch.Tensor]:
        inp_data, out_data = None, None
        if collect_input:
            inp_data, _ = self._quant_module_collector.collect_inp_out_data(model_inputs, collect_input=True,
                                                                            collect_output=False)
        if collect_output:
            _, out_data = self._orig_module_collector.collect_inp_out_data(model_inputs, collect_input=False,
                                                                           collect_output=True)
        return inp_data, out_data

    def sample_all_acts(self, cached_dataset, cached_quant_dataset=None) -> Tuple[torch.Tensor, torch.Tensor]:
        """All batches of the cached dataset, concatenated along dim 0 on the model's device."""
        all_inp_data, all_out_data = [], []
        if cached_quant_dataset is not None:
            assert len(cached_dataset) == len(cached_quant_dataset)
        for batch_index in range(len(cached_dataset)):
            if cached_quant_dataset is not None:
                inp_data, _ = self.sample_acts(cached_quant_dataset[batch_index], collect_input=True,
                                               collect_output=False)
                _, out_data = self.sample_acts(cached_dataset[batch_index], collect_input=False, collect_output=True)
            else:
                inp_data, out_data = self.sample_acts(cached_dataset[batch_index])
            all_inp_data.append(inp_data.detach().clone())
            all_out_data.append(out_data.detach().clone())
        return torch.cat(all_inp_data, dim=0), torch.cat(all_out_data, dim=0)

    # name kept for callers of the reference's API; nothing is moved to the CPU here
    sample_and_place_all_acts_on_cpu = sample_all_acts
