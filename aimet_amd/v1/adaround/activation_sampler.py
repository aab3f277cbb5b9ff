"""Collects, for one layer, the input the weight-quantized model feeds it and the output the original model produces.

Mirrors ActivationSampler of TrainingExtensions/torch/src/python/aimet_torch/v1/adaround/activation_sampler.py
(:175-264).  Activations are gathered into tensors on the model's device and stay there: one GPU's memory holds the
reference's whole default sample (2000 images) for any layer, so there is no CPU staging and no per-iteration
host-to-device copy.
"""
from typing import Any, Callable, Dict, List, Tuple, Union

import torch

from ... import utils


# ------------------------------------------------------------------------------------------ checkpointed models
# A model given as blocks (groups of consecutive modules, or named sub-modules) needs, for the layers of one block,
# forward passes through that block only: the inputs of the block are kept for the original and for the
# weight-quantized model, and each finished block's outputs become the next block's inputs.  Mirrors
# create_modulelist_for_group_modules / get_block_inputs / get_block_outputs / create_cached_block_schedule_list of the
# reference's activation_sampler.py (:52-172, :259-300).  The reference moves the models to the host and one block at a
# time to the device, and keeps the block inputs on the host or on disk; here models stay where they are and block
# inputs live on the device unless the checkpoints file asks for host memory (`cache_on_cpu`).

def create_modulelist_for_group_modules(model: torch.nn.Module, sim, grouped_modules: Dict[str, List[str]]) \
        -> Tuple[List[torch.nn.ModuleList], List[torch.nn.ModuleList]]:
    """One ModuleList per group, of the original model's modules and of the simulation model's, in the file's order."""
    fp_blocks, sim_blocks = [], []
    for names in grouped_modules.values():
        fp_blocks.append(torch.nn.ModuleList(utils.get_named_module(model, name) for name in names))
        sim_blocks.append(torch.nn.ModuleList(utils.get_named_module(sim.model, name) for name in names))
    return fp_blocks, sim_blocks


def get_block_inputs(model: torch.nn.Module, sim, breakpoint_module_name: str, cached_dataset, cache_on_cpu: bool,
                     forward_fn: Callable, num_batches: int, working_dir: str, incl_kwargs: bool = False) \
        -> Tuple[List, List]:
    """What the named module receives in the original model and in the simulation model, per batch."""
    # pylint: disable=too-many-arguments
    del num_batches, working_dir                         # every batch of `cached_dataset` is used; nothing goes to disk
    fp_inputs = utils.cache_intermediate_datasets(cached_dataset, cache_on_cpu, model, breakpoint_module_name,
                                                  forward_fn, incl_kwargs=incl_kwargs)
    quant_inputs = utils.cache_intermediate_datasets(cached_dataset, cache_on_cpu, sim.model, breakpoint_module_name,
                                                     forward_fn, incl_kwargs=incl_kwargs)
    return fp_inputs, quant_inputs


def get_block_outputs(fp_block: torch.nn.ModuleList, quant_block: torch.nn.ModuleList, include_static_inputs,
                      cached_fp_dataset: List, cached_quant_dataset: List, cache_on_cpu: bool, forward_fn: Callable,
                      device: torch.device, working_dir: str = None):
    """Runs every cached input through its block and stores the (first) output in its place, as the next block's
    input.  With `include_static_inputs` only the first input is replaced: the others (an attention mask, position
    ids) are the same for every block and stay."""
    # pylint: disable=too-many-arguments
    del working_dir
    keep_static = include_static_inputs in (True, "True")
    keep_on = torch.device('cpu') if cache_on_cpu else device

    def first_output(block, inputs):
        out = forward_fn(block, inputs)
        out = out[0] if isinstance(out, (tuple, list)) else out
        return utils.change_tensor_device_placement(out, keep_on)

    for index, (fp_inputs, quant_inputs) in enumerate(zip(cached_fp_dataset, cached_quant_dataset)):
        fp_inputs = utils.change_tensor_device_placement(fp_inputs, device)
        quant_inputs = utils.change_tensor_device_placement(quant_inputs, device)
        with utils.in_eval_mode(fp_block), utils.in_eval_mode(quant_block), torch.no_grad():
            fp_out, quant_out = first_output(fp_block, fp_inputs), first_output(quant_block, quant_inputs)
        if keep_static:
            cached_fp_dataset[index] = [fp_out, *utils.change_tensor_device_placement(list(fp_inputs[1:]), keep_on)]
            cached_quant_dataset[index] = [quant_out,
                                           *utils.change_tensor_device_placement(list(quant_inputs[1:]), keep_on)]
        else:
            cached_fp_dataset[index], cached_quant_dataset[index] = [fp_out], [quant_out]


def create_cached_block_schedule_list(model: torch.nn.Module, dummy_input, block_names: List[str],
                                      supported_modules: Tuple) -> List[Tuple[Any, List[List]]]:
    """The supported modules of `model` in forward order, cut into runs that belong to the same named block (or to
    none): [(None | (block name, block module), [[name, module], ...]), ...].  Inside a block, names are relative to
    the block."""
    block_of, name_of = {}, {}
    for name, module in utils.get_ordered_list_of_modules(model, dummy_input):
        if isinstance(module, supported_modules):
            block_of[module], name_of[module] = None, name
    for block_name in block_names:
        block = utils.get_named_module(model, block_name)
        for module in block.modules():
            if module in block_of:
                block_of[module] = (block_name, block)
                name_of[module] = name_of[module][len(block_name) + 1:]
    schedule = []
    for module, block in block_of.items():                # dicts keep insertion order: forward order
        if not schedule or schedule[-1][0] != block:
            schedule.append((block, []))
        schedule[-1][1].append([name_of[module], module])
    return schedule


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
