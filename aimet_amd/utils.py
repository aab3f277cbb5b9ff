"""Model-walking helpers the AdaRound flow needs (the counterparts of the few functions of
TrainingExtensions/torch/src/python/aimet_torch/utils.py that ADA/adaround_weight.py and ADA/activation_sampler.py
call: get_device, get_named_module, get_ordered_list_of_modules, CachedDataset, ModuleData, get_all_quantizers,
change_tensor_device_placement, in_eval_mode).  Graph questions are answered with forward hooks on one pass of the
model instead of the reference's traced ConnectedGraph.
"""
import contextlib
from typing import Any, Callable, Dict, List, Tuple, Union

import torch
from torch import nn


class StopForwardException(Exception):
    """Raised from a forward hook to abandon the rest of a forward pass."""


def get_device(model: nn.Module) -> torch.device:
    return next(model.parameters()).device


def get_named_module(model: nn.Module, name: str) -> nn.Module:
    module = model
    for part in name.split('.'):
        module = getattr(module, part)
    return module


def is_leaf_module(module: nn.Module) -> bool:
    return len(list(module.children())) == 0


def change_tensor_device_placement(data, device):
    """Moves a tensor, or a (nested) list / tuple of tensors, to `device`."""
    if isinstance(data, torch.Tensor):
        return data.to(device)
    if isinstance(data, (list, tuple)):
        return type(data)(change_tensor_device_placement(t, device) for t in data)
    return data


@contextlib.contextmanager
def in_eval_mode(model: nn.Module):
    was_training = model.training
    model.eval()
    try:
        yield
    finally:
        model.train(was_training)


def _default_forward(model, inputs):
    if isinstance(inputs, (list, tuple)):
        return model(*inputs)
    return model(inputs)


def get_ordered_list_of_modules(model: nn.Module, dummy_input: Union[torch.Tensor, Tuple],
                                fwd_func: Callable = None) -> List[List]:
    """[name, module] of every leaf module, in the order the forward pass reaches it."""
    fwd_func = fwd_func or _default_forward
    names = {m: n for n, m in model.named_modules()}
    order, handles = [], []

    def hook(module, _inputs, _output):
        order.append([names[module], module])

    for module in model.modules():
        if is_leaf_module(module) and module is not model:
            handles.append(module.register_forward_hook(hook))
    try:
        with in_eval_mode(model), torch.no_grad():
            fwd_func(model, dummy_input)
    finally:
        for h in handles:
            h.remove()
    return order


ACTIVATION_TYPES = (nn.ReLU, nn.ReLU6, nn.PReLU, nn.Sigmoid, nn.Tanh, nn.Hardtanh, nn.Hardswish, nn.SiLU, nn.GELU,
                    nn.LeakyReLU, nn.ELU, nn.Softplus, nn.Hardsigmoid)


def get_module_act_func_pair(model: nn.Module, dummy_input: Union[torch.Tensor, Tuple]) -> Dict[nn.Module, Any]:
    """Maps every leaf module to the activation module that directly consumes its output, or None.

    A module is paired when its output tensor has exactly one consumer among the leaf modules and that consumer is an
    activation (the relation the reference reads off its connected graph, connectedgraph_utils.get_module_act_func_pair).
    """
    producer: Dict[int, nn.Module] = {}
    edges: Dict[nn.Module, List[nn.Module]] = {}
    keep_alive, handles = [], []

    def hook(module, inputs, output):
        ins = [t for t in inputs if isinstance(t, torch.Tensor)]
        outs = [t for t in (output if isinstance(output, (tuple, list)) else (output,)) if isinstance(t, torch.Tensor)]
        keep_alive.extend(ins + outs)            # ids stay unique while the pass runs
        for t in ins:
            # resolved now, not afterwards: an in-place activation returns the tensor it was given
            if id(t) in producer:
                edges.setdefault(producer[id(t)], []).append(module)
        for t in outs:
            producer[id(t)] = module

    leaves = [m for m in model.modules() if is_leaf_module(m) and m is not model]
    for module in leaves:
        handles.append(module.register_forward_hook(hook))
    try:
        with in_eval_mode(model), torch.no_grad():
            _default_forward(model, dummy_input)
    finally:
        for h in handles:
            h.remove()
    pairs = {m: None for m in leaves}
    for module, users in edges.items():
        if len(users) == 1 and isinstance(users[0], ACTIVATION_TYPES):
            pairs[module] = users[0]
    return pairs


class CachedDataset:
    """The first `num_batches` batches of a data loader, held in memory.

    The reference (aimet_torch/utils.py, class CachedDataset) pickles every batch to a temporary directory and reads it
    back on each access; batches here stay where the loader put them (host memory, or the GPU's 288 GB when the loader
    yields device tensors).  `path` is accepted and ignored.
    """

    def __init__(self, data_loader, num_batches: int, path: str = None):
        if data_loader is not None and len(data_loader) < num_batches:
            raise ValueError(f'Can not fetch {num_batches} batches from a data loader of length {len(data_loader)}.')
        self._batches = []
        if data_loader is not None:
            for i, batch in enumerate(data_loader):
                if i >= num_batches:
                    break
                self._batches.append(batch)
        self._path = path

    def __len__(self):
        return len(self._batches)

    def __getitem__(self, index: int):
        return self._batches[index]

    def __iter__(self):
        return iter(self._batches)


class ModuleData:
    """Collects the input to / output of one module of a model during a forward pass that stops at that module."""

    def __init__(self, model: nn.Module, module: nn.Module, forward_fn: Callable = None):
        self._model = model
        self._module = module
        self._forward_fn = forward_fn or _default_forward

    def collect_inp_out_data(self, model_input, collect_input: bool, collect_output: bool):
        inp_data, out_data = [], []

        def hook(_module, inputs, output):
            if collect_input:
                inp_data.append(inputs[0] if isinstance(inputs, tuple) and len(inputs) == 1 else inputs)
            if collect_output:
                out_data.append(output)
            raise StopForwardException

        handle = self._module.register_forward_hook(hook)
        device = get_device(self._model)
        model_input = change_tensor_device_placement(model_input, device)
        try:
            with in_eval_mode(self._model), torch.no_grad():
                self._forward_fn(self._model, model_input)
        except StopForwardException:
            pass
        finally:
            handle.remove()
        return (inp_data[0] if inp_data else None), (out_data[0] if out_data else None)


def get_all_quantizers(model: nn.Module):
    """(param_quantizers, input_quantizers, output_quantizers) of every quantization wrapper in the model."""
    from .v1.qc_quantize_op import QcQuantizeWrapper   # pylint: disable=import-outside-toplevel
    param_quantizers, input_quantizers, output_quantizers = [], [], []
    for module in model.modules():
        if isinstance(module, QcQuantizeWrapper):
            param_quantizers.extend(module.param_quantizers.values())
            input_quantizers.extend(module.input_quantizers)
            output_quantizers.extend(module.output_quantizers)
    return param_quantizers, input_quantizers, output_quantizers
