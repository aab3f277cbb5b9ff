"""Model-walking helpers the AdaRound flow needs (the counterparts of the few functions of
TrainingExtensions/torch/src/python/aimet_torch/utils.py that ADA/adaround_weight.py and ADA/activation_sampler.py
call: get_device, get_named_module, get_ordered_list_of_modules, CachedDataset, ModuleData, get_all_quantizers,
change_tensor_device_placement, in_eval_mode), and the helpers of the encodings file format
(create_encoding_dict / create_encoding_from_dict, partial encodings, per-tensor <-> per-channel quantizer swaps).
Graph questions are answered with forward hooks on one pass of the model instead of the reference's traced
ConnectedGraph.
"""
import contextlib
import inspect
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


def add_foward_fn_kwargs_to_inputs(module: nn.Module, *args, **kwargs) -> Tuple:
    """A call `module(*args, **kwargs)` as positional arguments only: the parameters of `module.forward` that `args`
    does not reach take their keyword value, or else their default (reference aimet_torch/utils.py:1041-1061; the
    misspelt name is the reference's)."""
    parameters = [p for p in inspect.signature(module.forward).parameters.values()
                  if p.name != 'self' and p.kind in (p.POSITIONAL_ONLY, p.POSITIONAL_OR_KEYWORD, p.KEYWORD_ONLY)]
    extra = []
    for parameter in parameters[len(args):]:
        if parameter.name in kwargs:
            extra.append(kwargs[parameter.name])
        elif parameter.default is not inspect.Parameter.empty:
            extra.append(parameter.default)
    return (*args, *extra)


def cache_intermediate_datasets(cached_dataset, cache_on_cpu: bool, model: nn.Module, module_name: str,
                                forward_fn: Callable, path: str = None, incl_kwargs: bool = False) -> List[List]:
    """What the module called `module_name` receives for every batch of `cached_dataset`: one list of its positional
    inputs per batch (its keyword inputs laid behind them when `incl_kwargs`).  Each forward pass stops at that module.

    The reference (aimet_torch/utils.py:1064-1105) keeps these lists in host memory when `cache_on_cpu`, and otherwise
    pickles each to `path` and reads it back on every access.  Here `cache_on_cpu` decides between host memory and the
    device the model runs on -- one GPU's 288 GB hold the block inputs of models that do not fit a host's page cache --
    and `path` is accepted and ignored."""
    # pylint: disable=too-many-arguments
    del path
    module = get_named_module(model, module_name)
    forward_fn = forward_fn or _default_forward
    cached = []

    def keep_inputs_and_stop(_module, args, kwargs):
        if incl_kwargs and kwargs:
            args = add_foward_fn_kwargs_to_inputs(module, *args, **kwargs)
        inputs = [*args]
        cached.append(change_tensor_device_placement(inputs, torch.device('cpu')) if cache_on_cpu else inputs)
        raise StopForwardException

    handle = module.register_forward_pre_hook(keep_inputs_and_stop, with_kwargs=True)
    try:
        for batch in cached_dataset:
            try:
                with in_eval_mode(model), torch.no_grad():
                    forward_fn(model, batch)
            except StopForwardException:
                pass
    finally:
        handle.remove()
    if len(cached) != len(cached_dataset):
        raise RuntimeError(f"module '{module_name}' was reached by {len(cached)} of {len(cached_dataset)} forward "
                           "passes: a checkpoint has to lie on the path of every batch, once")
    return cached


class ModuleData:
    """Collects the input to / output of one module of a model during a forward pass that stops at that module."""

    def __init__(self, model: nn.Module, module: nn.Module, forward_fn: Callable = None):
        self._model = model
        self._module = module
        self._forward_fn = forward_fn or _default_forward

    def collect_inp_out_data(self, model_input, collect_input: bool, collect_output: bool):
        inp_data, out_data = [], []

        def hook(_module, inputs, keywords, output):
            if collect_input:
                if not inputs:
                    # called with keyword arguments only (module(input=x)): the first tensor among them
                    inputs = tuple(v for v in keywords.values() if isinstance(v, torch.Tensor))[:1]
                inp_data.append(inputs[0] if isinstance(inputs, tuple) and len(inputs) == 1 else inputs)
            if collect_output:
                out_data.append(output)
            raise StopForwardException

        handle = self._module.register_forward_hook(hook, with_kwargs=True)
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


# ------------------------------------------------------------------------------------ encodings on disk (v1 format)
# The JSON entry of one encoding is {'min', 'max', 'scale', 'offset', 'bitwidth', 'is_symmetric', 'dtype'}
# (reference aimet_torch/utils.py:785-800, 1140-1170).
def create_encoding_dict(encoding, quantizer, propagate_encodings: bool = False):
    """Exportable dictionary of one TfEncoding of `quantizer`; None when there is no encoding."""
    from .common.defs import QuantizationDataType  # pylint: disable=import-outside-toplevel
    if quantizer.data_type == QuantizationDataType.float:
        return {'bitwidth': quantizer.bitwidth, 'dtype': 'float'}
    if not encoding:
        return None
    if propagate_encodings:
        return {'bitwidth': encoding.bw, 'dtype': 'int'}
    return {'min': encoding.min, 'max': encoding.max, 'scale': encoding.delta, 'offset': int(encoding.offset),
            'bitwidth': encoding.bw, 'is_symmetric': str(quantizer.use_symmetric_encodings), 'dtype': 'int'}


def compute_encoding_for_given_bitwidth(data, bitwidth: int, quant_scheme, is_symmetric: bool, data_type) -> Dict:
    """Encoding dictionary of `data` (numpy array or tensor; it is analysed on the current GPU) for the given bitwidth,
    scheme and symmetry; {} when no valid encoding exists (reference aimet_torch/utils.py:803-829)."""
    # pylint: disable=import-outside-toplevel
    from .common.AimetTensorQuantizer import AimetTensorQuantizer
    from .common.defs import MAP_QUANT_SCHEME_TO_PYMO, QuantizationDataType
    tensor = torch.as_tensor(data, dtype=torch.float32).cuda()
    analyzer = AimetTensorQuantizer(MAP_QUANT_SCHEME_TO_PYMO[quant_scheme])
    analyzer.updateStats(tensor, True)
    encoding, is_encoding_valid = analyzer.getEncoding(bitwidth, is_symmetric, False, False)
    if not is_encoding_valid:
        return {}
    return {'min': encoding.min, 'max': encoding.max, 'scale': encoding.delta, 'offset': encoding.offset,
            'bitwidth': encoding.bw, 'is_symmetric': str(is_symmetric),
            'dtype': 'int' if data_type == QuantizationDataType.int else 'float'}


def create_encoding_from_dict(encoding_dict: dict):
    """TfEncoding from its dictionary form."""
    from .common import libpymo  # pylint: disable=import-outside-toplevel
    if encoding_dict.get('is_symmetric') not in ('True', 'False'):
        raise AssertionError(f"Unexpected value for is_symmetric: {encoding_dict.get('is_symmetric')}")
    return libpymo.TfEncoding(encoding_dict.get('min'), encoding_dict.get('max'), encoding_dict.get('scale'),
                              encoding_dict.get('offset'), encoding_dict.get('bitwidth'))


def _check_is_symmetric_flag(quantizer, encoding_dict: Dict, strict: bool):
    if 'is_symmetric' not in encoding_dict:
        raise AttributeError("Provided encoding doesn't have 'is_symmetric' flag")
    is_symmetric = encoding_dict['is_symmetric'] == 'True'
    if quantizer.use_symmetric_encodings != is_symmetric and strict:
        raise AssertionError(f"Provided 'is_symmetric' flag in encodings (set to {is_symmetric}) doesn't match with "
                             f"quantizer setting (set to {quantizer.use_symmetric_encodings})")


def validate_is_symmetric_flag(quantizer, encoding_dict: Dict, strict: bool = True):
    """The 'is_symmetric' flag of an imported encoding must agree with the quantizer: always for a full encoding,
    and for a partial one when `strict` (reference aimet_torch/utils.py:1199-1270)."""
    if not (encoding_dict.get('max', 0) == 0 and encoding_dict.get('min', 0) == 0) and \
            encoding_dict.get('delta', 0) != 0:
        _check_is_symmetric_flag(quantizer, encoding_dict, strict=True)
    _check_is_symmetric_flag(quantizer, encoding_dict, strict=strict)


def compute_partial_encoding(quantizer, encoding_dict: Dict) -> Dict:
    """Completes an encoding given only as (min, max) or only as (scale, offset)
    (reference aimet_torch/utils.py:1273-1302; the arithmetic is DlQuantization's computePartialEncoding,
    ModelOptimizations/DlQuantization/src/TensorQuantizer.cpp:327-343 and quantization_utils.cpp:158-238)."""
    from . import ops  # pylint: disable=import-outside-toplevel
    bw = encoding_dict.get('bitwidth')
    e_max, e_min = encoding_dict.get('max', 0), encoding_dict.get('min', 0)
    delta, offset = encoding_dict.get('scale', 0), encoding_dict.get('offset', 0)
    if not (e_max == 0 and e_min == 0) and delta != 0:
        return encoding_dict                                   # already complete
    sym, uns, strict = quantizer.use_symmetric_encodings, quantizer.use_unsigned_symmetric, \
        quantizer.use_strict_symmetric
    if not bw:
        raise ValueError("Encodings must have a valid non-zero bitwidth")
    if e_min == 0 and e_max == 0:
        # min / max from delta / offset
        if delta == 0 and offset > 0:
            raise ValueError("Encoding must have a valid non-zero delta/offset if min and max are zero")
        num_steps = 2.0 ** bw - 1
        if sym and strict:
            num_steps -= 1
        e_min = offset * delta
        if sym and (e_min < 0.0 or not uns):
            e_max = delta * (num_steps // 2)
        else:
            e_max = delta * num_steps + e_min
        if e_max - e_min < 1e-5:                               # gateMinMax: zero inside, a real range
            e_min, e_max = min(e_min, 0.0), max(e_max, 0.0)
            e_max = max(e_max, e_min + 1e-5)
    elif delta == 0:
        # delta / offset from min / max, which are kept as given
        if offset != 0:
            raise ValueError("Encoding delta and offset must be zero to use this function")
        computed = ops.get_computed_encodings(bw, e_min, e_max, sym, strict, uns)
        delta, offset = computed.delta, computed.offset
    else:
        raise RuntimeError("Cannot determine how to compute partial encoding")
    encoding_dict['max'], encoding_dict['min'] = e_max, e_min
    encoding_dict['scale'], encoding_dict['offset'] = delta, offset
    encoding_dict['is_symmetric'] = 'True' if quantizer.use_symmetric_encodings else 'False'
    return encoding_dict


def get_per_channel_quantizer_from_per_tensor(quantizer, original_module: nn.Module):
    """Per-channel quantizer with the settings of a per-tensor one (axis 0; axis 1 for transposed convolutions)."""
    from .v1.tensor_quantizer import StaticGridPerChannelQuantizer  # pylint: disable=import-outside-toplevel
    channel_axis = 0
    if isinstance(original_module, (nn.ConvTranspose1d, nn.ConvTranspose2d, nn.ConvTranspose3d)) and \
            len(original_module.weight.shape) > 1:
        channel_axis = 1
    new = StaticGridPerChannelQuantizer(quantizer.bitwidth, quantizer.round_mode, quantizer.quant_scheme,
                                        quantizer.use_symmetric_encodings,
                                        num_channels=original_module.weight.shape[channel_axis],
                                        enabled_by_default=quantizer.enabled, ch_axis=channel_axis,
                                        data_type=quantizer.data_type)
    new.use_strict_symmetric, new.use_unsigned_symmetric = quantizer.use_strict_symmetric, \
        quantizer.use_unsigned_symmetric
    return new


def get_per_tensor_quantizer_from_per_channel(quantizer):
    """Per-tensor quantizer with the settings of a per-channel one."""
    from .v1.tensor_quantizer import StaticGridPerTensorQuantizer  # pylint: disable=import-outside-toplevel
    new = StaticGridPerTensorQuantizer(quantizer.bitwidth, quantizer.round_mode, quantizer.quant_scheme,
                                       quantizer.use_symmetric_encodings, enabled_by_default=quantizer.enabled,
                                       data_type=quantizer.data_type)
    new.use_strict_symmetric, new.use_unsigned_symmetric = quantizer.use_strict_symmetric, \
        quantizer.use_unsigned_symmetric
    return new
