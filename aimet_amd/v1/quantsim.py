"""QuantizationSimModel of the v1 path.

Mirrors the user-facing surface of TrainingExtensions/torch/src/python/aimet_torch/v1/quantsim.py
(constructor :225-307, compute_encodings :381-448, encodings export :486-576) and the quantizer-configuration
semantics of TrainingExtensions/torch/src/python/aimet_torch/quantsim_config/quantsim_config.py:291-593 for the JSON
keys that matter to this path: defaults (ops / params / strict_symmetric / unsigned_symmetric /
per_channel_quantization), params, op_type, supergroups, model_input, model_output.

The reference discovers the graph with torch.jit.trace (ConnectedGraph).  Here one forward pass with hooks on the
leaf modules records the execution order and which module produced / consumed each tensor; that is enough to apply
the supergroup and model-input rules to models built from modules (functional ``+`` needs the ``Add`` module of
aimet_amd.v1.nn.modules.custom, as in the reference).
"""
import copy
import inspect
import json
import math
import os
import pickle
from typing import Dict, List, Tuple, Union

import torch
from torch import nn

from .. import ops
from ..common.defs import QuantizationDataType, QuantScheme
from .nn.modules import custom
from .qc_quantize_op import LearnedGridQuantWrapper, QcQuantizeOpMode, QcQuantizeWrapper, StaticGridQuantWrapper
from .tensor_quantizer import (LearnedGridTensorQuantizer, StaticGridPerChannelQuantizer,
                               initialize_learned_grid_quantizer_attributes)

# same rules as the reference's aimet_common/quantsim_config/default_config.json
DEFAULT_CONFIG = {
    "defaults": {"ops": {"is_output_quantized": "True"},
                 "params": {"is_quantized": "True", "is_symmetric": "True"},
                 "strict_symmetric": "False", "per_channel_quantization": "False"},
    "params": {"bias": {"is_quantized": "False"}},
    "op_type": {"Dropout": {"is_output_quantized": "False"}, "Flatten": {"is_output_quantized": "False"}},
    "supergroups": [{"op_list": ["Conv", "Relu"]}, {"op_list": ["ConvTranspose", "Relu"]},
                    {"op_list": ["Conv", "Clip"]}, {"op_list": ["Add", "Relu"]}, {"op_list": ["Gemm", "Relu"]}],
    "model_input": {"is_input_quantized": "True"},
    "model_output": {},
}

_OP_TYPES = (
    ((nn.ConvTranspose1d, nn.ConvTranspose2d, nn.ConvTranspose3d), "ConvTranspose"),
    ((nn.Conv1d, nn.Conv2d, nn.Conv3d), "Conv"),
    ((nn.Linear,), "Gemm"),
    ((nn.ReLU,), "Relu"),
    ((nn.ReLU6, nn.Hardtanh), "Clip"),
    ((nn.BatchNorm1d, nn.BatchNorm2d, nn.BatchNorm3d), "BatchNormalization"),
    ((nn.MaxPool1d, nn.MaxPool2d, nn.MaxPool3d), "MaxPool"),
    ((nn.AvgPool1d, nn.AvgPool2d, nn.AvgPool3d), "AveragePool"),
    ((nn.AdaptiveAvgPool1d, nn.AdaptiveAvgPool2d), "GlobalAveragePool"),
    ((nn.Dropout, nn.Dropout2d), "Dropout"),
    ((nn.Flatten,), "Flatten"),
    ((nn.Sigmoid,), "Sigmoid"),
    ((nn.Tanh,), "Tanh"),
    ((nn.Softmax,), "Softmax"),
    ((nn.LayerNorm,), "LayerNormalization"),
    ((custom.Add,), "Add"),
    ((custom.Subtract,), "Sub"),
    ((custom.Multiply,), "Mul"),
    ((custom.Concat,), "Concat"),
)


def _op_type(module: nn.Module) -> str:
    for classes, name in _OP_TYPES:
        if isinstance(module, classes):
            return name
    return type(module).__name__


def _declared_inputs(module: nn.Module) -> int:
    """Number of tensors a module that was never called would take: the positional parameters of its forward() that
    have no default (two for the elementwise modules), at least one."""
    try:
        params = inspect.signature(module.forward).parameters.values()
    except (TypeError, ValueError):
        return 1
    required = [p for p in params if p.kind in (p.POSITIONAL_ONLY, p.POSITIONAL_OR_KEYWORD) and p.default is p.empty]
    return max(1, len(required))


def _flag(d: dict, key: str, default=None):
    if key not in d:
        return default
    return str(d[key]) == "True"


_INIT_SCHEME = {
    QuantScheme.post_training_tf: QuantScheme.post_training_tf,
    QuantScheme.post_training_tf_enhanced: QuantScheme.post_training_tf_enhanced,
    QuantScheme.post_training_percentile: QuantScheme.post_training_percentile,
    QuantScheme.training_range_learning_with_tf_init: QuantScheme.post_training_tf,
    QuantScheme.training_range_learning_with_tf_enhanced_init: QuantScheme.post_training_tf_enhanced,
}


_CONSTANT = "__constant__"     # source of a module input that does not depend on the model's inputs
# torch functions, tensor methods and operators that the reference's connected graph lists as Add / Mul / Div / Concat
_ELEMENTWISE_FUNCTIONS = {
    **dict.fromkeys(('add', 'add_', '__add__', '__radd__', '__iadd__'), 'Add'),
    **dict.fromkeys(('mul', 'mul_', 'multiply', 'multiply_', '__mul__', '__rmul__', '__imul__'), 'Mul'),
    **dict.fromkeys(('div', 'div_', 'divide', 'divide_', 'true_divide', 'true_divide_', '__truediv__',
                     '__rtruediv__', '__itruediv__'), 'Div'),
    **dict.fromkeys(('cat', 'concat', 'concatenate'), 'Concat'),
}
_FLOAT16_ENTRY = object()     # marks a float16 quantizer in the export: it has no encoding, only a type


def _exported_encoding(quantizer):
    """The encoding a quantizer is exported with: learned-grid quantizers report the one their quant scheme means
    (reference get_encoding_by_quantizer, qc_quantize_op.py:1507-1519)."""
    if not quantizer.enabled:
        return None
    if quantizer.data_type == QuantizationDataType.float:
        return _FLOAT16_ENTRY if quantizer.bitwidth != 32 else None      # reference quantsim.py:2320
    if isinstance(quantizer, LearnedGridTensorQuantizer):
        return quantizer.get_effective_encoding()
    return quantizer.encoding


class QuantParams:
    """The quantization settings other techniques pass along to build a simulation model (reference :103-129)."""

    def __init__(self, weight_bw: int = 8, act_bw: int = 8, round_mode: str = 'nearest',
                 quant_scheme: Union[QuantScheme, str] = QuantScheme.post_training_tf_enhanced,
                 config_file: str = None):
        self.weight_bw, self.act_bw, self.round_mode = weight_bw, act_bw, round_mode
        self.quant_scheme, self.config_file = quant_scheme, config_file


class QuantizationSimModel:
    """Adds quantization simulation ops to a model for off-target simulation of quantized inference accuracy."""

    # pylint: disable=too-many-arguments
    def __init__(self, model: nn.Module, dummy_input: Union[torch.Tensor, Tuple],
                 quant_scheme: Union[str, QuantScheme] = QuantScheme.post_training_tf_enhanced,
                 rounding_mode: str = 'nearest', default_output_bw: int = 8, default_param_bw: int = 8,
                 in_place: bool = False, config_file: str = None,
                 default_data_type: QuantizationDataType = QuantizationDataType.int):
        if isinstance(quant_scheme, str):
            quant_scheme = {'tf': QuantScheme.post_training_tf,
                            'tf_enhanced': QuantScheme.post_training_tf_enhanced,
                            'percentile': QuantScheme.post_training_percentile}[quant_scheme]
        if quant_scheme not in _INIT_SCHEME:
            raise ValueError(f"quant_scheme {quant_scheme} is not implemented (tf, tf_enhanced, percentile and the "
                             "two range-learning schemes are)")
        if rounding_mode not in ('nearest', 'stochastic'):
            raise ValueError('Parameter round mode can only be nearest or stochastic')
        if default_param_bw < 4 or default_param_bw > 32 or default_output_bw < 4 or default_output_bw > 32:
            raise ValueError('Default bitwidth for parameters and activations must be between 4 and 32')
        if default_data_type == QuantizationDataType.float and \
                (default_output_bw not in (8, 16) or default_param_bw not in (8, 16)):
            raise ValueError('float data_type can only be used when default_output_bw and default_param_bw are '
                             '16 (float16) or 8 (8-bit float grid)')
        if default_data_type == QuantizationDataType.float and quant_scheme not in (
                QuantScheme.post_training_tf, QuantScheme.post_training_tf_enhanced,
                QuantScheme.post_training_percentile):
            raise NotImplementedError('range learning on float16 quantizers is not implemented')
        self._default_data_type = default_data_type
        self.model = model if in_place else copy.deepcopy(model)
        self._quant_scheme = quant_scheme
        self._percentile_value = 100                 # default of the reference (:278)
        self._rounding_mode = rounding_mode
        self._default_output_bw = default_output_bw
        self._default_param_bw = default_param_bw
        self._config = DEFAULT_CONFIG if config_file is None else self._load_config(config_file)
        dummy_input = dummy_input if isinstance(dummy_input, (tuple, list)) else (dummy_input,)
        self._graph = self._trace(self.model, dummy_input)
        self._add_quantization_wrappers()
        self._configure_quantization_ops()

    # ------------------------------------------------------------------------------------------------ construction
    @staticmethod
    def _load_config(config_file) -> dict:
        """`config_file`: path of a JSON configuration, or the configuration itself as a dictionary."""
        if isinstance(config_file, dict):
            return config_file
        with open(config_file) as f:
            return json.load(f)

    @staticmethod
    def _is_leaf(module: nn.Module) -> bool:
        return len(list(module.children())) == 0

    def _trace(self, model: nn.Module, dummy_input: Tuple):
        """One hooked forward pass: execution order of the leaf modules and tensor producers / consumers.

        Every positional input of a module is classified: produced by a module, a model input, an intermediate value
        that a functional op computed from the model's inputs (producer unknown: None), or a constant -- a tensor
        that does not depend on the model's inputs (a buffer, a tensor created in forward) or a python number.
        Constants are told from intermediates by following, through every torch function called during the pass,
        which tensors derive from the model's inputs.  The same watch names the results of the element-wise
        operations that the reference's configurator treats as ops of their own although no module stands for them
        (Add, Mul, Div, Concat written as functions or operators; quantsim_config.py:879-885): a module that reads
        such a result directly gets the source ("__functional__", type, index into self._functional_ops).
        """
        records, handles = [], []
        producer: Dict[int, str] = {}
        consumers: Dict[str, List[str]] = {}      # producing module -> consuming modules
        keep_alive = []
        derived = set()                           # ids of tensors computed from the model's inputs
        names = {m: n for n, m in model.named_modules()}

        def tensors_in(obj):
            if isinstance(obj, torch.Tensor):
                yield obj
            elif isinstance(obj, (list, tuple)):
                for item in obj:
                    yield from tensors_in(item)
            elif isinstance(obj, dict):
                for item in obj.values():
                    yield from tensors_in(item)

        for t in tensors_in(dummy_input):
            producer[id(t)] = "__model_input__"
            derived.add(id(t))

        functional: Dict[int, tuple] = {}         # id of a derived tensor -> source tuple of the functional op
        functional_ops = self._functional_ops = []    # per functional op: type, modules that made its operands

        class Follow(torch.overrides.TorchFunctionMode):
            def __torch_function__(self, func, types, args=(), kwargs=None):
                out = func(*args, **(kwargs or {}))
                if any(id(t) in derived for t in tensors_in((args, kwargs or {}))):
                    fname = getattr(func, '__name__', None) or ''
                    # what a leaf module computes inside belongs to that module
                    op_type = _ELEMENTWISE_FUNCTIONS.get(fname) if not inside_leaf[0] else None
                    in_place = (fname.endswith('_') and not fname.endswith('__')) or fname.startswith('__i')
                    if op_type is not None:
                        operands = [producer.get(id(t)) for t in tensors_in((args, kwargs or {}))]
                        functional_ops.append({"type": op_type, "producers": [
                            p for p in operands if p is not None and p != "__model_input__"]})
                    for t in tensors_in(out):
                        keep_alive.append(t)
                        derived.add(id(t))
                        if in_place or op_type is not None:
                            # an in-place operation hands back the tensor it was given: from here on the value is
                            # this operation's, no longer that of the module which made the tensor
                            producer.pop(id(t), None)
                            functional.pop(id(t), None)
                        if op_type is not None:
                            functional[id(t)] = ("__functional__", op_type, len(functional_ops) - 1)
                return out

        def classify(value):
            if isinstance(value, torch.Tensor):
                if id(value) in producer:
                    return producer[id(value)]
                if id(value) in functional:
                    return functional[id(value)]
                return None if id(value) in derived else _CONSTANT
            if isinstance(value, (int, float)) and not isinstance(value, bool):
                return _CONSTANT
            return None

        inside_leaf = [0]

        def pre_hook(module, inputs):
            inside_leaf[0] += 1

        def hook(module, inputs, output):
            inside_leaf[0] -= 1
            name = names[module]
            ins = [t for t in inputs if isinstance(t, torch.Tensor)]
            outs = [t for t in (output if isinstance(output, (tuple, list)) else (output,))
                    if isinstance(t, torch.Tensor)]
            keep_alive.extend(ins + outs)            # ids stay unique while the pass runs
            sources = [classify(value) for value in inputs]
            for src in sources:
                # resolved now, not afterwards: an in-place op returns the tensor it was given, so the tensor's id
                # says nothing about who produced the value a later module reads
                if isinstance(src, str) and src is not _CONSTANT:
                    consumers.setdefault(src, []).append(name)
            singleton = [value.numel() == 1 if isinstance(value, torch.Tensor) else src is _CONSTANT
                         for value, src in zip(inputs, sources)]
            records.append({"name": name, "module": module, "type": _op_type(module), "inputs": sources,
                            "singleton": singleton,
                            "num_inputs": max(1, len(inputs)), "num_outputs": max(1, len(outs))})
            for t in outs:
                producer[id(t)] = name
                functional.pop(id(t), None)
                derived.add(id(t))

        for module in model.modules():
            # nn.Identity is never wrapped (reference :205-207, :1430-1434); unhooked, the tensor it passes through
            # keeps its producer
            if self._is_leaf(module) and module is not model and not isinstance(module, nn.Identity):
                handles.append(module.register_forward_pre_hook(pre_hook))
                handles.append(module.register_forward_hook(hook))
        was_training = model.training
        model.eval()
        try:
            with torch.no_grad(), Follow():
                out = model(*dummy_input)
        finally:
            for h in handles:
                h.remove()
            model.train(was_training)
        records = self._one_record_per_module(records)
        model_outputs = {producer.get(id(t)) for t in tensors_in(out)}
        for r in records:
            r["consumers"] = list(consumers.get(r["name"], []))
            r["is_model_output"] = r["name"] in model_outputs
        # leaf modules that the forward pass never reached are wrapped too, with the default configuration
        # (the reference wraps every quantizable leaf, :1440-1454)
        reached = {r["name"] for r in records}
        for name, module in model.named_modules():
            if self._is_leaf(module) and module is not model and not isinstance(module, nn.Identity) \
                    and name not in reached and not isinstance(module, QcQuantizeWrapper):
                records.append({"name": name, "module": module, "type": _op_type(module), "inputs": [],
                                "num_inputs": _declared_inputs(module), "num_outputs": 1, "consumers": [],
                                "is_model_output": False})
        return records

    @staticmethod
    def _one_record_per_module(records):
        """A module that the forward pass runs more than once gets one wrapper, as every module does, and that wrapper's
        quantizers see all its uses (the reference does not stop at such a model either: its test
        test_no_hard_stop_upon_reused_modules).  For the configuration it is one node at the place of its first use:
        the readers of all its uses are its readers, a position that reads the model's input or a constant in a later
        use only counts as reading it, and it has as many input / output quantizers as its widest use."""
        first_use = {}
        kept = []
        for rec in records:
            first = first_use.get(rec["name"])
            if first is None:
                first_use[rec["name"]] = rec
                kept.append(rec)
                continue
            for position, source in enumerate(rec["inputs"]):
                if position >= len(first["inputs"]):
                    first["inputs"].append(source)
                    first["singleton"].append(rec["singleton"][position])
                elif first["inputs"][position] != source and (source == "__model_input__" or source is _CONSTANT):
                    first["inputs"][position] = source
                    first["singleton"][position] = rec["singleton"][position]
            first["num_inputs"] = max(first["num_inputs"], rec["num_inputs"])
            first["num_outputs"] = max(first["num_outputs"], rec["num_outputs"])
        return kept

    def _add_quantization_wrappers(self):
        for rec in self._graph:
            # range-learning schemes start as static-grid wrappers of the scheme they are initialised from and are
            # swapped for learned-grid wrappers once encodings have been computed
            wrapper = StaticGridQuantWrapper(rec["module"], self._default_param_bw, self._default_output_bw,
                                             self._rounding_mode, _INIT_SCHEME[self._quant_scheme],
                                             num_inputs=rec["num_inputs"], num_outputs=rec["num_outputs"],
                                             data_type=self._default_data_type)
            rec["wrapper"] = wrapper
            for idx, src in enumerate(rec["inputs"]):
                wrapper.input_quantizers[idx].is_const = src is _CONSTANT     # reference :1456-1471
                wrapper.input_quantizers[idx].is_singleton = rec["singleton"][idx]
            parent = self.model
            *path, leaf = rec["name"].split('.')
            for p in path:
                parent = getattr(parent, p)
            setattr(parent, leaf, wrapper)

    def _configure_quantization_ops(self):
        """Precedence as in the reference: defaults -> params -> op_type -> supergroups -> model_input -> model_output."""
        cfg = self._config
        defaults = cfg.get("defaults", {})
        out_q = _flag(defaults.get("ops", {}), "is_output_quantized", False)
        in_q = _flag(defaults.get("ops", {}), "is_input_quantized", False)
        act_sym = _flag(defaults.get("ops", {}), "is_symmetric", False)
        par_q = _flag(defaults.get("params", {}), "is_quantized", False)
        par_sym = _flag(defaults.get("params", {}), "is_symmetric", False)
        strict = _flag(defaults, "strict_symmetric", False)
        unsigned = _flag(defaults, "unsigned_symmetric", False)
        per_channel = _flag(defaults, "per_channel_quantization", False)
        by_name = {r["name"]: r for r in self._graph}
        for rec in self._graph:
            w: StaticGridQuantWrapper = rec["wrapper"]
            op_cfg = cfg.get("op_type", {}).get(rec["type"], {})
            w.enable_output_quantizers(_flag(op_cfg, "is_output_quantized", out_q))
            w.enable_input_quantizers(_flag(op_cfg, "is_input_quantized", in_q))
            for q in w.input_quantizers + w.output_quantizers:
                q.use_symmetric_encodings = _flag(op_cfg, "is_symmetric", act_sym)
                q.use_strict_symmetric, q.use_unsigned_symmetric = strict, unsigned
            fixed = op_cfg.get("encoding_constraints")
            if fixed is not None:
                # the op's outputs get this range whatever passes through them (reference quantsim_config.py:463-465,
                # :806-808, :842-843)
                for q in w.output_quantizers:
                    q.encoding_min_max_fixed_vals = (fixed["min"], fixed["max"])
            for pname, q in w.param_quantizers.items():
                pcfg = dict(cfg.get("params", {}).get(pname, {}))
                pcfg.update(op_cfg.get("params", {}).get(pname, {}))
                q.enabled = _flag(pcfg, "is_quantized", par_q)
                q.use_symmetric_encodings = _flag(pcfg, "is_symmetric", par_sym)
                q.use_strict_symmetric, q.use_unsigned_symmetric = strict, unsigned
            if rec["type"] == "BatchNormalization":
                w.enable_param_quantizers(False, None)        # BN statistics are never quantized
            if _flag(op_cfg, "per_channel_quantization", per_channel) and w.param_quantizers:
                w.enable_per_channel_quantization()
        # functional Add / Mul / Div / Concat have no wrapper: their "output quantizer" is the input quantizer of the
        # modules that read the result, their "input quantizers" are the output quantizers of the modules that made
        # the operands (reference quantsim_config.py:183-237)
        functional_readers: Dict[int, list] = {}
        for rec in self._graph:
            for idx, src in enumerate(rec["inputs"]):
                if isinstance(src, tuple):
                    functional_readers.setdefault(src[2], []).append(rec)
                    setting = _flag(cfg.get("op_type", {}).get(src[1], {}), "is_output_quantized", None)
                    if setting is not None:
                        rec["wrapper"].input_quantizers[idx].enabled = setting
                    elif out_q:
                        rec["wrapper"].input_quantizers[idx].enabled = True
        for op in self._functional_ops:
            setting = _flag(cfg.get("op_type", {}).get(op["type"], {}), "is_input_quantized", None)
            if setting is None and not in_q:
                continue
            for name in op["producers"]:
                by_name[name]["wrapper"].output_quantizers[0].enabled = True if setting is None else setting
        # a batch norm that is the only reader of a convolution / linear layer can be folded into it: such batch
        # norms are skipped when supergroups are matched, and afterwards take over the layer's output quantizer
        # (reference quantsim_config.py:486-560)
        def only_consumer(rec):
            readers = set(rec["consumers"])
            return by_name[next(iter(readers))] if len(readers) == 1 and not rec["is_model_output"] else None

        foldable = {}                             # batch norm name -> record of the layer it folds into
        for rec in self._graph:
            if rec["type"] in ("Conv", "ConvTranspose", "Gemm"):
                module = rec["module"]
                if isinstance(module, nn.ConvTranspose2d) and module.groups != 1:
                    continue
                reader = only_consumer(rec)
                if reader is not None and reader["type"] == "BatchNormalization":
                    foldable[reader["name"]] = rec

        def next_in_chain(rec):
            reader = only_consumer(rec)
            while reader is not None and reader["name"] in foldable:
                reader = only_consumer(reader)
            return reader

        # supergroups: inside a matched chain only the last op keeps its output quantizer
        for group in cfg.get("supergroups", []):
            ops_list = group["op_list"]
            for rec in self._graph:
                if rec["type"] != ops_list[0] or rec["name"] in foldable:
                    continue
                chain, cur = [rec], rec
                for want in ops_list[1:]:
                    cur = next_in_chain(cur)
                    if cur is None or cur["type"] != want:
                        chain = None
                        break
                    chain.append(cur)
                if chain is None:
                    continue
                for member in chain[:-1]:
                    member["wrapper"].enable_output_quantizers(False)
                for member in chain[1:]:
                    member["wrapper"].enable_input_quantizers(False)
            # a chain that starts at a functional op: the op itself has nothing to switch off, the modules after it
            # are treated as inside the chain (reference SupergroupConfigCallback, quantsim_config.py:80-104)
            for index, readers in functional_readers.items():
                if self._functional_ops[index]["type"] != ops_list[0] or len(readers) != 1 or len(ops_list) < 2:
                    continue
                chain, cur = [], readers[0]
                for position, want in enumerate(ops_list[1:]):
                    if position:
                        cur = next_in_chain(cur)
                    if cur is None or cur["type"] != want:
                        chain = None
                        break
                    chain.append(cur)
                if chain is None:
                    continue
                for member in chain[:-1]:
                    member["wrapper"].enable_output_quantizers(False)
                for member in chain:
                    member["wrapper"].enable_input_quantizers(False)
        for bn_name, layer in foldable.items():
            bn_wrapper, layer_wrapper = by_name[bn_name]["wrapper"], layer["wrapper"]
            bn_wrapper.enable_input_quantizers(False)
            bn_wrapper.enable_param_quantizers(False, None)
            for layer_q, bn_q in zip(layer_wrapper.output_quantizers, bn_wrapper.output_quantizers):
                bn_q.enabled = layer_q.enabled
                layer_q.enabled = False
        if _flag(cfg.get("model_input", {}), "is_input_quantized", False):
            for rec in self._graph:
                # model inputs and constant inputs alike (reference quantsim_config.py:560-581)
                for idx, src in enumerate(rec["inputs"]):
                    if (src == "__model_input__" or src is _CONSTANT) and idx < len(rec["wrapper"].input_quantizers):
                        rec["wrapper"].input_quantizers[idx].enabled = True
        if _flag(cfg.get("model_output", {}), "is_output_quantized", False):
            for rec in self._graph:
                if rec["is_model_output"]:
                    rec["wrapper"].enable_output_quantizers(True)

    # --------------------------------------------------------------------------------------------------- usage
    def quant_wrappers(self):
        """Generator of (name, wrapper) in the model."""
        for name, module in self.model.named_modules():
            if isinstance(module, QcQuantizeWrapper):
                yield name, module

    named_qmodules = quant_wrappers     # the newer name of the same generator (reference quantsim.py:1856-1868)

    def qmodules(self):
        """The wrappers without their names."""
        yield from (wrapper for _, wrapper in self.quant_wrappers())

    _get_qc_quantized_layers = staticmethod(lambda model: [(n, m) for n, m in model.named_modules()
                                                           if isinstance(m, QcQuantizeWrapper)])

    def __str__(self):
        lines = ["-------------------------", "Quantized Model Report", "-------------------------"]
        for name, w in self.quant_wrappers():
            lines.append(f"Layer: {name}")
            lines.append(f"  inputs : {[(q.enabled, q.bitwidth) for q in w.input_quantizers]}")
            lines.append(f"  params : {{{', '.join(f'{k}: ({q.enabled}, {q.bitwidth})' for k, q in w.param_quantizers.items())}}}")
            lines.append(f"  outputs: {[(q.enabled, q.bitwidth) for q in w.output_quantizers]}")
        return "\n".join(lines)

    def compute_encodings(self, forward_pass_callback, forward_pass_callback_args):
        """Runs `forward_pass_callback(model, args)` in ANALYSIS mode, then computes every encoding and switches the
        wrappers to ACTIVE (reference :425-448)."""
        self.prepare_sim_for_compute_encodings()
        was_training = self.model.training
        self.model.eval()
        try:
            # parameter encodings do not depend on the batches: observed and read back while the device is idle
            fed = [q for layer in self._static_grid_layers() for q in layer.observe_params_ahead()]
            for quantizer in fed:
                quantizer.compute_encoding()
            with torch.no_grad():
                forward_pass_callback(self.model, forward_pass_callback_args)
        finally:
            self.model.train(was_training)
            for layer in self._static_grid_layers():
                layer.drop_params_observed_in_vain()
        self.compute_layer_encodings_for_sim()
        if not self.model.training:
            self.quantize_params_together()

    def quantize_params_together(self) -> int:
        """Quantize-dequantizes the parameters of every static-grid wrapper in evaluation mode with ONE launch over
        all of them (aimet_amd.ops.QdqMulti) and leaves the results where the wrappers keep quantized parameters
        between forwards.  Called at the end of compute_encodings(); call it again after the weights have changed
        when the next forwards should not re-quantize tensor by tensor.  Returns the number of tensors it took;
        tensors that cannot go into such a launch (tiny channels, other data types, disabled quantizers) are left
        to their wrappers.  The reference has no counterpart: it quantizes each parameter in each forward
        (qc_quantize_op.py:747-763)."""
        groups = {}
        for layer in self._static_grid_layers():
            if not layer._params_may_be_kept():                      # pylint: disable=protected-access
                continue
            for name, param in layer.get_named_parameters():
                quantizer = layer.param_quantizers[name]
                if not (quantizer.enabled and quantizer.bitwidth != 32 and quantizer.has_encoding() and
                        quantizer.data_type == QuantizationDataType.int and param.is_cuda and
                        param.dtype in (torch.float32, torch.bfloat16) and param.data.is_contiguous()):
                    continue
                data = param.data
                if isinstance(quantizer, StaticGridPerChannelQuantizer):
                    sizes = [*data.shape, 1]
                    num_channel = sizes[quantizer.channel_axis]
                    n_per_channel = math.prod(sizes[quantizer.channel_axis + 1:])
                    params = quantizer.device_params(data.device)[:4]
                else:
                    enc = ops.fill_encoding_info(quantizer.encoding.bw, quantizer.encoding.min, quantizer.encoding.max)
                    num_channel, n_per_channel = 1, data.numel()
                    params = (enc.min, enc.max, enc.delta, enc.offset)       # uploaded below, all at once
                if n_per_channel < 16 or data.numel() >= 2 ** 31:
                    continue
                groups.setdefault((data.device, data.dtype), []).append(
                    (layer, name, param, quantizer, data, num_channel, n_per_channel, params))
        taken = 0
        for (device, _), items in groups.items():
            scalars = [it[7] for it in items if not isinstance(it[7][0], torch.Tensor)]
            uploaded = torch.tensor(scalars, dtype=torch.float64).to(torch.float32).to(device) if scalars else None
            k = 0
            entries = []
            for it in items:
                params = it[7]
                if not isinstance(params[0], torch.Tensor):
                    params = tuple(uploaded[k, j:j + 1] for j in range(4))
                    k += 1
                entries.append((it[4], it[5], it[6], *params))
            for first in range(0, len(entries), ops.QdqMulti.MAX_SEGMENTS):
                chunk = entries[first:first + ops.QdqMulti.MAX_SEGMENTS]
                outputs = ops.QdqMulti(chunk)()
                for it, out in zip(items[first:first + len(chunk)], outputs):
                    layer, name, param, quantizer = it[:4]
                    layer.__dict__.setdefault('_param_cache', {})[name] = (layer._param_cache_key(param, quantizer), out)  # pylint: disable=protected-access
                    taken += 1
        return taken

    def _static_grid_layers(self):
        return [m for _, m in self._get_qc_quantized_layers(self.model) if isinstance(m, StaticGridQuantWrapper)]

    def prepare_sim_for_compute_encodings(self):
        """Statistics cleared, wrappers in ANALYSIS mode (reference :384-403)."""
        for layer in self._static_grid_layers():
            layer.reset_encodings()
            layer.set_mode(QcQuantizeOpMode.ANALYSIS)
            if self._quant_scheme == QuantScheme.post_training_percentile:
                layer.set_percentile_value(self._percentile_value)     # reference :395-400

    def compute_layer_encodings_for_sim(self):
        """Encodings from the gathered statistics, wrappers back to ACTIVE; a quantizer that saw no data is switched
        off (reference :405-423)."""
        layers = self._static_grid_layers()
        # every per-tensor search is started before the first result is waited for: one round trip to the device for
        # the whole model instead of one per quantizer
        for layer in layers:
            for quantizer in list(layer.input_quantizers) + list(layer.output_quantizers):
                quantizer.queue_encoding()
        for layer in layers:
            layer.compute_encoding()
            layer.set_mode(QcQuantizeOpMode.ACTIVE)
        self.replace_wrappers_for_quantize_dequantize()

    def replace_wrappers_for_quantize_dequantize(self):
        """For the range-learning schemes: every static-grid wrapper becomes a learned-grid wrapper that starts from
        the calibrated encodings (reference quantsim.py:764-847)."""
        if self._quant_scheme not in (QuantScheme.training_range_learning_with_tf_init,
                                      QuantScheme.training_range_learning_with_tf_enhanced_init):
            return
        try:
            device = next(self.model.parameters()).device
        except StopIteration:
            device = torch.device('cuda', torch.cuda.current_device())
        replaced = {}
        self._replace_quantization_wrapper(self.model, device, replaced)
        for rec in self._graph:
            rec["wrapper"] = replaced.get(rec["wrapper"], rec["wrapper"])

    def _replace_quantization_wrapper(self, model: nn.Module, device, replaced: dict):
        for name, child in list(model.named_children()):
            if isinstance(child, StaticGridQuantWrapper):
                replaced[child] = self._construct_and_initialize_trainable_wrapper(child, device)
                setattr(model, name, replaced[child])
            elif not isinstance(child, QcQuantizeWrapper):
                self._replace_quantization_wrapper(child, device, replaced)

    def _construct_and_initialize_trainable_wrapper(self, post_training_module: StaticGridQuantWrapper,
                                                    device) -> LearnedGridQuantWrapper:
        # pylint: disable=protected-access
        trainable = LearnedGridQuantWrapper(post_training_module._module_to_wrap, self._default_param_bw,
                                            self._default_output_bw, self._rounding_mode, self._quant_scheme,
                                            device=device, num_inputs=len(post_training_module.input_quantizers),
                                            num_outputs=len(post_training_module.output_quantizers),
                                            data_type=QuantizationDataType.int)
        pairs = list(zip(trainable.output_quantizers, post_training_module.output_quantizers)) + \
            list(zip(trainable.input_quantizers, post_training_module.input_quantizers)) + \
            [(trainable.param_quantizers[n], q) for n, q in post_training_module.param_quantizers.items()]
        for new, old in pairs:
            if isinstance(old, StaticGridPerChannelQuantizer):
                new._ch_axis = old.channel_axis
            initialize_learned_grid_quantizer_attributes(new, old)
            if new.encoding_min_max_fixed_vals is not None:
                new.freeze_encoding()
        return trainable

    def set_percentile_value(self, percentile_value: float):
        """Percentile used by the quantizers of the percentile scheme at the next compute_encodings
        (reference quantsim.py:478-484)."""
        if percentile_value < 90 or percentile_value > 100:
            raise ValueError("Percentile value must be in range [90, 100]")
        self._percentile_value = percentile_value

    def exclude_layers_from_quantization(self, layers_to_exclude: List[nn.Module]):
        """Replaces the given quantization wrappers by the modules they wrap (reference quantsim.py:1419-1433)."""
        self._replace_wrappers(self.model, set(layers_to_exclude))

    @classmethod
    def _replace_wrappers(cls, module: nn.Module, only=None):
        for name, child in list(module.named_children()):
            if isinstance(child, QcQuantizeWrapper):
                if only is None or child in only:
                    setattr(module, name, child.get_original_module())
            else:
                cls._replace_wrappers(child, only)

    @classmethod
    def remove_quantization_wrappers(cls, module: nn.Module):
        """Strips every quantization wrapper below `module` (reference SaveUtils.remove_quantization_wrappers)."""
        cls._replace_wrappers(module, None)

    # ------------------------------------------------------------------------------------ encodings on disk
    @staticmethod
    def _encoding_dict(enc, symmetric: bool) -> dict:
        # the reference's legacy format (aimet_torch/utils.py:1140-1170)
        return {'min': enc.min, 'max': enc.max, 'scale': enc.delta, 'offset': int(enc.offset), 'bitwidth': enc.bw,
                'is_symmetric': str(symmetric), 'dtype': 'int'}

    def get_encodings_dict(self) -> dict:
        param_enc, act_enc = {}, {}
        for name, w in self.quant_wrappers():
            for pname, q in w.param_quantizers.items():
                encoding = _exported_encoding(q)
                if encoding is _FLOAT16_ENTRY:
                    param_enc[f"{name}.{pname}"] = [{'bitwidth': q.bitwidth, 'dtype': 'float'}]
                elif encoding is not None:
                    encs = encoding if isinstance(encoding, list) else [encoding]
                    param_enc[f"{name}.{pname}"] = [self._encoding_dict(e, q.use_symmetric_encodings) for e in encs]
            entry = {}
            for kind, qs in (('input', w.input_quantizers), ('output', w.output_quantizers)):
                for i, q in enumerate(qs):
                    encoding = _exported_encoding(q)
                    if encoding is _FLOAT16_ENTRY:
                        entry.setdefault(kind, {})[str(i)] = {'bitwidth': q.bitwidth, 'dtype': 'float'}
                    elif encoding is not None:
                        entry.setdefault(kind, {})[str(i)] = self._encoding_dict(encoding,
                                                                                 q.use_symmetric_encodings)
            if entry:
                act_enc[name] = entry
        return {'version': '0.6.1', 'activation_encodings': act_enc, 'param_encodings': param_enc,
                'quantizer_args': {'activation_bitwidth': self._default_output_bw,
                                   'param_bitwidth': self._default_param_bw,
                                   'dtype': 'float' if self._default_data_type == QuantizationDataType.float
                                   else 'int',
                                   'quant_scheme': self._quant_scheme.name}}

    def export_encodings(self, path: str, filename_prefix: str) -> str:
        os.makedirs(path, exist_ok=True)
        file = os.path.join(path, filename_prefix + '.encodings')
        with open(file, 'w') as f:
            json.dump(self.get_encodings_dict(), f, sort_keys=True, indent=4)
        return file

    def exclude_param_from_quantization(self, param_name_to_exclude: str):
        """Switches off every quantizer of parameters of this name (reference quantsim.py:753-762)."""
        for _, wrapper in self.quant_wrappers():
            if param_name_to_exclude in wrapper.param_quantizers:
                wrapper.param_quantizers[param_name_to_exclude].enabled = False

    def get_activation_param_encodings(self):
        """(activation encodings, parameter encodings) by module / parameter name (reference quantsim.py:692-728)."""
        exported = self.get_encodings_dict()
        return exported['activation_encodings'], exported['param_encodings']

    def export_weights_to_safetensors(self, path: str, filename_prefix: str):
        """The state dictionary of the model without its quantization wrappers, as `<path>/<prefix>.safetensors`
        (reference :660-678; metadata from the model's `mpp_meta` attribute when it has one)."""
        from safetensors.torch import save_file               # pylint: disable=import-outside-toplevel
        plain = QuantizationSimModel.get_original_model(self.model)
        tensors = {name: value.detach().cpu().contiguous() for name, value in plain.state_dict().items()}
        metadata = {str(k): str(v) for k, v in getattr(self.model, 'mpp_meta', {}).items()}
        save_file(tensors, os.path.join(path, filename_prefix + '.safetensors'), metadata=metadata or None)

    def save_encodings_to_json(self, path: str, filename_prefix: str):
        """<path>/<filename_prefix>.json with the activation and parameter encodings (reference quantsim.py:680-690)."""
        activation_encodings, param_encodings = self.get_activation_param_encodings()
        os.makedirs(path, exist_ok=True)
        with open(os.path.join(path, filename_prefix + '.json'), 'w') as f:
            json.dump({'activation_encodings': activation_encodings, 'param_encodings': param_encodings}, f,
                      sort_keys=True, indent=4)

    @classmethod
    def get_original_model(cls, model: nn.Module, qdq_weights: bool = False) -> nn.Module:
        """A copy of the simulation's model without its quantization wrappers; with qdq_weights the parameters hold
        their quantize-dequantized values (reference quantsim.py:1519-1533)."""
        original = copy.deepcopy(model)
        if qdq_weights:
            cls._apply_qdq_to_model_parameters(original)
        cls.remove_quantization_wrappers(original)
        return original

    @classmethod
    @torch.no_grad()
    def _apply_qdq_to_model_parameters(cls, model: nn.Module):
        # pylint: disable=protected-access
        for module in model.modules():
            if not isinstance(module, QcQuantizeWrapper):
                continue
            was_training = module.training
            module.eval()
            try:
                if isinstance(module, LearnedGridQuantWrapper):
                    module._quantize_params()                       # leaves results of an autograd function in place
                    wrapped = module._module_to_wrap
                    for name, value in list(wrapped._parameters.items()):
                        if value is not None and not isinstance(value, nn.Parameter):
                            wrapped._parameters[name] = nn.Parameter(value.detach(), requires_grad=False)
                else:
                    module._quantize_dequantize_params()
            finally:
                module.train(was_training)

    def export(self, path: str, filename_prefix: str, dummy_input=None, onnx_export_args=None,
               propagate_encodings: bool = False, export_to_torchscript: bool = False,
               use_embedded_encodings: bool = False, export_model: bool = True,
               filename_prefix_encodings: str = None):
        """Writes what the reference's export() (quantsim.py:486-560) writes on the torch side:
        <filename_prefix>.pth, the model without quantization wrappers and with quantize-dequantized weights, and
        <filename_prefix_encodings>_torch.encodings, the encodings by torch module and parameter names.

        The reference goes on to trace an ONNX (or TorchScript) graph and to write a second encodings file keyed by
        that graph's tensor names; graph export is not part of this library, and the arguments that only concern it
        (dummy_input, onnx_export_args, propagate_encodings) are accepted and not used.  export_to_torchscript and
        use_embedded_encodings, which ask for other kinds of graph, raise NotImplementedError."""
        # pylint: disable=too-many-arguments, unused-argument
        if export_to_torchscript or use_embedded_encodings:
            raise NotImplementedError("TorchScript and embedded-encodings exports need the graph exporters, which "
                                      "this library does not have")
        os.makedirs(path, exist_ok=True)
        if export_model:
            torch.save(self.get_original_model(self.model, qdq_weights=True),
                       os.path.join(path, filename_prefix + '.pth'))
        return self.export_encodings(path, (filename_prefix_encodings or filename_prefix) + '_torch')

    def load_encodings(self, encodings, strict: bool = True, partial: bool = True, requires_grad=None,
                       allow_overwrite: bool = True):
        """Imports parameter and activation encodings from a dictionary or a JSON file
        (reference quantsim.py:1695-1836).

        strict: raise when the file names modules / parameters the model does not have, or when an encoding cannot
        be set as the quantizers are configured.  partial: quantizers without an entry are left alone (otherwise
        they are disabled).  requires_grad: for learned-grid quantizers, whether the imported min / max train.
        allow_overwrite: False freezes every imported encoding."""
        if isinstance(encodings, (str, os.PathLike)):
            with open(encodings) as f:
                encodings = json.load(f)
        if 'param_encodings' not in encodings:
            param_encodings, activation_encodings = encodings, {}      # the older AdaRound export: parameters only
        else:
            param_encodings = encodings.get('param_encodings', {})
            activation_encodings = encodings.get('activation_encodings', {})
        if not param_encodings and not activation_encodings:
            raise RuntimeError("the encodings hold neither parameter nor activation entries")
        if strict:
            model_keys = set()
            for name, module in self.model.named_modules():
                model_keys.add(name.replace("._module_to_wrap", ""))
                for pname, _ in module.named_parameters(recurse=False):
                    model_keys.add(f"{name}.{pname}".replace("._module_to_wrap", ""))
            missing = (set(param_encodings) | set(activation_encodings)) - model_keys
            if missing:
                raise RuntimeError("Encoding dictionary contains modules/parameters that doesn't exist in the "
                                   f"model: {', '.join(sorted(missing))}")
        for name, wrapper in self.quant_wrappers():
            try:
                mine = {pname: param_encodings[f'{name}.{pname}'] for pname in wrapper.param_quantizers
                        if f'{name}.{pname}' in param_encodings}
                wrapper.import_param_encodings(mine, strict, partial, requires_grad, allow_overwrite)
                entry = activation_encodings.get(name, {})
                wrapper.import_input_encodings(entry.get('input', {}), strict, partial, requires_grad,
                                               allow_overwrite)
                wrapper.import_output_encodings(entry.get('output', {}), strict, partial, requires_grad,
                                                allow_overwrite)
            except RuntimeError as e:
                raise RuntimeError(f"Encoding import failed for module: {name}.\n{e}") from e

    def load_and_freeze_encodings(self, encoding_path: str, ignore_when_quantizer_disabled: bool = False):
        """Sets parameter and activation encodings from a file exported by this class and freezes them
        (reference :1758-1773)."""
        self.load_encodings(encoding_path, strict=not ignore_when_quantizer_disabled, partial=True,
                            requires_grad=False, allow_overwrite=False)

    def set_and_freeze_param_encodings(self, encoding_path: str):
        """Sets and freezes the parameter encodings of a file written by export_encodings / Adaround
        (reference :1838-1854)."""
        with open(encoding_path) as f:
            encodings = json.load(f)
        encodings.pop('activation_encodings', None)
        self.load_encodings(encodings, strict=True, partial=True, requires_grad=False, allow_overwrite=False)


def load_encodings_to_sim(quant_sim_model: QuantizationSimModel, pytorch_encoding_path: str):
    """Loads an exported encodings file into a simulation model configured like the one that wrote it: wrappers go to
    ACTIVE mode, every quantizer the file has no entry for is switched off, and range-learning models get their
    learned-grid wrappers (reference quantsim.py:2277-2298)."""
    for module in quant_sim_model.model.modules():
        if isinstance(module, QcQuantizeWrapper):
            module.set_mode(QcQuantizeOpMode.ACTIVE)
    quant_sim_model.load_encodings(pytorch_encoding_path, strict=True, partial=False, requires_grad=None,
                                   allow_overwrite=None)
    if isinstance(quant_sim_model, QuantizationSimModel):
        quant_sim_model.replace_wrappers_for_quantize_dequantize()          # a v2 simulation has no wrappers


def save_checkpoint(quant_sim_model, file_path: str):
    """The whole simulation model, pickled, to continue fine-tuning later (reference quantsim.py:2215-2226).  Device
    objects and what the host layer keeps between forwards are not part of the pickle; they are made again on use."""
    with open(file_path, 'wb') as file:
        pickle.dump(quant_sim_model, file)


def load_checkpoint(file_path: str):
    """A simulation model that save_checkpoint() wrote (reference quantsim.py:2229-2238).  As any pickle, only for
    files you wrote yourself."""
    with open(file_path, 'rb') as file:
        return pickle.load(file)


def has_valid_encodings(qc_quantize_op: QcQuantizeWrapper) -> bool:
    """True if any enabled input, parameter or output quantizer of the wrapper holds an encoding (or simulates
    float16, which needs none) -- reference quantsim.py:2301-2323."""
    if not isinstance(qc_quantize_op, QcQuantizeWrapper):
        raise AssertionError("has_valid_encodings is only supported for quantization wrappers")
    quantizers = list(qc_quantize_op.input_quantizers) + list(qc_quantize_op.output_quantizers) + \
        list(qc_quantize_op.param_quantizers.values())
    return any(_exported_encoding(q) is not None for q in quantizers)


def compute_encodings_for_sims(sim_list: List[QuantizationSimModel], forward_pass_callback,
                               forward_pass_callback_args):
    """Calibrates several simulation models with one callback, which receives the list of their models in the order
    of `sim_list` (reference quantsim.py:2326-2356).  All models run in eval mode and without autograd during the
    callback and get their own mode back afterwards."""
    modes = [sim.model.training for sim in sim_list]
    for sim in sim_list:
        sim.prepare_sim_for_compute_encodings()
        sim.model.eval()
    try:
        with torch.no_grad():
            forward_pass_callback([sim.model for sim in sim_list], forward_pass_callback_args)
    finally:
        for sim, mode in zip(sim_list, modes):
            sim.model.train(mode)
    for sim in sim_list:
        sim.compute_layer_encodings_for_sim()
