"""The reference's configurator tests (TrainingExtensions/torch/test/python/test_quantsim_config.py) for the settings
that decide where the quantize-dequantize kernels run: defaults, params, op_type, supergroups, element-wise ops written
as functions, model inputs / outputs, symmetric modes.  Same models (models/test_models.py:158-210, :268-321, :467-500),
same configuration dictionaries, same assertions.  Cases about supported_kernels / hw_version / dtype-override rules
belong to the reference's target-specific kernel tables, which are not rebuilt.
"""
import pytest
import torch
from torch import nn

pytestmark = pytest.mark.gpu

from aimet_amd.common.defs import QuantScheme                                               # noqa: E402
from aimet_amd.v1.nn.modules.custom import Add                                              # noqa: E402
from aimet_amd.v1.qc_quantize_op import QcQuantizeWrapper                                   # noqa: E402
from aimet_amd.v1.quantsim import QuantizationSimModel                                      # noqa: E402


class SingleResidual(nn.Module):
    def __init__(self, num_classes=10, module_add=False):
        super().__init__()
        self.conv1 = nn.Conv2d(3, 32, kernel_size=2, stride=2, padding=2, bias=False)
        self.bn1, self.relu1 = nn.BatchNorm2d(32), nn.ReLU(inplace=True)
        self.maxpool = nn.MaxPool2d(kernel_size=2, stride=2, padding=1)
        self.conv2 = nn.Conv2d(32, 16, kernel_size=2, stride=2, padding=2, bias=False)
        self.bn2, self.relu2 = nn.BatchNorm2d(16), nn.ReLU(inplace=True)
        self.conv3 = nn.Conv2d(16, 8, kernel_size=2, stride=2, padding=2, bias=False)
        if module_add:
            self.add = Add()
        self.relu3 = nn.ReLU(inplace=True)
        self.avgpool = nn.AvgPool2d(3, stride=1)
        self.conv4 = nn.Conv2d(32, 8, kernel_size=2, stride=2, padding=2, bias=True)
        self.ada = nn.AdaptiveAvgPool2d(5)
        self.fc = nn.Linear(72, num_classes)
        self.module_add = module_add

    def forward(self, *inputs):
        x = self.maxpool(self.relu1(self.bn1(self.conv1(inputs[0]))))
        residual = x
        x = self.conv3(self.relu2(self.bn2(self.conv2(x))))
        residual = self.ada(self.conv4(residual))
        if self.module_add:
            x = self.add(x, residual)
        else:
            x += residual
        x = self.avgpool(self.relu3(x))
        return self.fc(x.view(x.size(0), -1))


class QuantSimTinyModel(nn.Module):
    def __init__(self):
        super().__init__()
        self.conv1 = nn.Conv2d(3, 32, kernel_size=2, stride=2, padding=2, bias=False)
        self.bn1, self.relu1 = nn.BatchNorm2d(32), nn.ReLU(inplace=True)
        self.maxpool = nn.MaxPool2d(kernel_size=2, stride=2, padding=1)
        self.conv2 = nn.Conv2d(32, 16, kernel_size=2, stride=2, padding=2, bias=False)
        self.bn2, self.relu2 = nn.BatchNorm2d(16), nn.ReLU6(inplace=True)
        self.conv3 = nn.Conv2d(16, 8, kernel_size=2, stride=2, padding=2, bias=False)
        self.relu3, self.avgpool = nn.ReLU(inplace=True), nn.AvgPool2d(3, stride=1)
        self.conv4 = nn.Conv2d(8, 4, kernel_size=2, stride=2, padding=2, bias=True)
        self.fc = nn.Linear(36, 12)

    def forward(self, *inputs):
        x = self.maxpool(self.relu1(self.bn1(self.conv1(inputs[0]))))
        x = self.relu2(self.bn2(self.conv2(x)))
        x = self.conv4(self.avgpool(self.relu3(self.conv3(x))))
        return self.fc(x.view(x.size(0), -1))


def _config(ops=None, default_params=None, **sections):
    config = {"defaults": {"ops": ops or {}, "params": default_params or {}}, "params": {}, "op_type": {}, "supergroups": [],
              "model_input": {}, "model_output": {}}
    for key, value in sections.items():
        if key in ("per_channel_quantization", "strict_symmetric", "unsigned_symmetric"):
            config["defaults"][key] = value
        else:
            config[key] = value
    return config


def _sim(model, config, dummy_input=None, in_place=False):
    dummy_input = torch.rand(1, 3, 32, 32).cuda() if dummy_input is None else dummy_input
    return QuantizationSimModel(model.cuda().eval(), quant_scheme=QuantScheme.post_training_tf_enhanced,
                                config_file=config, dummy_input=dummy_input, in_place=in_place)


def _wrappers(sim):
    return [(n, m) for n, m in sim.model.named_modules() if isinstance(m, QcQuantizeWrapper)]


def test_parse_config_file_defaults():              # :83-139
    sim = _sim(SingleResidual(), _config({"is_output_quantized": "True", "is_symmetric": "False"},
                                         {"is_quantized": "False", "is_symmetric": "True"},
                                         per_channel_quantization="True"), in_place=True)
    for name, module in _wrappers(sim):
        # the functional add's result is quantized at the input of relu3
        assert module.input_quantizers[0].enabled == (name == 'relu3')
        # conv1 and conv2 hand their output quantizer to the batch norm that follows
        assert module.output_quantizers[0].enabled == (name not in ["conv1", "conv2"])
        for q in list(module.input_quantizers) + list(module.output_quantizers):
            assert not q.use_symmetric_encodings and not q.use_strict_symmetric and not q.use_unsigned_symmetric
        for q in module.param_quantizers.values():
            assert not q.enabled
            assert q.use_symmetric_encodings and not q.use_strict_symmetric and not q.use_unsigned_symmetric
            assert len(q._cppOp) > 1


def test_parse_config_file_params():                # :141-185
    sim = _sim(SingleResidual(), _config({"is_output_quantized": "True", "is_symmetric": "False"},
                                         {"is_quantized": "False", "is_symmetric": "True"},
                                         params={"weight": {"is_quantized": "True", "is_symmetric": "False"}}))
    for _, module in _wrappers(sim):
        for param_name, q in module.param_quantizers.items():
            if param_name == 'weight':
                assert q.enabled == (module not in (sim.model.bn1, sim.model.bn2))
                assert not q.use_symmetric_encodings
            else:
                assert not q.enabled
                assert q.use_symmetric_encodings


def test_parse_config_file_op_type():               # :273-340
    op_type = {"Conv": {"is_input_quantized": "True", "is_symmetric": "False",
                        "params": {"bias": {"is_quantized": "True", "is_symmetric": "False"}}}}
    sim = _sim(SingleResidual(), _config({"is_output_quantized": "True", "is_symmetric": "False"},
                                         {"is_quantized": "False", "is_symmetric": "True"}, op_type=op_type))
    for name, module in _wrappers(sim):
        is_conv = isinstance(module._module_to_wrap, nn.Conv2d)
        if is_conv:
            assert module.input_quantizers[0].enabled
            assert module.output_quantizers[0].enabled == (name not in ["conv1", "conv2"])
        else:
            assert module.input_quantizers[0].enabled == (name == 'relu3')
            assert module.output_quantizers[0].enabled
        assert not module.input_quantizers[0].use_symmetric_encodings
        assert not module.output_quantizers[0].use_symmetric_encodings
        for param_name, q in module.param_quantizers.items():
            if is_conv and param_name == 'bias':
                assert q.enabled and not q.use_symmetric_encodings
            else:
                assert not q.enabled and q.use_symmetric_encodings


def test_parse_config_file_supergroups():           # :804-873
    supergroups = [{"op_list": ["Conv", "Relu"]}, {"op_list": ["Relu", "MaxPool"]},
                   {"op_list": ["Conv", "Relu", "AveragePool"]}, {"op_list": ["Conv", "Clip"]}]
    sim = _sim(QuantSimTinyModel(), _config({"is_output_quantized": "True", "is_symmetric": "False"},
                                            {"is_quantized": "False", "is_symmetric": "False"},
                                            supergroups=supergroups), in_place=True)
    # in -> [conv1->bn1->relu1->maxpool] -> [conv2->bn2->relu2] -> [conv3->relu3->avgpool] -> [conv4] -> [fc] -> out
    for _, module in _wrappers(sim):
        assert not module.input_quantizers[0].enabled
    enabled = {name: module.output_quantizers[0].enabled for name, module in _wrappers(sim)}
    assert enabled == {"conv1": False, "bn1": False, "relu1": False, "maxpool": True,
                       "conv2": False, "bn2": False, "relu2": True,
                       "conv3": False, "relu3": False, "avgpool": True, "conv4": True, "fc": True}


def test_parse_config_file_elementwise_ops():       # :875-908
    sim = _sim(SingleResidual(), _config(op_type={"Add": {"is_input_quantized": "True"}}))
    for name, module in _wrappers(sim):
        # conv3 and ada make the operands of the add
        assert module.output_quantizers[0].enabled == (name in ['conv3', 'ada'])
        assert not module.input_quantizers[0].enabled


def test_parse_config_file_model_inputs():          # :910-968
    class MultiInputWithConstant(nn.Module):
        def __init__(self):
            super().__init__()
            self.conv1 = nn.Conv2d(3, 16, kernel_size=2, stride=2, padding=3, bias=False)
            self.conv2 = nn.Conv2d(16, 8, kernel_size=3, stride=2, padding=2)
            self.conv3 = nn.Conv2d(3, 8, kernel_size=3, stride=2, padding=2)
            self.add1, self.add2 = Add(), Add()

        def forward(self, *inputs):
            x = self.add1(self.conv2(self.conv1(inputs[0])), self.conv3(inputs[1]))
            return self.add2(x, torch.tensor(2.0, device=x.device))

    sim = _sim(MultiInputWithConstant(), _config(model_input={"is_input_quantized": "True"}),
               dummy_input=(torch.rand(1, 3, 32, 32).cuda(), torch.rand(1, 3, 20, 20).cuda()), in_place=True)
    for name, module in _wrappers(sim):
        if name in ('conv1', 'conv3'):
            assert module.input_quantizers[0].enabled
        elif name == 'add2':
            assert not module.input_quantizers[0].enabled
            assert module.input_quantizers[1].enabled
            assert module.input_quantizers[1].is_const
        else:
            assert not module.input_quantizers[0].enabled
        assert not module.output_quantizers[0].enabled
        assert not module.input_quantizers[0].use_symmetric_encodings
        assert not module.output_quantizers[0].use_symmetric_encodings


def test_parse_config_file_model_outputs():         # :970-1001
    sim = _sim(SingleResidual(), _config(model_output={"is_output_quantized": "True"}))
    for name, module in _wrappers(sim):
        assert module.output_quantizers[0].enabled == (name == 'fc')
        assert not module.input_quantizers[0].enabled


def test_supergroups_with_functional_add():         # :1003-1039
    sim = _sim(SingleResidual(), _config({"is_output_quantized": "True"}, supergroups=[{"op_list": ["Add", "Relu"]}]),
               in_place=True)
    # were the add not part of the supergroup, relu3's input quantizer would be enabled
    assert not sim.model.relu3.input_quantizers[0].enabled
    assert sim.model.relu3.output_quantizers[0].enabled


def test_supergroups_with_module_add():             # :1041-1078
    model = SingleResidual(module_add=True)
    sim = _sim(model, _config({"is_output_quantized": "True"}, supergroups=[{"op_list": ["Add", "Relu"]}]),
               in_place=True)
    for _, module in _wrappers(sim):
        assert module.output_quantizers[0].enabled == (module not in [model.add, model.conv1, model.conv2])
        assert not module.input_quantizers[0].enabled


def test_parse_config_file_symmetric_modes():       # :1080-1120
    sim = _sim(SingleResidual(), _config(None, {"is_symmetric": "True"}, per_channel_quantization="True",
                                         strict_symmetric="True",
                                         unsigned_symmetric="False"))
    for _, module in _wrappers(sim):
        for q in list(module.input_quantizers) + list(module.output_quantizers) + \
                list(module.param_quantizers.values()):
            assert q.use_strict_symmetric
            assert not q.use_unsigned_symmetric


def test_encoding_constraints():                    # :2129-2183
    """A range the configuration prescribes for an op type replaces what passes through the op's outputs: the quantizer
    switches to the min/max scheme and its encoding covers exactly that range."""
    import numpy as np
    config = {"defaults": {"ops": {"is_output_quantized": "True", "is_symmetric": "False"},
                           "params": {"is_quantized": "False", "is_symmetric": "True"}},
              "params": {}, "op_type": {"Softmax": {"encoding_constraints": {"min": -5.0, "max": 5.0}}},
              "supergroups": [], "model_input": {}, "model_output": {}}

    class SoftmaxModel(nn.Module):
        def __init__(self):
            super().__init__()
            self.softmax = nn.Softmax(dim=0)

        def forward(self, inp):
            return self.softmax(inp)

    x = torch.tensor([0.5, 0.5]).cuda()
    for config_file in (None, config):
        sim = QuantizationSimModel(SoftmaxModel().cuda(), x, quant_scheme=QuantScheme.post_training_tf_enhanced,
                                   config_file=config_file)
        sim.compute_encodings(lambda m, _: m(x), None)
        q = sim.model.softmax.output_quantizers[0]
        if config_file is None:
            assert q.quant_scheme == QuantScheme.post_training_tf_enhanced
            assert q.encoding.min == 0.0
            assert np.allclose(q.encoding.max, 0.5, atol=1e-2)
        else:
            assert q.quant_scheme == QuantScheme.post_training_tf
            assert q.encoding_min_max_fixed_vals == (-5.0, 5.0)
            assert np.allclose(q.encoding.min, -5.0, atol=1e-1)
            assert np.allclose(q.encoding.max, 5.0, atol=1e-1)
            # the grid is the 8-bit one over [-5, 5]: 0.5 lands on a multiple of its step
            y = sim.model(x)
            assert torch.allclose(y / q.encoding.delta, (y / q.encoding.delta).round(), atol=1e-3)
            # range learning keeps such a quantizer frozen (reference v1/quantsim.py:817-829)
            sim = QuantizationSimModel(SoftmaxModel().cuda(), x,
                                       quant_scheme=QuantScheme.training_range_learning_with_tf_init,
                                       config_file=config_file)
            sim.compute_encodings(lambda m, _: m(x), None)
            assert sim.model.softmax.output_quantizers[0].is_encoding_frozen
