"""The v1 simulation model against the v2 simulation model on the same network, configuration, quant scheme and
calibration data, after the reference's TrainingExtensions/torch/test/python/v2/ab_test/test_quantsim_logits.py:
same configurations (:54-180), same models (the residual, tiny, softmax + pooling and two-input models of
models_/models_to_test.py), same criterion (:256-262) -- the v2 logits must keep at least 95 % of the v1 logits'
signal-to-quantization-noise ratio against the float model.

On this build both simulation models run their quantize-dequantize and calibration in different HIP kernels (the
DlQuantization arithmetic with its 512-bucket histograms for v1, the torch arithmetic with the 2048-bin observer for
v2), so the comparison crosses the two halves of the library.
"""
import pytest
import torch
from torch import nn

from test_gpu_reference_cases_quantsim_config import QuantSimTinyModel, SingleResidual

pytestmark = pytest.mark.gpu

_OPS = {"is_output_quantized": "True", "is_symmetric": "False"}


def _config(params_default, per_channel=None, params=None, op_type=None, supergroups=None):
    defaults = {"ops": dict(_OPS), "params": params_default}
    if per_channel is not None:
        defaults["per_channel_quantization"] = per_channel
    return {"defaults": defaults, "params": params or {}, "op_type": op_type or {}, "supergroups": supergroups or [],
            "model_input": {}, "model_output": {}}


_NO_PARAMS = {"is_quantized": "False", "is_symmetric": "True"}
CONFIG_DEFAULT = _config(_NO_PARAMS, per_channel="True")
CONFIG_PARAM_QUANT = _config(_NO_PARAMS, params={"weight": {"is_quantized": "True", "is_symmetric": "False"}})
CONFIG_OP_SPECIFIC_QUANT = _config(_NO_PARAMS, op_type={"Conv": {
    "is_input_quantized": "True", "is_symmetric": "False",
    "params": {"bias": {"is_quantized": "True", "is_symmetric": "False"}}}})
CONFIG_OP_SPECIFIC_QUANT_PER_CHANNEL = _config({"is_quantized": "True", "is_symmetric": "True"}, per_channel="True",
                                               params={"bias": {"is_quantized": "False"}},
                                               op_type={"Conv": {"per_channel_quantization": "True"}})
CONFIG_SUPERGROUP = _config({"is_quantized": "False", "is_symmetric": "False"}, supergroups=[
    {"op_list": ["Conv", "Relu"]}, {"op_list": ["Relu", "MaxPool"]}, {"op_list": ["Conv", "Relu", "AveragePool"]},
    {"op_list": ["Conv", "Clip"]}])


class SoftMaxAvgPoolModel(nn.Module):
    def __init__(self):
        super().__init__()
        self.sfmax, self.avgpool = nn.Softmax(dim=1), nn.AvgPool2d(3)

    def forward(self, inp):
        return self.avgpool(self.sfmax(inp))


class MultiInput(nn.Module):
    def __init__(self, num_classes=3):
        super().__init__()
        self.conv1 = nn.Conv2d(3, 16, kernel_size=2, stride=2, padding=3, bias=False)
        self.conv2 = nn.Conv2d(16, 8, kernel_size=3, stride=2, padding=2)
        self.conv3 = nn.Conv2d(3, 8, kernel_size=3, stride=2, padding=2)
        self.bn1, self.relu1 = nn.BatchNorm2d(8), nn.ReLU(inplace=True)
        self.maxpool = nn.MaxPool2d(kernel_size=2, stride=2, padding=1)
        self.fc = nn.Linear(288, num_classes)

    def forward(self, *inputs):
        x = self.conv2(self.conv1(inputs[0])) + self.conv3(inputs[1])
        x = self.maxpool(self.relu1(self.bn1(x)))
        return self.fc(x.view(x.size(0), -1))


def _sqnr(float_out, noisy):
    noise = float_out - noisy
    return float(float_out.square().mean() / (noise.square().mean() + 0.0001))


@torch.no_grad()
def _check(config, quant_scheme, model, dummy_input):
    from aimet_amd.v1.quantsim import QuantizationSimModel as V1Sim
    from aimet_amd.v2.quantsim import QuantizationSimModel as V2Sim
    model = model.cuda().eval()
    inputs = tuple(t.cuda() for t in (dummy_input if isinstance(dummy_input, tuple) else (dummy_input,)))
    logits = []
    for sim_cls in (V1Sim, V2Sim):
        sim = sim_cls(model, inputs if len(inputs) > 1 else inputs[0], quant_scheme, default_param_bw=8,
                      default_output_bw=16, config_file=config)
        sim.set_percentile_value(99)
        sim.compute_encodings(lambda m, _: m(*inputs), None)
        logits.append(sim.model(*inputs))
    float_logits = model(*inputs)
    v1_sqnr, v2_sqnr = _sqnr(float_logits, logits[0]), _sqnr(float_logits, logits[1])
    assert v1_sqnr * 0.95 < v2_sqnr, (v1_sqnr, v2_sqnr)
    return v1_sqnr, v2_sqnr


_SCHEMES = ("tf", "training_range_learning_with_tf_init", "percentile", "tf_enhanced")


def _scheme(name):
    from aimet_amd.common.defs import QuantScheme
    return {"tf": QuantScheme.post_training_tf,
            "training_range_learning_with_tf_init": QuantScheme.training_range_learning_with_tf_init,
            "percentile": QuantScheme.post_training_percentile,
            "tf_enhanced": QuantScheme.post_training_tf_enhanced}[name]


@pytest.mark.parametrize("quant_scheme", _SCHEMES)
@pytest.mark.parametrize("seed", range(3))
class TestLogits:
    @pytest.mark.parametrize("model_cls,input_shape", [(SingleResidual, (10, 3, 32, 32)),
                                                       (SoftMaxAvgPoolModel, (10, 4, 64, 128)),
                                                       (QuantSimTinyModel, (10, 3, 32, 32))])
    def test_default_config(self, model_cls, input_shape, quant_scheme, seed):
        torch.manual_seed(seed)
        _check(CONFIG_DEFAULT, _scheme(quant_scheme), model_cls(), torch.randn(input_shape))

    @pytest.mark.parametrize("model_cls", [SingleResidual, QuantSimTinyModel])
    def test_param_quant(self, model_cls, quant_scheme, seed):
        torch.manual_seed(seed)
        _check(CONFIG_PARAM_QUANT, _scheme(quant_scheme), model_cls(), torch.randn(10, 3, 32, 32))

    @pytest.mark.parametrize("model_cls", [SingleResidual, QuantSimTinyModel])
    def test_op_specific_quant(self, model_cls, quant_scheme, seed):
        torch.manual_seed(seed)
        model, x = model_cls(), torch.randn(10, 3, 32, 32)
        _check(CONFIG_OP_SPECIFIC_QUANT, _scheme(quant_scheme), model, x)
        _check(CONFIG_OP_SPECIFIC_QUANT_PER_CHANNEL, _scheme(quant_scheme), model, x)

    def test_supergroup(self, quant_scheme, seed):
        torch.manual_seed(seed)
        _check(CONFIG_SUPERGROUP, _scheme(quant_scheme), QuantSimTinyModel(), torch.randn(10, 3, 32, 32))

    def test_multi_input(self, quant_scheme, seed):
        torch.manual_seed(seed)
        _check(CONFIG_DEFAULT, _scheme(quant_scheme), MultiInput(),
               (torch.rand(10, 3, 32, 32), torch.rand(10, 3, 20, 20)))
