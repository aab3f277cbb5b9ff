"""The v2 quantized modules as the reference's TrainingExtensions/torch/test/python/v2/nn/deprecated/test_linear.py and
test_activation.py use them: a quantized Linear / Softmax built directly or from a float module, quantizers placed by
hand into its input, output and parameter slots, and the output against the float operation with quantize-dequantize
applied by hand at those points -- equal to the bit.  (The cases of test_activation.py that pass QuantizedTensor
objects between modules belong to the reference's tensor subclasses, which are not part of the path.)"""
import pytest
import torch
import torch.nn.functional as F
from torch import nn

pytestmark = pytest.mark.gpu


@pytest.fixture
def x():
    return (torch.arange(-5, 5) / 10).cuda()


def _api():
    from aimet_amd.v2.nn import QuantizationMixin, QuantizedLinear
    from aimet_amd.v2.quantization.affine import QuantizeDequantize, quantize_dequantize
    from aimet_amd.v2.quantization.encoding_analyzer import MinMaxEncodingAnalyzer

    class Api:
        pass
    a = Api()
    a.QuantizationMixin, a.QuantizedLinear, a.quantize_dequantize = QuantizationMixin, QuantizedLinear, \
        quantize_dequantize
    a.activation = lambda: QuantizeDequantize((), bitwidth=8, symmetric=False,
                                              encoding_analyzer=MinMaxEncodingAnalyzer(())).cuda()
    a.weight = lambda: QuantizeDequantize((10, 1), bitwidth=4, symmetric=True,
                                          encoding_analyzer=MinMaxEncodingAnalyzer((10, 1))).cuda()
    return a


def _by_hand(a, tensor, quantizer, signed=False):
    return a.quantize_dequantize(tensor, quantizer.get_scale(), quantizer.get_offset(), quantizer.bitwidth,
                                 signed=signed)


def test_linear_without_quantizers(x):
    a = _api()
    layer = a.QuantizedLinear(10, 10).cuda()
    assert layer.input_quantizers[0] is None and layer.output_quantizers[0] is None
    assert layer.param_quantizers['weight'] is None and layer.param_quantizers['bias'] is None
    assert torch.equal(layer(x), F.linear(x, layer.weight, layer.bias))


def test_linear_input_quantizer(x):
    a = _api()
    layer = a.QuantizedLinear(10, 10).cuda()
    layer.input_quantizers[0] = a.activation()
    assert layer.param_quantizers['weight'] is None and layer.output_quantizers[0] is None
    with pytest.raises(RuntimeError):
        layer(x)                                                    # no encodings yet
    with layer.compute_encodings():
        layer(x)
    expected = F.linear(_by_hand(a, x, layer.input_quantizers[0]), layer.weight, layer.bias)
    assert torch.equal(layer(x), expected)


def test_linear_output_quantizer(x):
    a = _api()
    layer = a.QuantizedLinear(10, 10).cuda()
    layer.output_quantizers[0] = a.activation()
    assert layer.input_quantizers[0] is None and layer.param_quantizers['weight'] is None
    with pytest.raises(RuntimeError):
        layer(x)
    with layer.compute_encodings():
        layer(x)
    expected = _by_hand(a, F.linear(x, layer.weight, layer.bias), layer.output_quantizers[0])
    assert torch.equal(layer(x), expected)


@pytest.mark.parametrize("bias", [True, False])
def test_linear_weight_quantizer_needs_no_calibration(x, bias):
    a = _api()
    layer = a.QuantizedLinear(10, 10, bias=bias).cuda()
    layer.param_quantizers['weight'] = a.weight()
    assert layer.input_quantizers[0] is None and layer.output_quantizers[0] is None
    out = layer(x)                                                  # the weights are there: their range is taken now
    expected = F.linear(x, _by_hand(a, layer.weight, layer.param_quantizers['weight'], signed=True), layer.bias)
    assert torch.equal(out, expected)


def test_linear_from_module(x):
    a = _api()
    plain = nn.Linear(10, 10).cuda()
    layer = a.QuantizationMixin.from_module(plain)
    layer.input_quantizers[0], layer.output_quantizers[0] = a.activation(), a.activation()
    layer.param_quantizers['weight'] = a.weight()
    with layer.compute_encodings():
        layer(x)
    expected = F.linear(_by_hand(a, x, layer.input_quantizers[0]),
                        _by_hand(a, layer.weight, layer.param_quantizers['weight'], signed=True), layer.bias)
    expected = _by_hand(a, expected, layer.output_quantizers[0])
    assert torch.equal(layer(x), expected)
    # the two modules share their parameters' storage ...
    with torch.no_grad():
        plain.weight.add_(1)
    assert torch.equal(plain.weight, layer.weight)
    # ... (the quantized weight follows the edit: the kept copy is keyed on the parameter's version)
    expected = F.linear(_by_hand(a, x, layer.input_quantizers[0]),
                        _by_hand(a, layer.weight, layer.param_quantizers['weight'], signed=True), layer.bias)
    assert torch.equal(layer(x), _by_hand(a, expected, layer.output_quantizers[0]))
    # ... but not their attributes: a new parameter on one does not reach the other
    plain.weight = nn.Parameter(torch.zeros(10, 10).cuda())
    assert not torch.any(plain.weight == layer.weight)


def test_softmax_quantizers(x):
    a = _api()
    for slot in ("input", "output"):
        layer = a.QuantizationMixin.from_module(nn.Softmax(dim=-1))
        assert layer.input_quantizers[0] is None and layer.output_quantizers[0] is None
        assert torch.equal(layer(x), F.softmax(x, dim=-1))
        quantizers = layer.input_quantizers if slot == "input" else layer.output_quantizers
        quantizers[0] = a.activation()
        with pytest.raises(RuntimeError):
            layer(x)
        with layer.compute_encodings():
            layer(x)
        if slot == "input":
            expected = F.softmax(_by_hand(a, x, quantizers[0]), dim=-1)
        else:
            expected = _by_hand(a, F.softmax(x, dim=-1), quantizers[0])
        assert torch.equal(layer(x), expected)


def test_quantizers_taken_out_and_put_back(x):
    """After the reference's v2/nn/test_true_quant.py:567-636: under each `_remove_..._quantizers()` context the output
    is computed without those quantizers and they come back afterwards; called without `with`, they stay out."""
    a = _api()
    layer = a.QuantizedLinear(10, 10, bias=False).cuda()
    layer.input_quantizers[0], layer.output_quantizers[0] = q_in, q_out = a.activation(), a.activation()
    layer.param_quantizers['weight'] = q_w = a.weight()
    with layer.compute_encodings():
        layer(x)
    w = _by_hand(a, layer.weight, q_w, signed=True)
    with layer._remove_input_quantizers(0):
        assert layer.input_quantizers[0] is None
        assert torch.equal(layer(x), _by_hand(a, F.linear(x, w), q_out))
    assert layer.input_quantizers[0] is q_in
    with layer._remove_param_quantizers('weight'):
        assert layer.param_quantizers['weight'] is None
        assert torch.equal(layer(x), _by_hand(a, F.linear(_by_hand(a, x, q_in), layer.weight), q_out))
    assert layer.param_quantizers['weight'] is q_w
    with layer._remove_output_quantizers(0):
        assert layer.output_quantizers[0] is None
        assert torch.equal(layer(x), F.linear(_by_hand(a, x, q_in), w))
    assert layer.output_quantizers[0] is q_out
    with layer._remove_activation_quantizers():
        assert layer.input_quantizers[0] is None and layer.output_quantizers[0] is None
        assert torch.equal(layer(x), F.linear(x, w))
    assert layer.input_quantizers[0] is q_in and layer.output_quantizers[0] is q_out
    with layer._remove_all_quantizers():
        assert layer.param_quantizers['weight'] is None
        assert torch.equal(layer(x), F.linear(x, layer.weight))
    assert (layer.input_quantizers[0], layer.output_quantizers[0], layer.param_quantizers['weight']) == \
        (q_in, q_out, q_w)
    with pytest.raises(KeyError):
        layer._remove_param_quantizers('bias')                      # no such parameter: nothing is changed
    assert layer.param_quantizers['weight'] is q_w
    layer._remove_input_quantizers(0)
    layer._remove_param_quantizers('weight')
    layer._remove_output_quantizers(0)
    assert layer.input_quantizers[0] is None and layer.param_quantizers['weight'] is None
    assert layer.output_quantizers[0] is None


@pytest.mark.parametrize("which", ["input", "output", "param", "activation", "all"])
def test_quantizers_taken_out_of_a_whole_model(which):
    """After the reference's v2/test_utils_.py:229-353: the model-level helpers, as a context and for good."""
    from aimet_amd.v2 import utils
    from aimet_amd.v2.nn import BaseQuantizationMixin
    from aimet_amd.v2.quantsim import QuantizationSimModel
    torch.manual_seed(0)
    model = nn.Sequential(nn.Conv2d(8, 8, 3), nn.BatchNorm2d(8), nn.ReLU()).cuda().eval()
    dummy = torch.rand(1, 8, 16, 16).cuda()
    sim = QuantizationSimModel(model, dummy)
    sim.compute_encodings(lambda m, _: m(dummy), None)
    remove = getattr(utils, f"remove_{which}_quantizers")
    qmodules = [m for m in sim.model.modules() if isinstance(m, BaseQuantizationMixin)]
    before = [(list(m.input_quantizers), list(m.output_quantizers), dict(m.param_quantizers)) for m in qmodules]
    assert any(q is not None for ins, outs, params in before for q in ins + outs + list(params.values()))

    def gone():
        for m in qmodules:
            if which in ("input", "activation", "all"):
                assert all(q is None for q in m.input_quantizers)
            if which in ("output", "activation", "all"):
                assert all(q is None for q in m.output_quantizers)
            if which in ("param", "all"):
                assert all(q is None for q in m.param_quantizers.values())
    modules_before = list(sim.model.modules())
    quantized = sim.model(dummy)
    with remove(sim.model):
        gone()
        if which == "all":
            assert torch.equal(sim.model(dummy), model(dummy))
    assert list(sim.model.modules()) == modules_before
    now = [(list(m.input_quantizers), list(m.output_quantizers), dict(m.param_quantizers)) for m in qmodules]
    assert all(x is y for (a1, b1, c1), (a2, b2, c2) in zip(before, now)
               for x, y in zip(a1 + b1 + list(c1.values()), a2 + b2 + list(c2.values())))
    assert torch.equal(sim.model(dummy), quantized)
    remove(sim.model)
    gone()
