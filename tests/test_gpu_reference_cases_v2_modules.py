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
