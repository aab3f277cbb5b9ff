"""The cases of the reference's own v2 quantizer-module tests (TrainingExtensions/torch/test/python/v2/quantization/
affine/test_affine_quantizer.py) on the GPU backend: compute_encodings semantics, forward / backward, initialisation
tracking, symmetric / asymmetric invariants under every optimizer, sub-float32 dtypes, grid attributes.

The reference's Quantize returns a QuantizedTensor; here it returns the integer-valued tensor itself, which is what
these cases compare."""
import math
import pickle

import pytest
import torch
from torch import nn
from torch.optim import SGD, Adagrad, Adam, AdamW, RMSprop

pytestmark = pytest.mark.gpu

_PARAMETER_SHAPE = (100,)


@pytest.fixture(scope="module")
def Q():
    from aimet_amd.v2.quantization import affine, encoding_analyzer

    class Api:
        pass
    a = Api()
    a.affine, a.Quantize, a.QuantizeDequantize = affine, affine.Quantize, affine.QuantizeDequantize
    a.MinMaxEncodingAnalyzer = encoding_analyzer.MinMaxEncodingAnalyzer
    return a


@pytest.fixture(autouse=True)
def set_seed():
    torch.manual_seed(0)


@pytest.fixture()
def x():
    # rows [-2, -1.01], [-1, -0.01], [0, 0.99], [1, 1.99] (:112-121)
    return (torch.arange(-200, 200).view(4, 100) / 100).cuda()


def _initialize(q, symmetric):
    # :64-81
    total_bins = 2 ** q.bitwidth - 1
    negative_bins, positive_bins = math.ceil(total_bins / 2), math.floor(total_bins / 2)
    mn = torch.full(_PARAMETER_SHAPE, -1.0)
    mx = torch.full(_PARAMETER_SHAPE, 1.0 * positive_bins / negative_bins)
    if not symmetric:
        mn, mx = mn + 1, mx + 1
    q.min = nn.Parameter(mn.cuda())
    q.max = nn.Parameter(mx.cuda())


def _make(Q, kind, symmetric, initialized, bitwidth=8):
    cls = Q.Quantize if kind == "q" else Q.QuantizeDequantize
    q = cls(shape=_PARAMETER_SHAPE, bitwidth=bitwidth, symmetric=symmetric,
            encoding_analyzer=Q.MinMaxEncodingAnalyzer(shape=_PARAMETER_SHAPE)).cuda()
    if initialized:
        _initialize(q, symmetric)
    return q


def _minmax_to_scaleoffset(mn, mx, symmetric, bitwidth):
    scale = (mx - mn) / (2 ** bitwidth - 1)
    offset = torch.zeros_like(scale) if symmetric else torch.round(mn / scale)
    return scale, offset


ALL4 = [(s, i) for s in (True, False) for i in (False, True)]


@pytest.mark.parametrize("kind", ["q", "qdq"])
@pytest.mark.parametrize("symmetric,initialized", ALL4)
def test_compute_encodings(Q, x, kind, symmetric, initialized):
    # :159-241: inside the context forward is dynamic quantization; on exit min / max are the batch's
    q = _make(Q, kind, symmetric, initialized)
    num_quant_bins = math.pow(2, q.bitwidth) - 1
    dynamic_min, dynamic_max = q.encoding_analyzer.compute_dynamic_encodings(x, num_quant_bins, q.symmetric)
    dynamic_scale, dynamic_offset = _minmax_to_scaleoffset(dynamic_min, dynamic_max, q.symmetric, bitwidth=8)
    fn = Q.affine.quantize if kind == "q" else Q.affine.quantize_dequantize
    expected = fn(x, dynamic_scale, dynamic_offset, q.qmin, q.qmax)
    with q.compute_encodings():
        out = q(x)
    assert torch.allclose(out, expected)
    assert torch.allclose(q.min, dynamic_min) and torch.allclose(q.max, dynamic_max)
    assert torch.allclose(q.get_scale(), dynamic_scale) and torch.allclose(q.get_offset(), dynamic_offset)


@pytest.mark.parametrize("kind", ["q", "qdq"])
@pytest.mark.parametrize("initialized", [False, True])
def test_compute_encodings_with_no_input(Q, kind, initialized):
    # :243-283
    q = _make(Q, kind, True, initialized)
    original_min, original_max = q.get_min(), q.get_max()
    if original_min is not None:
        original_min, original_max = original_min.clone().detach(), original_max.clone().detach()
    with q.compute_encodings():
        pass
    if original_min is None:
        assert q.get_min() is None and q.get_max() is None
    else:
        assert torch.equal(q.get_min(), original_min) and torch.equal(q.get_max(), original_max)


@pytest.mark.parametrize("kind", ["q", "qdq"])
@pytest.mark.parametrize("symmetric", [True, False])
def test_backward_during_compute_encodings(Q, x, kind, symmetric):
    # :286-313: min / max are not trainable inside the context
    q = _make(Q, kind, symmetric, True)
    x = x.clone().requires_grad_(True)
    with q.compute_encodings():
        output = q(x)
        output.backward(torch.zeros_like(output))
    assert q.min.grad is None and q.max.grad is None


@pytest.mark.parametrize("kind", ["q", "qdq"])
def test_compute_encodings_updates_parameters_upon_exit(Q, x, kind):
    # :316-352
    q = _make(Q, kind, True, False)
    getters = (q.get_min, q.get_max, q.get_scale, q.get_offset)
    assert all(g() is None for g in getters)
    with q.compute_encodings():
        assert all(g() is None for g in getters)
        _ = q(x)
        assert all(g() is None for g in getters)
    assert all(g() is not None for g in getters)


@pytest.mark.parametrize("kind", ["q", "qdq"])
@pytest.mark.parametrize("symmetric", [True, False])
def test_forward_and_backward(Q, x, kind, symmetric):
    # :355-432
    q = _make(Q, kind, symmetric, True)
    fn = Q.affine.quantize if kind == "q" else Q.affine.quantize_dequantize
    output = q(x)
    assert torch.allclose(output, fn(x, q.get_scale(), q.get_offset(), q.qmin, q.qmax))
    output.backward(torch.zeros_like(output))
    assert q.min.grad is not None and q.max.grad is not None


@pytest.mark.parametrize("kind", ["q", "qdq"])
@pytest.mark.parametrize("symmetric", [True, False])
def test_backward_with_no_grad(Q, x, kind, symmetric):
    # :435-461
    q = _make(Q, kind, symmetric, True)
    x = x.clone().requires_grad_(True)
    with torch.no_grad():
        output = q(x)
    output = output + x
    output.backward(torch.zeros_like(output))
    assert q.min.grad is None and q.max.grad is None


@pytest.mark.parametrize("kind", ["q", "qdq"])
def test_uninitialized_quantize(Q, x, kind):
    # :464-484
    q = _make(Q, kind, True, False)
    assert q.get_min() is None and q.get_max() is None and q.get_scale() is None and q.get_offset() is None
    with pytest.raises(RuntimeError):
        _ = q(x)


def _check_symmetric_invariants(q):
    # :487-527
    mn, mx, scale, offset = q.get_min(), q.get_max(), q.get_scale(), q.get_offset()
    total_bins = 2 ** q.bitwidth - 1
    positive_bins, negative_bins = math.floor(total_bins / 2), math.ceil(total_bins / 2)
    atol = scale.abs().max().item() * 1e-5
    assert torch.allclose(mn, -scale * negative_bins, rtol=1e-3, atol=atol)
    assert torch.allclose(mx, scale * positive_bins, rtol=1e-3, atol=atol)
    rng = torch.maximum(-mn * total_bins / negative_bins, mx * total_bins / positive_bins)
    assert torch.allclose(scale, rng / total_bins, rtol=1e-3, atol=atol)
    assert torch.equal(offset, torch.zeros_like(offset))
    assert not offset.requires_grad


def _check_asymmetric_invariants(q):
    # :530-561
    mn, mx, scale, offset = q.get_min(), q.get_max(), q.get_scale(), q.get_offset()
    bw = q.bitwidth
    assert torch.allclose(mn, scale * offset, rtol=1e-3, atol=mn.abs().max().item() * 1e-5)
    assert torch.allclose(mx, mn + scale * (2 ** bw - 1), rtol=1e-3, atol=mx.abs().max().item() * 1e-5)
    assert torch.allclose(scale, (mx - mn) / (2 ** bw - 1), rtol=1e-3, atol=scale.abs().max().item() * 1e-5)
    assert torch.equal(torch.round(mn / scale), offset)
    assert offset.requires_grad


@pytest.mark.parametrize("kind", ["q", "qdq"])
@pytest.mark.parametrize("symmetric", [True, False])
def test_invariants_after_compute_encodings(Q, x, kind, symmetric):
    # :564-576, 619-631
    q = _make(Q, kind, symmetric, False)
    with q.compute_encodings():
        _ = q(x)
    (_check_symmetric_invariants if symmetric else _check_asymmetric_invariants)(q)


@pytest.mark.parametrize("optim_cls", [SGD, RMSprop, Adagrad, Adam, AdamW])
@pytest.mark.parametrize("kind", ["q", "qdq"])
@pytest.mark.parametrize("symmetric", [True, False])
def test_invariants_while_learning(Q, x, kind, symmetric, optim_cls):
    # :579-668: ten optimizer steps at lr = 1 on random gradients
    q = _make(Q, kind, symmetric, True)
    original = [t.clone().detach() for t in (q.get_min(), q.get_max(), q.get_scale(), q.get_offset())]
    optimizer = optim_cls(q.parameters(), lr=1.0)
    for _ in range(10):
        output = q(x)
        output.backward(torch.randn_like(output))
        optimizer.step()
        (_check_symmetric_invariants if symmetric else _check_asymmetric_invariants)(q)
    assert not torch.equal(q.get_min(), original[0]) and not torch.equal(q.get_max(), original[1])
    assert not torch.equal(q.get_scale(), original[2])
    assert torch.equal(q.get_offset(), original[3]) == symmetric


def test_extreme_values_warning(Q):
    # :670-682
    extreme_val = torch.finfo(torch.float16).max
    dummy_input = torch.arange(start=0, end=extreme_val, dtype=torch.float16).cuda()
    qdq = Q.QuantizeDequantize((1,), 8, True, Q.MinMaxEncodingAnalyzer((1,))).cuda()
    with pytest.warns(UserWarning, match="Extreme values"):
        with qdq.compute_encodings():
            qdq(dummy_input)


def test_invalid_encoding_analyzer(Q):
    # :684-722
    dummy_input = torch.randn((30, 10, 11)).cuda()
    param_shape = (10, 11)
    with pytest.raises(RuntimeError):
        _ = Q.QuantizeDequantize(param_shape, 8, True, Q.MinMaxEncodingAnalyzer((12,)))
    for encoding_shape in ((10, 11), (11,), (10, 1), 11, 1):
        qdq = Q.QuantizeDequantize(param_shape, 8, True, Q.MinMaxEncodingAnalyzer(encoding_shape)).cuda()
        with qdq.compute_encodings():
            _ = qdq(dummy_input)
        assert qdq.is_initialized() and qdq.get_min().shape == param_shape


@torch.no_grad()
def test_is_initialized(Q):
    # :725-757
    def new():
        return Q.QuantizeDequantize((10,), bitwidth=8, symmetric=True,
                                    encoding_analyzer=Q.MinMaxEncodingAnalyzer((10,)))
    qdq = new()
    assert isinstance(qdq.min, nn.Parameter) and isinstance(qdq.max, nn.Parameter)
    assert not qdq.is_initialized()
    qdq.to(device="cuda", dtype=torch.float16)
    assert not qdq.is_initialized()                       # moving / casting initialises nothing
    qdq = new()
    qdq.min.copy_(torch.zeros(10))
    assert not qdq.is_initialized()                       # max still untouched
    qdq.max.add_(3)
    assert qdq.is_initialized()
    qdq = new()
    qdq.min = nn.Parameter(-torch.ones(10) * 2)
    assert not qdq.is_initialized()
    qdq.max = nn.Parameter(torch.ones(10) * 2)
    assert qdq.is_initialized()
    # the flag survives state_dict round trips and pickling, in both states
    fresh = new()
    fresh.load_state_dict(qdq.state_dict())
    assert fresh.is_initialized() and torch.equal(fresh.max, qdq.max)
    assert pickle.loads(pickle.dumps(qdq)).is_initialized()
    assert not pickle.loads(pickle.dumps(new())).is_initialized()
    other = new()
    other.load_state_dict(new().state_dict())
    assert not other.is_initialized()


@torch.no_grad()
@pytest.mark.parametrize("symmetric", [True, False])
def test_quantize_dequantize_then_quantize_and_dequantize_equality(Q, x, symmetric):
    # :923-936
    qdq, q = Q.QuantizeDequantize((), 8, symmetric).cuda(), Q.Quantize((), 8, symmetric).cuda()
    with qdq.compute_encodings(), q.compute_encodings():
        _ = qdq(x)
        _ = q(x)
    a = qdq(x)
    b = Q.affine.dequantize(q(x), q.get_scale(), q.get_offset())
    assert torch.equal(a, b)


@pytest.mark.parametrize("kind,symmetric", [("q", False), ("qdq", True)])
def test_allow_overwrite(Q, x, kind, symmetric):
    # :938-955
    q = (Q.Quantize if kind == "q" else Q.QuantizeDequantize)(_PARAMETER_SHAPE, 8, symmetric).cuda()
    with q.compute_encodings():
        q(x)
    q_min, q_max = q.min.detach().clone(), q.max.detach().clone()
    q.allow_overwrite(False)
    with q.compute_encodings():
        q(x * 10)
    assert torch.equal(q_min, q.min) and torch.equal(q_max, q.max)


def _grid(bitwidth, signed):
    qmin, qmax = (-2 ** (bitwidth - 1), 2 ** (bitwidth - 1) - 1) if signed else (0, 2 ** bitwidth - 1)
    return torch.arange(qmin, qmax + 1, dtype=torch.long)


FLOAT32_EPS = torch.tensor(torch.finfo(torch.float32).eps)
FLOAT32_TINY = torch.tensor(torch.finfo(torch.float32).tiny)


@pytest.mark.parametrize('tiny_scale', [FLOAT32_EPS, FLOAT32_TINY])
@pytest.mark.parametrize('dtype', [torch.float16, torch.bfloat16])
@pytest.mark.parametrize('symmetric', [True, False])
@pytest.mark.parametrize('bitwidth', [4, 8, 16])
def test_sub_float32_quantize_dequantize(Q, dtype, bitwidth, symmetric, tiny_scale):
    # :1214-1250: the scale never drops below float32 eps, and the result equals the float32 computation
    min_scale = FLOAT32_EPS.cuda()
    x_int = _grid(bitwidth, signed=symmetric)
    x = (x_int * tiny_scale).to(dtype).cuda()
    qtzr = Q.QuantizeDequantize((), bitwidth, symmetric).to(dtype).cuda()
    with qtzr.compute_encodings():
        _ = qtzr(x)
    assert torch.allclose(qtzr.get_scale(dtype=torch.float32), min_scale)
    assert torch.allclose(qtzr.get_offset(dtype=torch.float32), torch.zeros([], device="cuda"))
    out = qtzr(x)
    assert out.dtype == x.dtype and torch.all(out.isfinite())
    expected = Q.affine.quantize_dequantize(x.float(), min_scale, torch.zeros([], device="cuda"),
                                            qmin=int(x_int.min()), qmax=int(x_int.max())).to(dtype)
    assert torch.equal(out, expected)
    assert torch.allclose(out, x, atol=float(min_scale) / 2)


@pytest.mark.parametrize('dtype,bitwidth,symmetric', [(torch.float16, 13, True), (torch.float16, 12, False),
                                                      (torch.bfloat16, 10, True), (torch.bfloat16, 9, False)])
def test_sub_float32_error(Q, dtype, bitwidth, symmetric):
    # :1307-1325: the integer grid is not representable in the tensor's dtype
    x_int = _grid(bitwidth, signed=symmetric)
    x = (x_int.double() / x_int.max().double()).to(dtype).cuda()
    qtzr = Q.Quantize((), bitwidth, symmetric).to(dtype).cuda()
    with qtzr.compute_encodings():
        with pytest.raises(RuntimeError):
            _ = qtzr(x)


@pytest.mark.parametrize('qmin,qmax,bitwidth,symmetric', [(0, 15, 4, False), (-8, 7, 4, True)])
def test_qmin_qmax_consistency(Q, qmin, qmax, bitwidth, symmetric):
    # :1328-1363
    q = Q.Quantize((), qmin, qmax, symmetric).cuda()
    x = torch.arange(2 ** 16, dtype=torch.float).cuda()
    with q.compute_encodings():
        q(x)
    expected_qmin, expected_qmax, expected_bitwidth = qmin, qmax, bitwidth
    while q.bitwidth < 16:
        assert (q.qmin, q.qmax, q.bitwidth) == (expected_qmin, expected_qmax, expected_bitwidth)
        q.bitwidth += 1
        expected_qmin, expected_qmax, expected_bitwidth = expected_qmin * 2, (expected_qmax + 1) * 2 - 1, \
            expected_bitwidth + 1
    while q.bitwidth > 4:
        assert (q.qmin, q.qmax, q.bitwidth) == (expected_qmin, expected_qmax, expected_bitwidth)
        q.bitwidth -= 1
        expected_qmin, expected_qmax, expected_bitwidth = expected_qmin / 2, (expected_qmax + 1) / 2 - 1, \
            expected_bitwidth - 1
    q.signed = not q.signed
    assert q.bitwidth == 4 and (q.qmin == 0) == symmetric
    irregular = Q.Quantize((), -7, 7, True)
    with pytest.raises(RuntimeError):
        _ = irregular.bitwidth
    with pytest.raises(TypeError):
        q.bitwidth = 4.5
