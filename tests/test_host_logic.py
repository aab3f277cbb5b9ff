"""Host-side logic that needs no GPU: configuration of the simulation model, graph helpers of the AdaRound flow,
argument handling of the v2 quantizers, the backend registry, and the failure behaviour of the loader."""
import importlib
import json
import math
import os

import pytest
import torch
from torch import nn


class _Net(nn.Module):
    def __init__(self):
        super().__init__()
        self.conv1 = nn.Conv2d(3, 4, 3, padding=1)
        self.relu1 = nn.ReLU(inplace=True)
        self.conv2 = nn.Conv2d(4, 4, 3, padding=1)
        self.bn = nn.BatchNorm2d(4)
        self.drop = nn.Dropout(0.1)
        self.flatten = nn.Flatten()
        self.fc = nn.Linear(4 * 4 * 4, 5)
        self.act = nn.ReLU()

    def forward(self, x):
        x = self.relu1(self.conv1(x))
        x = self.drop(self.bn(self.conv2(x)))
        return self.act(self.fc(self.flatten(x)))


def test_quantsim_default_configuration():
    """Which quantizers the default configuration switches on (reference default_config.json semantics: outputs
    quantized, parameters symmetric, bias off, Conv+Relu / Gemm+Relu supergroups, model input quantized)."""
    from aimet_amd.v1.quantsim import QuantizationSimModel
    from aimet_amd.v1.qc_quantize_op import QcQuantizeOpMode, StaticGridQuantWrapper
    model = _Net().eval()
    sim = QuantizationSimModel(model, dummy_input=torch.randn(1, 3, 4, 4), default_param_bw=4, default_output_bw=16)
    w = dict(sim.quant_wrappers())
    assert list(w) == ["conv1", "relu1", "conv2", "bn", "drop", "flatten", "fc", "act"]
    assert all(isinstance(x, StaticGridQuantWrapper) for x in w.values())
    assert w["conv1"].input_quantizers[0].enabled and not w["conv2"].input_quantizers[0].enabled
    assert not w["conv1"].output_quantizers[0].enabled and w["relu1"].output_quantizers[0].enabled   # Conv+Relu
    # conv2 hands its output quantizer to the batch norm that can be folded into it
    assert not w["conv2"].output_quantizers[0].enabled and w["bn"].output_quantizers[0].enabled
    assert not w["bn"].input_quantizers[0].enabled
    assert not w["fc"].output_quantizers[0].enabled and w["act"].output_quantizers[0].enabled        # Gemm+Relu
    assert not w["drop"].output_quantizers[0].enabled and not w["flatten"].output_quantizers[0].enabled
    assert w["conv1"].param_quantizers["weight"].enabled and not w["conv1"].param_quantizers["bias"].enabled
    assert not any(q.enabled for q in w["bn"].param_quantizers.values())
    assert w["conv1"].param_quantizers["weight"].bitwidth == 4 and w["relu1"].output_quantizers[0].bitwidth == 16
    assert w["conv1"].param_quantizers["weight"].use_symmetric_encodings
    assert not w["relu1"].output_quantizers[0].use_symmetric_encodings
    assert w["conv1"]._mode is QcQuantizeOpMode.ANALYSIS
    # the original model is untouched; exclusion and stripping of wrappers
    assert isinstance(model.conv1, nn.Conv2d)
    sim.exclude_layers_from_quantization([w["bn"]])
    assert isinstance(sim.model.bn, nn.BatchNorm2d)
    QuantizationSimModel.remove_quantization_wrappers(sim.model)
    assert not list(sim.quant_wrappers())
    with pytest.raises(ValueError):
        QuantizationSimModel(model, torch.randn(1, 3, 4, 4), default_param_bw=2)
    with pytest.raises(ValueError):
        QuantizationSimModel(model, torch.randn(1, 3, 4, 4), rounding_mode='up')


def test_quantsim_config_file(tmp_path):
    from aimet_amd.v1.quantsim import QuantizationSimModel
    from aimet_amd.v1.tensor_quantizer import StaticGridPerChannelQuantizer
    cfg = {"defaults": {"ops": {"is_output_quantized": "True", "is_symmetric": "True"},
                        "params": {"is_quantized": "True", "is_symmetric": "False"},
                        "strict_symmetric": "True", "per_channel_quantization": "True"},
           "params": {"bias": {"is_quantized": "False"}},
           "op_type": {"Relu": {"is_output_quantized": "False"}, "Conv": {"is_input_quantized": "True"}},
           "supergroups": [], "model_input": {}, "model_output": {"is_output_quantized": "True"}}
    path = os.path.join(str(tmp_path), "c.json")
    with open(path, "w") as f:
        json.dump(cfg, f)
    sim = QuantizationSimModel(_Net().eval(), torch.randn(1, 3, 4, 4), quant_scheme='tf', config_file=path)
    w = dict(sim.quant_wrappers())
    assert isinstance(w["conv1"].param_quantizers["weight"], StaticGridPerChannelQuantizer)
    assert len(w["conv1"].param_quantizers["weight"]._cppOp) == 4
    assert w["conv2"].input_quantizers[0].enabled and w["conv1"].output_quantizers[0].enabled
    assert not w["relu1"].output_quantizers[0].enabled
    assert w["act"].output_quantizers[0].enabled                        # model output overrides the op-type rule
    assert w["conv1"].output_quantizers[0].use_symmetric_encodings and w["conv1"].output_quantizers[0].use_strict_symmetric
    assert not w["conv1"].param_quantizers["weight"].use_symmetric_encodings


def test_graph_helpers():
    from aimet_amd import utils
    model = _Net().eval()
    x = torch.randn(2, 3, 4, 4)
    order = [n for n, _ in utils.get_ordered_list_of_modules(model, x)]
    assert order == ["conv1", "relu1", "conv2", "bn", "drop", "flatten", "fc", "act"]
    pairs = utils.get_module_act_func_pair(model, x)
    assert pairs[model.conv1] is model.relu1          # through the in-place ReLU
    assert pairs[model.conv2] is None and pairs[model.fc] is model.act
    assert utils.get_named_module(model, "fc") is model.fc
    loader = [(torch.randn(2, 3, 4, 4), torch.zeros(2)) for _ in range(3)]
    cached = utils.CachedDataset(loader, 2)
    assert len(cached) == 2 and cached[1][0] is loader[1][0]
    with pytest.raises(ValueError):
        utils.CachedDataset(loader, 4)
    inp, out = utils.ModuleData(model, model.conv2, lambda m, b: m(b[0])).collect_inp_out_data(loader[0], True, True)
    with torch.no_grad():
        want_in = model.relu1(model.conv1(loader[0][0]))
    assert torch.allclose(inp, want_in) and torch.allclose(out, model.conv2(want_in))


def test_adaround_parameters_and_schedule():
    from aimet_amd.v1.adaround.adaround_loss import AdaroundHyperParameters, AdaroundLoss
    from aimet_amd.v1.adaround.adaround_weight import AdaroundParameters
    with pytest.raises(ValueError):
        AdaroundParameters([1, 2], num_batches=3)
    p = AdaroundParameters([1, 2, 3], num_batches=2)
    assert (p.num_iterations, p.reg_param, p.beta_range, p.warm_start) == (None, 0.01, (20, 2), 0.2)
    # known answers of the reference's tests (test_adaround_loss.py:76-100)
    assert AdaroundLoss._compute_beta(10000, 8000, (20, 2), 0.2) == 4.636038969321072
    import numpy as np
    np.random.seed(0)
    alpha = torch.from_numpy(np.random.rand(1, 3, 12, 12))
    hp = AdaroundHyperParameters(10000, 0.01, (20, 2), 0.2)
    assert AdaroundLoss.compute_round_loss(alpha, hp, 10) == 0
    assert AdaroundLoss.compute_round_loss(alpha, hp, 8000).item() == pytest.approx(4.266156963161077, abs=1e-5)
    a, b = torch.rand(8, 3, 4, 4), torch.rand(8, 3, 4, 4)
    assert AdaroundLoss.compute_recon_loss(a, b).item() == pytest.approx(
        torch.nn.functional.mse_loss(a, b, reduction='none').sum(1).mean().item(), abs=1e-5)


def test_v2_quantizer_arguments_and_registry():
    from aimet_amd.v2.quantization.affine import QuantizeDequantize, backends
    from aimet_amd.v2.quantization.affine.backends import _derive_qmin_qmax
    assert _derive_qmin_qmax(bitwidth=8, signed=True) == (-128, 127)
    assert _derive_qmin_qmax(bitwidth=4, signed=False) == (0, 15)
    assert _derive_qmin_qmax(num_steps=254, signed=True) == (-127, 127)
    q = QuantizeDequantize((4, 1), 8, True)
    assert (q.qmin, q.qmax, q.symmetric, q.bitwidth, q.signed) == (-128, 127, True, 8, True)
    q = QuantizeDequantize((), qmin=0, qmax=15, symmetric=False)
    assert q.bitwidth == 4 and not q.signed and not q.is_initialized()
    with pytest.raises(ValueError):
        QuantizeDequantize((), qmin=5, qmax=5, symmetric=False)
    with pytest.raises(TypeError):
        QuantizeDequantize((), 8)
    with pytest.raises(RuntimeError):
        q(torch.randn(3))                                   # not initialised
    q.set_range(torch.tensor(-1.0), torch.tensor(2.0))
    assert q.is_initialized() and q.get_scale().item() == pytest.approx(3 / 15)
    assert q.get_offset().item() == round(-1.0 / (3 / 15))
    with pytest.raises(RuntimeError):
        q(torch.randn(3))                                   # CPU tensor: the backend computes on the GPU only
    with pytest.raises(RuntimeError):
        backends.set_global_backend("nope")
    with pytest.raises(RuntimeError):
        backends.add_backend("hip_gfx950", object())
    enc = q.get_legacy_encodings()
    assert enc[0]["bitwidth"] == 4 and enc[0]["is_symmetric"] == "False"


def test_v2_minmax_analyzer_formulas():
    """MinMaxEncodingAnalyzer.compute_encodings_from_stats on CPU statistics (pure tensor arithmetic): the cases of
    the reference's test_encoding_analyzer.py for min-max (zero included, symmetric grid, degenerate range)."""
    from aimet_amd.v2.quantization.encoding_analyzer import MinMaxEncodingAnalyzer, _MinMaxRange
    from aimet_amd.v2.utils import StatisticsNotFoundError
    an = MinMaxEncodingAnalyzer((1,))
    mn, mx = an.compute_encodings_from_stats(_MinMaxRange(torch.tensor([2.0]), torch.tensor([5.0])), 255, False)
    assert mn.item() == 0 and mx.item() == 5
    mn, mx = an.compute_encodings_from_stats(_MinMaxRange(torch.tensor([-3.0]), torch.tensor([5.0])), 255, True)
    delta = max(5 / 127, 3 / 128)
    assert mn.item() == pytest.approx(-128 * delta) and mx.item() == pytest.approx(127 * delta)
    mn, mx = an.compute_encodings_from_stats(_MinMaxRange(torch.tensor([0.0]), torch.tensor([0.0])), 255, False)
    assert mn.item() == 0 and mx.item() == pytest.approx(255 * torch.finfo(torch.float32).eps)
    with pytest.raises(StatisticsNotFoundError):
        an.compute_encodings(255, False)
    with pytest.raises(ValueError):
        an.compute_encodings_from_stats(_MinMaxRange(torch.tensor([0.0]), torch.tensor([1.0])), 0, False)


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    """There is no CPU fallback: without libmiq.so the package's loader raises ImportError."""
    import aimet_amd._lib as lib_mod
    monkeypatch.setattr(lib_mod, "LIB_PATH", os.path.join(str(tmp_path), "libmiq.so"))
    with pytest.raises(ImportError, match="no CPU fallback"):
        lib_mod._load()


def test_cpu_tensors_are_rejected_everywhere():
    from aimet_amd import ops
    x = torch.randn(16)
    for call in (lambda: ops.qdq_per_tensor(x, -1.0, 1.0, 8), lambda: ops.minmax(x),
                 lambda: ops.v2_qdq(x, 1, 16, torch.ones(1), torch.zeros(1), 0, 255),
                 lambda: ops.adaround_init_alpha(x, 1, 16, torch.ones(1)),
                 lambda: ops.Analyzer(1, torch.device("cpu")).update_stats(x)):
        with pytest.raises((RuntimeError, AssertionError)):
            call()


# ---------------------------------------------------------------------------------- v2 channel layouts and blocks
@pytest.mark.parametrize("shape,param_shape,copies", [
    ((6, 5, 4), (), False), ((6, 5, 4), (6, 1, 1), False), ((6, 5, 4), (5, 1), False), ((6, 5, 4), (4,), False),
    ((6, 5, 4), (6, 5, 1), False), ((6, 5, 4), (6, 1, 4), True), ((2, 6, 1, 4), (6, 1, 4), False),
    ((4, 1, 3, 2), (4, 1, 3, 1), False),          # Linear weight [4, 6] split into blocks of 2 along the input axis
    ((2, 2, 3, 2), (2, 1, 3, 1), True),           # blocks along both axes
])
def test_channel_view_groups_elements_by_parameter(shape, param_shape, copies):
    from aimet_amd.v2.utils import channel_view, channel_view_restore
    n_param = int(math.prod(param_shape))
    which = torch.arange(n_param, dtype=torch.float32).reshape(param_shape).expand(shape)
    values = torch.arange(math.prod(shape), dtype=torch.float32).reshape(shape)
    t3, perm = channel_view(which, param_shape)
    v3, perm_v = channel_view(values, param_shape)
    assert (perm is not None) == copies and perm == perm_v
    assert t3.dim() == 3 and t3.shape[1] == n_param
    # every run of channel c holds elements that broadcast against parameter element c
    assert torch.equal(t3, torch.arange(n_param, dtype=torch.float32).view(1, -1, 1).expand_as(t3))
    assert torch.equal(channel_view_restore(v3, shape, perm), values)
    if not copies:
        # no copy: the flat order is untouched, which is what the kernels' (i / run) % channels indexing assumes
        assert torch.equal(v3.reshape(-1), values.reshape(-1))


def test_block_reshape_helpers_follow_the_reference_shapes():
    # test_backend.py:627-639 of the reference
    from aimet_amd.v2.utils import get_encoding_shape_with_blocks, reshape_tensor_for_blocks
    inp = torch.randn(8, 6, 8, 3)
    assert reshape_tensor_for_blocks(inp, (4, 3, 8, 1), [-1, 2, 1, 3]).shape == (4, 2, 3, 2, 8, 1, 1, 3)
    assert get_encoding_shape_with_blocks((4, 3, 8, 1), [-1, 2, 1, 3]) == (4, 1, 3, 1, 8, 1, 1, 1)
    assert reshape_tensor_for_blocks(inp, (4, 3, 8, 1), None) is inp
    assert get_encoding_shape_with_blocks((4, 3), None) == (4, 3)
    # leading axes beyond the block specification stay as they are
    assert reshape_tensor_for_blocks(torch.randn(3, 5, 4, 6), (2, 3), [2, 2]).shape == (3, 5, 2, 2, 3, 2)


def test_affine_call_forms():
    # reference backends/__init__.py:334-356
    from aimet_amd.v2.quantization.affine.backends import _parse_args
    assert _parse_args((8,), {}) == (0, 255, None)
    assert _parse_args((8, True), {}) == (-128, 127, None)
    assert _parse_args((4, True, (1, 2)), {}) == (-8, 7, (1, 2))
    assert _parse_args((-7, 7), {"block_size": [2, 1]}) == (-7, 7, [2, 1])
    assert _parse_args((), {"num_steps": 254, "signed": True}) == (-127, 127, None)
    assert _parse_args((), {"qmin": 0, "qmax": 15}) == (0, 15, None)


# ------------------------------------------------------------------------------ v1 range learning, host-side logic
def _learned_wrapper(module=None, **kw):
    from aimet_amd.common import libpymo
    from aimet_amd.common.defs import QuantScheme
    from aimet_amd.v1.qc_quantize_op import LearnedGridQuantWrapper
    return LearnedGridQuantWrapper(module or nn.Conv2d(1, 32, 5), round_mode=libpymo.RoundingMode.ROUND_NEAREST,
                                   quant_scheme=QuantScheme.training_range_learning_with_tf_init,
                                   is_output_quantized=True, activation_bw=kw.get("activation_bw", 8), weight_bw=8,
                                   device='cpu')


def test_learned_grid_set_and_freeze_encoding():
    # test_tensor_quantizer.py:224-258 of the reference
    from aimet_amd.common import libpymo
    w = _learned_wrapper()
    enc_old = libpymo.TfEncoding(-1, 0.5, 1, 0.2, 8)
    enc_new = libpymo.TfEncoding(-0.98, 0.4, 1, 0.2, 8)
    w.output_quantizers[0].encoding = enc_old
    w.output_quantizers[0].freeze_encoding()
    assert w.output_quantizers[0].encoding.min == pytest.approx(enc_old.min, abs=1e-6)
    assert not w.output0_encoding_min.requires_grad and not w.output0_encoding_max.requires_grad
    with pytest.raises(RuntimeError):
        w.output_quantizers[0].encoding = enc_new
    assert w.output_quantizers[0].encoding.min == pytest.approx(enc_old.min, abs=1e-6)
    with pytest.raises(RuntimeError):
        w.input_quantizers[0].freeze_encoding()              # never initialised
    # names of the learnable parameters
    names = {n for n, _ in w.named_parameters()}
    assert {'output0_encoding_min', 'output0_encoding_max', '_module_to_wrap.weight', '_module_to_wrap.bias'} <= names


def test_learned_grid_n_and_p_and_bitwidth_check():
    # test_tensor_quantizer.py:320-352
    from aimet_amd.common import libpymo
    from aimet_amd.common.defs import QuantizationDataType, QuantScheme
    from aimet_amd.v1.tensor_quantizer import LearnedGridTensorQuantizer
    q = LearnedGridTensorQuantizer(bitwidth=8, round_mode=libpymo.RoundingMode.ROUND_NEAREST,
                                   quant_scheme=QuantScheme.training_range_learning, use_symmetric_encodings=True,
                                   enabled_by_default=True, data_type=QuantizationDataType.int)
    assert q.n() == 0.0 and q.p() == 255.0
    q.bitwidth = 16
    assert q.n() == 0.0 and q.p() == 65535.0
    q.use_strict_symmetric = True
    assert q.n() == 0.0 and q.p() == 65534.0
    q.bitwidth = 8
    with pytest.raises(RuntimeError):
        q.encoding = libpymo.TfEncoding(-0.98, 0.4, 1, 0.2, 4)
    with pytest.raises(ValueError):
        LearnedGridTensorQuantizer(8, libpymo.RoundingMode.ROUND_NEAREST, QuantScheme.training_range_learning, True,
                                   True, QuantizationDataType.float)


def test_learned_grid_encoding_getter_and_effective_encoding():
    # test_tensor_quantizer.py:403-421: asymmetric 16-bit
    from aimet_amd.common import libpymo
    w = _learned_wrapper(nn.Conv2d(1, 1, 1), activation_bw=16)
    w.output_quantizers[0].enabled = True
    w.output_quantizers[0].encoding = libpymo.TfEncoding(-0.98, 0.4, 0, 0, 16)
    e = w.output_quantizers[0].encoding
    assert e.max == pytest.approx(0.4, rel=1e-3) and e.min == pytest.approx(-0.98, rel=1e-3)
    assert e.delta == pytest.approx((e.max - e.min) / (2 ** e.bw - 1), rel=1e-3)
    assert e.offset == pytest.approx(e.min / e.delta, rel=1e-3)
    # signed symmetric, not strict: learned with max == -min, reported with min one step lower
    q = w.param_quantizers['weight']
    q.use_symmetric_encodings = True
    q.encoding = libpymo.TfEncoding(-1.27, 1.27, 0.01, -128, 8)
    inner, shown = q.encoding, q.get_effective_encoding()
    assert inner.min == pytest.approx(-1.27) and inner.delta == pytest.approx(0.01) and inner.offset == -128
    assert shown.min == pytest.approx(-1.28) and shown.max == pytest.approx(1.27)


def test_get_computed_encodings_follows_the_cpp_rules():
    # quantsim_straight_through_grad.py:121-162 of the reference; cross-checked with the oracle's fillEncodingInfo
    import oracle
    from aimet_amd.v1.quantsim_straight_through_grad import get_computed_encodings
    emin, emax = torch.tensor([-1.0, -0.3, 0.0]), torch.tensor([0.5, 2.0, 4.0])
    delta, offset, steps = get_computed_encodings(8, emin, emax, False, False, False)
    assert steps.tolist() == [255.0] * 3
    for i in range(3):
        e = oracle.lib.tf_compute_encoding(float(emin[i]), float(emax[i]), 8)
        assert delta[i].item() == pytest.approx(e.delta, rel=1e-6) and offset[i].item() == e.offset
    delta, offset, steps = get_computed_encodings(8, -emax, emax, True, False, False)
    assert torch.allclose(delta, emax / 127) and offset.tolist() == [-128.0] * 3 and steps[0] == 255
    delta, offset, steps = get_computed_encodings(8, -emax, emax, True, True, False)
    assert torch.allclose(delta, emax / 127) and offset.tolist() == [-127.0] * 3 and steps[0] == 254


def test_gating_keeps_learned_ranges_ordered():
    from aimet_amd.v1.tensor_quantizer import set_encoding_min_max_gating_threshold
    mn = nn.Parameter(torch.tensor([0.3, -1.0, -1e-7]))
    mx = nn.Parameter(torch.tensor([0.5, -0.2, 0.0]))
    set_encoding_min_max_gating_threshold(mn, mx)
    assert mn.tolist() == pytest.approx([0.0, -1.0, -1e-7]) and mx.tolist() == pytest.approx([0.5, 0.0, 1e-5 - 1e-7])


def test_per_channel_fused_statistics_go_with_the_scheme():
    """The per-channel quantizer keeps TF statistics outside its analyzer objects (one fused min/max pass).  A change of
    scheme or fixed min/max values re-instantiates the analyzers (reference tensor_quantizer.py:222-247) and must
    drop those statistics with them; reset does the same."""
    from aimet_amd.common import libpymo
    from aimet_amd.common.defs import QuantScheme
    from aimet_amd.v1.tensor_quantizer import StaticGridPerChannelQuantizer
    q = StaticGridPerChannelQuantizer(8, libpymo.RoundingMode.ROUND_NEAREST, QuantScheme.post_training_tf,
                                      use_symmetric_encodings=True, num_channels=4, enabled_by_default=True)
    stale = torch.tensor([[-1.0] * 4, [1.0] * 4])
    q._tf_minmax = stale                                    # pylint: disable=protected-access
    q.quant_scheme = QuantScheme.post_training_tf_enhanced
    assert q._tf_minmax is None                             # pylint: disable=protected-access
    q.quant_scheme = QuantScheme.post_training_tf
    q._tf_minmax = stale                                    # pylint: disable=protected-access
    q.encoding_min_max_fixed_vals = (-0.5, 0.5)
    assert q._tf_minmax is None and q.quant_scheme == QuantScheme.post_training_tf  # pylint: disable=protected-access
    q._tf_minmax = stale                                    # pylint: disable=protected-access
    q.reset_encoding_stats()
    assert q._tf_minmax is None                             # pylint: disable=protected-access


def test_encoding_list_built_on_first_read():
    """A quantizer whose encodings were computed on the device holds a builder until the list is read: asking whether
    an encoding exists, or for its stamp, does not run the builder; reading does, once; assigning drops it; pickling
    carries the list."""
    import pickle
    from aimet_amd.common import libpymo
    from aimet_amd.common.defs import QuantScheme
    from aimet_amd.v1.tensor_quantizer import StaticGridPerChannelQuantizer
    q = StaticGridPerChannelQuantizer(8, libpymo.RoundingMode.ROUND_NEAREST, QuantScheme.post_training_tf, True, 3,
                                      enabled_by_default=True)
    assert not q.has_encoding() and q.encoding is None
    built = []

    def builder():
        built.append(1)
        return [libpymo.TfEncoding(-1.0 - c, 1.0 + c, 0.01, -128, 8) for c in range(3)]
    q.__dict__['_pending_encoding'] = builder
    stamp = q.encoding_stamp()
    assert q.has_encoding() and stamp[0] == 'on device' and built == []
    enc = q.encoding
    assert built == [1] and len(enc) == 3 and q.encoding is enc and built == [1]
    assert q.encoding_stamp() != stamp and q.encoding_stamp()[0] == id(enc)
    serial = q.__dict__['_encoding_serial']
    q.encoding = enc[:2]
    assert q.__dict__['_encoding_serial'] == serial + 1 and len(q.encoding) == 2
    q.__dict__['_pending_encoding'] = builder
    clone = pickle.loads(pickle.dumps(q))
    assert [e.max for e in clone.encoding] == [1.0, 2.0, 3.0] and clone.__dict__.get('_pending_encoding') is None
    q.__dict__['_pending_encoding'] = builder
    q.encoding = None                                              # an assignment wins over what was pending
    assert not q.has_encoding() and q.encoding is None


def test_v2_range_warnings_one_by_one_and_batched():
    """The warnings about non-finite or extreme ranges (reference encoding_analyzer.py:388-395) are the same whether a
    quantizer checks its own range at once or many of them are examined together at the end."""
    import warnings
    from aimet_amd.v2.quantization.affine import quantizer as qz
    fine = (torch.tensor([-1.0, -2.0]), torch.tensor([1.0, 2.0]))
    nan = (torch.tensor([float('nan')]), torch.tensor([1.0]))
    huge = (torch.tensor([-1.0]), torch.tensor([torch.finfo(torch.float32).max * 0.97]))

    def messages(fn):
        with warnings.catch_warnings(record=True) as caught:
            warnings.simplefilter("always")
            fn()
        return sorted(str(w.message)[:8] for w in caught)

    assert messages(lambda: qz._flag_extreme_min_max(*fine)) == []
    assert messages(lambda: qz._flag_extreme_min_max(*nan)) == ['Infinite']
    assert messages(lambda: qz._flag_extreme_min_max(*huge)) == ['Extreme ']
    # torch's own formulation of the same two tests
    for mn, mx in (fine, nan, huge):
        extreme = torch.full_like(mn, torch.finfo(mn.dtype).max)
        want_extreme = bool(torch.any(torch.isclose(mn.abs(), extreme, rtol=0.05)) or
                            torch.any(torch.isclose(mx.abs(), extreme, rtol=0.05)))
        want_bad = not bool(torch.all(torch.isfinite(mn)) and torch.all(torch.isfinite(mx)))
        got = messages(lambda: qz._flag_extreme_min_max(mn, mx))
        assert ('Extreme ' in got) == want_extreme and ('Infinite' in got) == want_bad

    def batched():
        with qz.batched_range_checks():
            for pair in (fine, nan, fine, huge):
                qz._flag_extreme_min_max(*pair)
            assert qz._pending_range_checks and len(qz._pending_range_checks) == 4      # held back
    assert messages(batched) == ['Extreme ', 'Infinite']
    assert qz._pending_range_checks is None


def test_v2_grid_representability_is_memoised():
    from aimet_amd.v2.quantization.affine.backends import hip_gfx950 as backend
    backend._is_grid_representable.cache_clear()
    assert backend._is_grid_representable(torch.float32, -128, 127)
    assert backend._is_grid_representable(torch.float32, -128, 127)
    assert backend._is_grid_representable.cache_info().hits == 1
    assert not backend._is_grid_representable(torch.float16, 0, 2 ** 16 - 1)      # 65535 is not a float16
    assert backend._is_grid_representable(torch.bfloat16, -128, 127)
    assert not backend._is_grid_representable(torch.bfloat16, 0, 2 ** 9 - 1)       # 511 needs nine bits


def test_checkpointed_flow_helpers_on_plain_modules():
    """The helpers under apply_adaround_with_cache / checkpointed sequential MSE are tensor plumbing: what a block
    receives per batch (keyword inputs laid behind the positional ones, host copies when asked), a block's outputs
    handed on as the next block's inputs with and without the static inputs, and the cut of a model's layers into runs
    per named block."""
    from types import SimpleNamespace

    from aimet_amd import utils
    from aimet_amd.v1.adaround import activation_sampler as sampler

    class Scaled(nn.Module):
        def __init__(self):
            super().__init__()
            self.fc = nn.Linear(6, 6)

        def forward(self, x, scale=None, shift=1.0):
            return self.fc(x) * scale + shift, scale

    class Stack(nn.Module):
        def __init__(self):
            super().__init__()
            self.first, self.block_a, self.between, self.block_b = nn.Linear(6, 6), Scaled(), nn.Linear(6, 6), Scaled()

        def forward(self, x, scale):
            x, _ = self.block_a(self.first(x), scale=scale)
            return self.block_b(self.between(x), scale=scale)[0]

    torch.manual_seed(0)
    model = Stack().eval()
    other = Stack().eval()                                          # stands in for the simulation model
    x, scale = torch.randn(3, 6), torch.full((3, 1), 2.0)
    batches = [(x, scale), (x + 1, scale)]
    forward = lambda m, batch: m(*batch)

    assert utils.add_foward_fn_kwargs_to_inputs(model.block_a, x, scale=scale) == (x, scale, 1.0)
    assert utils.add_foward_fn_kwargs_to_inputs(model.block_a, x, scale, 3.0) == (x, scale, 3.0)

    fp_in, q_in = sampler.get_block_inputs(model, SimpleNamespace(model=other), "block_a", batches, True, forward, 2,
                                           None, incl_kwargs=True)
    assert len(fp_in) == len(q_in) == 2 and len(fp_in[0]) == 3
    assert torch.equal(fp_in[1][0], model.first(x + 1)) and torch.equal(q_in[1][0], other.first(x + 1))
    assert torch.equal(fp_in[0][1], scale) and fp_in[0][2] == 1.0
    without_keywords = utils.cache_intermediate_datasets(batches, True, model, "block_a", forward)
    assert len(without_keywords[0]) == 1                            # positional inputs only
    model.unused = nn.Linear(6, 6)
    with pytest.raises(RuntimeError):
        utils.cache_intermediate_datasets(batches, True, model, "unused", forward)
    del model.unused

    fp_blocks, q_blocks = sampler.create_modulelist_for_group_modules(model, SimpleNamespace(model=other),
                                                                      {"a": ["block_a"], "b": ["between"]})
    assert fp_blocks[0][0] is model.block_a and q_blocks[1][0] is other.between
    expected = model.block_a(*fp_in[0])[0]
    run = lambda block, inputs: block[0](*inputs)
    sampler.get_block_outputs(fp_blocks[0], q_blocks[0], "True", fp_in, q_in, True, run, torch.device("cpu"))
    assert torch.equal(fp_in[0][0], expected) and len(fp_in[0]) == 3 and torch.equal(fp_in[0][1], scale)
    fp_next, q_next = [[t[0]] for t in fp_in], [[t[0]] for t in q_in]
    sampler.get_block_outputs(fp_blocks[1], q_blocks[1], "False", fp_next, q_next, True, run, torch.device("cpu"))
    assert len(q_next[0]) == 1 and torch.equal(q_next[0][0], other.between(q_in[0][0]))
    assert torch.equal(fp_next[1][0], model.between(fp_in[1][0]))

    schedule = sampler.create_cached_block_schedule_list(model, (x, scale), ["block_a", "block_b"], (nn.Linear,))
    assert [(b if b is None else b[0], [n for n, _ in layers]) for b, layers in schedule] == \
        [(None, ["first"]), ("block_a", ["fc"]), (None, ["between"]), ("block_b", ["fc"])]


def test_v2_quantization_parameters_registered_by_a_subclass():
    """register_quantization_parameter (reference v2/quantization/base/quantizer.py:99-135): a parameter registered
    this way counts towards is_initialized(), travels in the extra state, and survives copies and pickles."""
    import copy
    import pickle
    from aimet_amd.v2.quantization.affine import QuantizeDequantize
    quantizer = QuantizeDequantize((), 8, False)
    quantizer.register_quantization_parameter('gamma', nn.Parameter(torch.ones(())))
    assert sorted(dict(quantizer.named_parameters())) == ['gamma', 'max', 'min']
    with torch.no_grad():
        quantizer.min.fill_(-1.)
        quantizer.max.fill_(2.)
    assert not quantizer.is_initialized()                           # gamma is still the object it was created as
    with torch.no_grad():
        quantizer.gamma.mul_(1.)
    assert quantizer.is_initialized()
    assert sorted(quantizer.get_extra_state()) == ['gamma', 'max', 'min']
    assert copy.deepcopy(quantizer).is_initialized() and pickle.loads(pickle.dumps(quantizer)).is_initialized()
    fresh = QuantizeDequantize((), 8, False)
    fresh.register_quantization_parameter('gamma', nn.Parameter(torch.ones(())))
    assert not fresh.is_initialized()
    fresh.load_state_dict(quantizer.state_dict())
    assert fresh.is_initialized() and float(fresh.max.detach()) == 2.0
