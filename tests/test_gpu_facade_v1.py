"""GPU tests of the v1 host-side interface (tensor quantizers, wrappers, QuantizationSimModel) against the CPU oracle.

The cases follow the reference's own unit tests of this interface (TrainingExtensions/torch/test/python/
test_tensor_quantizer.py, test_quantizer.py): statistics -> encoding -> quantize-dequantize -> straight-through
gradient, per tensor and per channel, then the model-level flow compute_encodings / forward / export.
Encodings and quantized values must be identical to the oracle's; nothing here is a tolerance test.
"""
import json
import os

import numpy as np
import pytest
import torch
from torch import nn

pytestmark = pytest.mark.gpu

@pytest.fixture(scope="module")
def api():
    from aimet_amd.common import libpymo
    from aimet_amd.common.defs import QuantScheme
    from aimet_amd.v1 import qc_quantize_op, quantsim, tensor_quantizer

    class Api:
        pass
    a = Api()
    a.libpymo, a.QuantScheme, a.qc, a.quantsim, a.tq = libpymo, QuantScheme, qc_quantize_op, quantsim, tensor_quantizer
    a.nearest = libpymo.RoundingMode.ROUND_NEAREST
    return a


def _enc_tuple(e):
    return (e.min, e.max, e.delta, e.offset, e.bw)


@pytest.mark.parametrize("scheme", ["tf", "tfe"])
@pytest.mark.parametrize("bw,sym", [(8, False), (8, True), (4, False)])
def test_per_tensor_quantizer(api, oracle, scheme, bw, sym):
    qs = api.QuantScheme.post_training_tf if scheme == "tf" else api.QuantScheme.post_training_tf_enhanced
    q = api.tq.StaticGridPerTensorQuantizer(bw, api.nearest, qs, sym, enabled_by_default=True)
    rng = np.random.default_rng(3)
    batches = [(rng.standard_normal(20000) * s).astype(np.float32) for s in (1.0, 1.5)]
    for b in batches:
        q.update_encoding_stats(torch.from_numpy(b).cuda())
    q.compute_encoding()
    if scheme == "tf":
        mn = min(float(b.min()) for b in batches)
        mx = max(float(b.max()) for b in batches)
        expect = oracle.tf_compute_encoding(mn, mx, bw, sym)
    else:
        pdf = oracle.new_pdf()
        for b in batches:
            pdf.update(b)
        expect, _, _ = pdf.compute_encoding(bw, sym)
    assert _enc_tuple(q.encoding) == expect.astuple()
    x = (rng.standard_normal(5003) * 2).astype(np.float32)
    xg = torch.from_numpy(x).cuda().requires_grad_(True)
    y = q.quantize_dequantize(xg, api.nearest)
    assert np.array_equal(y.detach().cpu().numpy(), oracle.qdq_per_tensor(x, expect.min, expect.max, bw))
    g = rng.standard_normal(x.size).astype(np.float32)
    y.backward(torch.from_numpy(g).cuda())
    assert np.array_equal(xg.grad.cpu().numpy(), oracle.ste_bwd_per_tensor(x, g, expect.min, expect.max))
    codes = q.quantize(torch.from_numpy(x).cuda(), api.nearest)
    # quantize-only shifts to the signed range unless the quantizer is unsigned-symmetric
    assert np.array_equal(codes.cpu().numpy(), oracle.quantize_per_tensor(x, expect.min, expect.max, bw, True))


@pytest.mark.parametrize("scheme", ["tf", "tfe"])
@pytest.mark.parametrize("shape,axis", [((16, 8, 3, 3), 0), ((6, 10, 3, 3), 1), ((32, 48), 0)])
def test_per_channel_quantizer(api, oracle, scheme, shape, axis):
    qs = api.QuantScheme.post_training_tf if scheme == "tf" else api.QuantScheme.post_training_tf_enhanced
    q = api.tq.StaticGridPerChannelQuantizer(8, api.nearest, qs, True, num_channels=shape[axis],
                                             enabled_by_default=True, ch_axis=axis)
    rng = np.random.default_rng(5)
    w = (rng.laplace(0, 0.02, size=shape)).astype(np.float32)
    q.update_encoding_stats(torch.from_numpy(w).cuda())
    q.compute_encoding()
    expect = []
    for c in range(shape[axis]):
        sl = np.ascontiguousarray(np.take(w, c, axis=axis)).reshape(-1)
        if scheme == "tf":
            expect.append(oracle.tf_compute_encoding(float(sl.min()), float(sl.max()), 8, True))
        else:
            pdf = oracle.new_pdf()
            pdf.update(sl)
            expect.append(pdf.compute_encoding(8, True)[0])
    assert [_enc_tuple(e) for e in q.encoding] == [e.astuple() for e in expect]
    xg = torch.from_numpy(w * 1.3).cuda().requires_grad_(True)
    y = q.quantize_dequantize(xg, api.nearest)
    npc = int(np.prod(shape[axis + 1:]))
    params = oracle.per_channel_params(np.array([e.min for e in expect], np.float32),
                                       np.array([e.max for e in expect], np.float32), 8)
    want = oracle.qdq_per_channel((w * 1.3).astype(np.float32).reshape(-1), shape[axis], npc, params)
    assert np.array_equal(y.detach().cpu().numpy().reshape(-1), want)
    g = rng.standard_normal(w.size).astype(np.float32)
    y.backward(torch.from_numpy(g.reshape(shape)).cuda())
    want_g = oracle.ste_bwd_per_channel((w * 1.3).astype(np.float32).reshape(-1), g, shape[axis], npc,
                                        np.array([e.min for e in expect], np.float32),
                                        np.array([e.max for e in expect], np.float32))
    assert np.array_equal(xg.grad.cpu().numpy().reshape(-1), want_g)


def test_cpu_tensors_are_rejected(api):
    q = api.tq.StaticGridPerTensorQuantizer(8, api.nearest, api.QuantScheme.post_training_tf, False, True)
    with pytest.raises(RuntimeError):
        q.update_encoding_stats(torch.randn(10))


def test_disabled_and_frozen_quantizers(api):
    """test_tensor_quantizer.py: a disabled quantizer ignores statistics; a frozen one keeps its encoding."""
    q = api.tq.StaticGridPerTensorQuantizer(8, api.nearest, api.QuantScheme.post_training_tf, False, True)
    with pytest.raises(RuntimeError):
        q.freeze_encoding()
    q.update_encoding_stats(torch.randn(100).cuda())
    q.compute_encoding()
    first = _enc_tuple(q.encoding)
    q.freeze_encoding()
    q.reset_encoding_stats()
    q.update_encoding_stats(torch.randn(100).cuda() * 10)
    q.compute_encoding()
    assert _enc_tuple(q.encoding) == first and q.is_encoding_frozen
    with pytest.raises(RuntimeError):
        q.encoding = q.encoding
    # no statistics at all -> quantizer disables itself
    q2 = api.tq.StaticGridPerTensorQuantizer(8, api.nearest, api.QuantScheme.post_training_tf, False, True)
    q2.compute_encoding()
    assert q2.enabled is False and q2.encoding is None


class _Net(nn.Module):
    def __init__(self):
        super().__init__()
        self.conv1 = nn.Conv2d(3, 8, 3, padding=1)
        self.relu1 = nn.ReLU()
        self.conv2 = nn.Conv2d(8, 8, 3, padding=1, bias=False)
        self.bn = nn.BatchNorm2d(8)
        self.flatten = nn.Flatten()
        self.fc = nn.Linear(8 * 6 * 6, 5)

    def forward(self, x):
        x = self.relu1(self.conv1(x))
        x = self.bn(self.conv2(x))
        return self.fc(self.flatten(x))


def _calibrate(model, batches):
    for b in batches:
        model(b)


def test_quantsim_flow(api, oracle, tmp_path):
    torch.manual_seed(0)
    model = _Net().eval().cuda()
    dummy = torch.randn(2, 3, 6, 6).cuda()
    sim = api.quantsim.QuantizationSimModel(model, dummy_input=dummy, quant_scheme='tf_enhanced',
                                            default_output_bw=8, default_param_bw=8)
    w = dict(sim.quant_wrappers())
    assert set(w) == {"conv1", "relu1", "conv2", "bn", "flatten", "fc"}
    # default configuration: model input quantized, Conv+Relu supergroup, bias not quantized, Flatten transparent
    assert w["conv1"].input_quantizers[0].enabled
    assert not w["conv1"].output_quantizers[0].enabled
    assert w["relu1"].output_quantizers[0].enabled
    assert w["conv1"].param_quantizers["weight"].enabled and not w["conv1"].param_quantizers["bias"].enabled
    assert not w["flatten"].output_quantizers[0].enabled
    assert w["fc"].output_quantizers[0].enabled

    batches = [torch.randn(4, 3, 6, 6).cuda() for _ in range(3)]
    captured = []
    handle = w["relu1"]._module_to_wrap.register_forward_hook(lambda m, i, o: captured.append(o.detach().cpu()))
    sim.compute_encodings(_calibrate, batches)
    handle.remove()
    # the relu output quantizer saw exactly the captured activations
    pdf = oracle.new_pdf()
    for a in captured[:3]:
        pdf.update(a.numpy().reshape(-1))
    expect, _, _ = pdf.compute_encoding(8, False)
    enc = w["relu1"].output_quantizers[0].encoding
    assert _enc_tuple(enc) == expect.astuple()
    # weight encodings: symmetric TF-Enhanced on the weight tensor
    pdf = oracle.new_pdf()
    pdf.update(model.conv2.weight.detach().cpu().numpy().reshape(-1))
    expect_w, _, _ = pdf.compute_encoding(8, True)
    assert _enc_tuple(w["conv2"].param_quantizers["weight"].encoding) == expect_w.astuple()

    # forward in ACTIVE mode: the model output lies on the grid of the last output quantizer
    x = torch.randn(4, 3, 6, 6).cuda()
    with torch.no_grad():
        y = sim.model(x)
    e = w["fc"].output_quantizers[0].encoding
    steps = y.double().cpu().numpy() / e.delta
    assert np.abs(steps - np.round(steps)).max() < 1e-3
    assert y.min().item() >= e.min - 1e-6 and y.max().item() <= e.max + 1e-6
    # parameters are restored after the pass
    assert torch.equal(sim.model.conv2._module_to_wrap.weight, model.conv2.weight)

    # backward reaches the input and the parameters
    x.requires_grad_(True)
    sim.model(x).sum().backward()
    assert x.grad is not None and torch.isfinite(x.grad).all()
    assert sim.model.fc._module_to_wrap.weight.grad is not None

    # export and re-import of parameter encodings
    path = sim.export_encodings(str(tmp_path), "net")
    with open(path) as f:
        data = json.load(f)
    assert "conv2.weight" in data["param_encodings"] and "relu1" in data["activation_encodings"]
    assert data["param_encodings"]["conv2.weight"][0]["scale"] == expect_w.delta
    sim2 = api.quantsim.QuantizationSimModel(model, dummy_input=dummy, quant_scheme='tf_enhanced')
    sim2.set_and_freeze_param_encodings(path)
    q = dict(sim2.quant_wrappers())["conv2"].param_quantizers["weight"]
    assert q.is_encoding_frozen and q.encoding.delta == expect_w.delta


def test_quantsim_per_channel_config(api, tmp_path):
    cfg = {"defaults": {"ops": {"is_output_quantized": "True"},
                        "params": {"is_quantized": "True", "is_symmetric": "True"},
                        "per_channel_quantization": "True"},
           "params": {"bias": {"is_quantized": "False"}}, "op_type": {}, "supergroups": [],
           "model_input": {"is_input_quantized": "True"}, "model_output": {}}
    p = os.path.join(str(tmp_path), "cfg.json")
    with open(p, "w") as f:
        json.dump(cfg, f)
    torch.manual_seed(1)
    model = _Net().eval().cuda()
    dummy = torch.randn(2, 3, 6, 6).cuda()
    sim = api.quantsim.QuantizationSimModel(model, dummy_input=dummy, quant_scheme='tf', config_file=p)
    w = dict(sim.quant_wrappers())
    assert isinstance(w["conv1"].param_quantizers["weight"], api.tq.StaticGridPerChannelQuantizer)
    sim.compute_encodings(_calibrate, [torch.randn(4, 3, 6, 6).cuda()])
    encs = w["conv1"].param_quantizers["weight"].encoding
    assert len(encs) == 8
    wt = model.conv1.weight.detach()
    for c, e in enumerate(encs):
        absmax = wt[c].abs().max().item()
        assert e.max == pytest.approx(absmax, rel=1e-6)      # symmetric TF encoding: max = |w|max of the channel
    with torch.no_grad():
        y = sim.model(dummy)
    assert torch.isfinite(y).all()


class _ReluNet(nn.Module):
    def __init__(self, inplace=False):
        super().__init__()
        self.conv1, self.relu1 = nn.Conv2d(3, 8, 3, padding=1), nn.ReLU(inplace=inplace)
        self.conv2, self.relu2 = nn.Conv2d(8, 8, 3, padding=1), nn.ReLU(inplace=inplace)

    def forward(self, x):
        return self.relu2(self.conv2(self.relu1(self.conv1(x))))


def test_relu_absorbed_by_output_quantizer(api, monkeypatch):
    """A ReLU whose output quantizer has encoding.min == 0 is not executed in inference (the quantizer's clamp does
    its work): results must be identical, element for element, to those with the ReLU executed, for negative, huge,
    infinite and NaN pre-activations alike; and the ReLU must run whenever that identity does not hold."""
    torch.manual_seed(3)
    model = _ReluNet().eval().cuda()
    dummy = torch.randn(2, 3, 6, 6).cuda()
    sim = api.quantsim.QuantizationSimModel(model, dummy_input=dummy, quant_scheme='tf')
    sim.compute_encodings(_calibrate, [torch.randn(8, 3, 6, 6).cuda() for _ in range(2)])
    w = dict(sim.quant_wrappers())
    assert w["relu1"].output_quantizers[0].encoding.min == 0.0
    calls = []
    for name in ("relu1", "relu2"):
        w[name]._module_to_wrap.register_forward_hook(lambda m, i, o, name=name: calls.append(name))

    x = torch.randn(8, 3, 6, 6).cuda() * 3
    with torch.no_grad():
        y_absorbed = sim.model(x)
    assert calls == []
    with monkeypatch.context() as mp:
        mp.setattr(api.qc.StaticGridQuantWrapper, "_relu_is_absorbed", lambda self, inputs, kwargs: False)
        with torch.no_grad():
            y_executed = sim.model(x)
    assert calls == ["relu1", "relu2"]
    assert torch.equal(y_absorbed, y_executed)

    # the wrapper alone, on special values
    special = torch.tensor([-float('inf'), -3e38, -1.0, -1e-30, -0.0, 0.0, 1e-30, 0.3, 1e30, float('inf'),
                            float('nan')], device='cuda')
    calls.clear()
    with torch.no_grad():
        got = w["relu1"](special)
    assert calls == []
    enc = w["relu1"].output_quantizers[0].encoding
    want = w["relu1"].output_quantizers[0].quantize_dequantize(torch.relu(special), api.nearest)
    assert torch.equal(got, want) and got[-1].item() == pytest.approx(enc.max)

    # with autograd the ReLU runs (its gradient at 0 differs from the quantizer's mask)
    calls.clear()
    sim.model(x.clone().requires_grad_(True)).sum().backward()
    assert calls == ["relu1", "relu2"]
    # a symmetric (signed) output grid does not clamp at zero: the ReLU runs
    calls.clear()
    q = w["relu1"].output_quantizers[0]
    q.use_symmetric_encodings = True
    q.reset_encoding_stats()
    q.update_encoding_stats(torch.randn(1000, device='cuda'))
    q.compute_encoding()
    assert q.encoding.min < 0
    with torch.no_grad():
        sim.model(x)
    assert calls == ["relu1"]

    # an in-place ReLU also rewrites its input: it always runs
    model = _ReluNet(inplace=True).eval().cuda()
    sim = api.quantsim.QuantizationSimModel(model, dummy_input=dummy, quant_scheme='tf')
    sim.compute_encodings(_calibrate, [torch.randn(8, 3, 6, 6).cuda()])
    calls.clear()
    for name, wrapper in sim.quant_wrappers():
        if name.startswith("relu"):
            wrapper._module_to_wrap.register_forward_hook(lambda m, i, o, name=name: calls.append(name))
    with torch.no_grad():
        sim.model(x)
    assert calls == ["relu1", "relu2"]


def test_float16_data_type(api, tmp_path):
    """QuantizationDataType.float with bitwidth 16: quantize-dequantize is tensor.half().float() (reference
    tensor_quantizer.py:1104-1107), there are no statistics and no encoding, the gradient passes through, and the
    export names only the type.  Values, special ones included, must equal torch's own conversion bit for bit."""
    from aimet_amd.common.defs import QuantizationDataType
    from aimet_amd import ops
    x = torch.randn(100_003, device="cuda") * 100
    x[:12] = torch.tensor([0.0, -0.0, 65504.0, 65519.9, 65520.0, -70000.0, 1e-8, 5.96e-8, 2.98e-8, 6.1e-5,
                           float("inf"), float("nan")], device="cuda")
    want = x.half().float()
    got = ops.fp16_round_trip(x)
    assert torch.equal(got.view(torch.int32), want.view(torch.int32))
    got = ops.fp16_round_trip(x[1:])                      # 4-byte aligned only: the element-wise kernel
    assert torch.equal(got.view(torch.int32), want[1:].view(torch.int32))

    q = api.tq.StaticGridPerTensorQuantizer(16, api.nearest, api.QuantScheme.post_training_tf_enhanced, False,
                                            enabled_by_default=True, data_type=QuantizationDataType.float)
    q.update_encoding_stats(x)
    q.compute_encoding()
    assert q.encoding is None and q.enabled
    xr = x[12:].clone().requires_grad_(True)
    y = q.quantize_dequantize(xr, api.nearest)
    assert torch.equal(y.detach(), want[12:])
    y.backward(torch.full_like(y, 2.0))
    assert torch.equal(xr.grad, torch.full_like(xr, 2.0))
    xb = x[12:1000].bfloat16()
    assert torch.equal(q.quantize_dequantize(xb, api.nearest), xb.half().float())
    with pytest.raises(ValueError):                       # float grids exist for 16 and 8 bits
        api.tq.StaticGridPerTensorQuantizer(4, api.nearest, api.QuantScheme.post_training_tf, False, True,
                                            data_type=QuantizationDataType.float)

    # a wrapper: parameters and output pass through float16
    torch.manual_seed(2)
    lin = nn.Linear(32, 16).cuda()
    w = api.qc.StaticGridQuantWrapper(lin, 16, 16, 'nearest', api.QuantScheme.post_training_tf,
                                      data_type=QuantizationDataType.float)
    inp = torch.randn(8, 32, device="cuda")
    w.set_mode(api.qc.QcQuantizeOpMode.ANALYSIS)
    w(inp)
    w.compute_encoding()
    w.set_mode(api.qc.QcQuantizeOpMode.ACTIVE)
    with torch.no_grad():
        out = w(inp)
    ref = torch.nn.functional.linear(inp, lin.weight.half().float(), lin.bias.half().float()).half().float()
    assert torch.equal(out, ref)
    assert torch.equal(w._module_to_wrap.weight, lin.weight)

    # the simulation model
    model = _Net().eval().cuda()
    dummy = torch.randn(2, 3, 6, 6).cuda()
    with pytest.raises(ValueError):                       # float needs bitwidths 16 or 8
        api.quantsim.QuantizationSimModel(model, dummy_input=dummy, default_output_bw=4,
                                          default_data_type=QuantizationDataType.float)
    sim = api.quantsim.QuantizationSimModel(model, dummy_input=dummy, quant_scheme='tf', default_output_bw=16,
                                            default_param_bw=16, default_data_type=QuantizationDataType.float)
    sim.compute_encodings(_calibrate, [torch.randn(4, 3, 6, 6).cuda()])
    with torch.no_grad():
        y = sim.model(dummy)
        h = torch.relu(torch.nn.functional.conv2d(dummy.half().float(), model.conv1.weight.half().float(),
                                                  model.conv1.bias, padding=1)).half().float()
        h = torch.nn.functional.conv2d(h, model.conv2.weight.half().float(), padding=1).half().float()
        h = model.bn(h).half().float()
        want_y = torch.nn.functional.linear(h.flatten(1), model.fc.weight.half().float(), model.fc.bias).half().float()
    assert torch.allclose(y, want_y, rtol=1e-3, atol=1e-3)      # same casts; convolution algorithms may differ
    data = sim.get_encodings_dict()
    assert data["param_encodings"]["conv2.weight"] == [{"bitwidth": 16, "dtype": "float"}]
    assert data["activation_encodings"]["relu1"]["output"]["0"] == {"bitwidth": 16, "dtype": "float"}
    assert data["quantizer_args"]["dtype"] == "float"


class _LinearNet(nn.Module):
    def __init__(self):
        super().__init__()
        self.fc1, self.relu1 = nn.Linear(64, 128), nn.ReLU()
        self.fc2, self.relu2 = nn.Linear(128, 128), nn.ReLU()
        self.fc3 = nn.Linear(128, 10)

    def forward(self, x):
        return self.fc3(self.relu2(self.fc2(self.relu1(self.fc1(x)))))


def test_simulation_forward_in_a_hip_graph(api):
    """Inference through the simulation model queues kernels on torch's current stream and never waits for the device,
    so it can be captured once and replayed (a small-batch forward is bound by launch and Python overhead otherwise).
    Replays are interleaved with eager work and synchronisations and each one is checked against the eager result."""
    torch.manual_seed(11)
    model = _LinearNet().eval().cuda()
    dummy = torch.randn(4, 64).cuda()
    cfg = {"defaults": {"ops": {"is_output_quantized": "True"},
                        "params": {"is_quantized": "True", "is_symmetric": "True"},
                        "per_channel_quantization": "True"},
           "params": {"bias": {"is_quantized": "False"}}, "op_type": {},
           "supergroups": [{"op_list": ["Gemm", "Relu"]}], "model_input": {"is_input_quantized": "True"},
           "model_output": {}}
    sim = api.quantsim.QuantizationSimModel(model, dummy_input=dummy, quant_scheme='tf_enhanced', config_file=cfg)
    sim.compute_encodings(_calibrate, [torch.randn(32, 64).cuda() for _ in range(2)])
    static_x = torch.randn(16, 64).cuda()
    with torch.no_grad():
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(3):
                sim.model(static_x)                         # warm-up outside the capture
        torch.cuda.current_stream().wait_stream(side)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            static_y = sim.model(static_x)
        for rep in range(5):
            x = torch.randn(16, 64).cuda() * (rep + 1)
            static_x.copy_(x)
            graph.replay()
            torch.cuda.synchronize()
            eager = sim.model(x)                            # eager work between the replays
            assert torch.equal(static_y, eager), rep
            torch.cuda.synchronize()


@pytest.mark.parametrize("bw,sym,strict,unsigned", [(8, True, False, False), (4, True, False, False), (8, False, False, False),
                                                     (8, True, True, False), (8, True, False, True), (16, False, False, False)])
def test_per_channel_tf_encodings_stay_on_the_device(api, oracle, bw, sym, strict, unsigned):
    """The min / max encodings of a per-channel quantizer are computed by one launch and left on the device; the list of
    TfEncoding objects is built when it is read.  Encodings, kernel parameters, quantized values and gradients are
    those of the host path (one computation per channel), bit for bit, including channels that are all zero, all
    positive, tiny and huge."""
    import pickle
    rng = np.random.default_rng(17)
    w = (rng.laplace(0, 0.03, (48, 70))).astype(np.float32)
    w[0] = 0.0                      # no range at all
    w[1] = np.abs(w[1]) + 0.5       # strictly positive (the unsigned grid differs here)
    w[2] = -np.abs(w[2]) - 0.5      # strictly negative
    w[3] *= 1e-30
    w[4] *= 1e30
    w[5, 0] = np.float32(3e38)
    wg = torch.from_numpy(w).cuda()

    def make(on_device):
        q = api.tq.StaticGridPerChannelQuantizer(bw, api.nearest, api.QuantScheme.post_training_tf, sym, 48,
                                                 enabled_by_default=True, ch_axis=0)
        q.use_strict_symmetric, q.use_unsigned_symmetric = strict, unsigned
        q.compute_tf_encodings_on_device = on_device
        q.update_encoding_stats(wg)
        q.update_encoding_stats(wg * 0.5)
        q.compute_encoding()
        return q

    dev, host = make(True), make(False)
    # (the unsigned-symmetric flag of a quantizer is decided from every channel's encoding: that reads the list)
    lazy = not (sym and unsigned)
    pending = lambda q: q.__dict__.get('_pending_encoding') is not None
    assert pending(dev) == lazy and not pending(host)
    for a, b in zip(dev.device_params(wg.device), host.device_params(wg.device)):
        assert torch.equal(a.view(torch.int32), b.view(torch.int32))             # as bits: NaN included
    assert pending(dev) == lazy                                                  # still not built
    x = torch.from_numpy((rng.standard_normal(w.shape) * 0.1).astype(np.float32)).cuda()
    outs = []
    for q in (dev, host):
        xg = x.clone().requires_grad_(True)
        y = q.quantize_dequantize(xg, api.nearest)
        y.backward(torch.ones_like(y))
        outs.append((y.detach(), xg.grad))
    assert torch.equal(outs[0][0].view(torch.int32), outs[1][0].view(torch.int32))
    assert torch.equal(outs[0][1].view(torch.int32), outs[1][1].view(torch.int32))
    assert pending(dev) == lazy                                                  # quantizing needs no list
    got, want = dev.encoding, host.encoding                                      # now it is built
    assert dev.__dict__.get('_pending_encoding') is None and isinstance(got, list) and len(got) == 48
    assert [_enc_tuple(e) for e in got] == [_enc_tuple(e) for e in want]
    mn, mx = np.minimum(w, w * 0.5).min(axis=1), np.maximum(w, w * 0.5).max(axis=1)
    for c in (1, 2, 7):
        lo, hi = min(0.0, float(mn[c])), max(0.0, float(mx[c]))
        assert _enc_tuple(got[c]) == oracle.tf_compute_encoding(lo, max(hi, lo + 0.01), bw, sym, strict, unsigned).astuple()
    assert dev.is_unsigned_symmetric == host.is_unsigned_symmetric
    # a pending list travels through pickle as the list
    again = make(True)
    clone = pickle.loads(pickle.dumps(again))
    assert [_enc_tuple(e) for e in clone.encoding] == [_enc_tuple(e) for e in want]


def test_training_mode_wrapper_recomputes_parameter_encodings_on_the_device(api):
    """A wrapper in training mode recomputes its parameter encodings in every forward (reference
    qc_quantize_op.py:769-777).  With per-channel min / max encodings that is one launch and no wait; outputs, input
    and weight gradients are those of the host computation."""
    torch.manual_seed(9)
    x = torch.randn(4, 8, 10, 10).cuda()

    def run(on_device):
        torch.manual_seed(10)
        conv = nn.Conv2d(8, 16, 3, padding=1).cuda()
        wrapper = api.qc.StaticGridQuantWrapper(conv, 8, 8, 'nearest', api.QuantScheme.post_training_tf)
        wrapper.enable_per_channel_quantization()
        q = wrapper.param_quantizers['weight']
        q.compute_tf_encodings_on_device = on_device
        q.use_symmetric_encodings = True
        wrapper.set_mode(api.qc.QcQuantizeOpMode.ANALYSIS)
        wrapper(x)
        wrapper.compute_encoding()
        wrapper.set_mode(api.qc.QcQuantizeOpMode.ACTIVE)
        wrapper.train()
        outs = []
        for step in range(2):
            xi = x.clone().requires_grad_(True)
            conv.weight.grad = None
            y = wrapper(xi)
            y.pow(2).sum().backward()
            outs.append((y.detach().clone(), xi.grad.clone(), conv.weight.grad.clone()))
            with torch.no_grad():
                conv.weight.mul_(1.1)                     # the next pass must see the new range
        return outs, q

    dev, qd = run(True)
    host, qh = run(False)
    assert qd.__dict__.get('_pending_encoding') is not None and qh.__dict__.get('_pending_encoding') is None
    for a, b in zip(dev, host):
        assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])
        # (the convolution's weight-gradient kernel adds in no fixed order: equal up to that, and zero in the same places,
        # which is what the straight-through gate of the parameter decides)
        assert torch.allclose(a[2], b[2], rtol=1e-4, atol=1e-4 * a[2].abs().max().item())
        assert torch.equal(a[2] == 0, b[2] == 0)
    assert not torch.equal(dev[0][0], dev[1][0])
    assert [_enc_tuple(e) for e in qd.encoding] == [_enc_tuple(e) for e in qh.encoding]


@pytest.mark.parametrize("bw,sym", [(8, True), (4, True), (8, False)])
def test_per_channel_tf_enhanced_encodings_stay_on_the_device(api, bw, sym):
    """The per-channel TF-Enhanced search leaves its encodings on the device as well: same encodings, parameters and
    quantized values as with the read-back per call; a quantizer without statistics still ends up disabled."""
    rng = np.random.default_rng(23)
    w = torch.from_numpy((rng.laplace(0, 0.03, (40, 300))).astype(np.float32)).cuda()

    def make(on_device, feed=True):
        q = api.tq.StaticGridPerChannelQuantizer(bw, api.nearest, api.QuantScheme.post_training_tf_enhanced, sym, 40,
                                                 enabled_by_default=True, ch_axis=0)
        q.compute_tf_encodings_on_device = on_device
        if feed:
            q.update_encoding_stats(w)
            q.update_encoding_stats(w * 1.5)
        q.compute_encoding()
        return q

    dev, host = make(True), make(False)
    assert dev.__dict__.get('_pending_encoding') is not None and host.__dict__.get('_pending_encoding') is None
    for a, b in zip(dev.device_params(w.device), host.device_params(w.device)):
        assert torch.equal(a.view(torch.int32), b.view(torch.int32))
    assert torch.equal(dev.quantize_dequantize(w, api.nearest), host.quantize_dequantize(w, api.nearest))
    assert dev.__dict__.get('_pending_encoding') is not None
    assert [_enc_tuple(e) for e in dev.encoding] == [_enc_tuple(e) for e in host.encoding]
    empty = make(True, feed=False)
    assert not empty.enabled and not empty.encoding
