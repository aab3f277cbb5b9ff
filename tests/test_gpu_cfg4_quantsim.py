"""The simulation-model configuration at its size: QuantizationSimModel forward on the random-init ResNet-50-shaped
net, batch 64, int8 per-channel symmetric weight quantizers and int8 per-tensor activation quantizers
(reference flow: TrainingExtensions/torch/src/python/aimet_torch/v1/quantsim.py:381-448, qc_quantize_op.py:705-897).

Every quantize-dequantize call of one forward pass is intercepted: the tensor the GPU kernel produced is compared bit
for bit with the CPU oracle's quantize-dequantize of the same input under the quantizer's encoding, and the oracle's
tensor is what flows on, so the logits of that pass are those of the model evaluated with oracle-quantized weights
and activations.  They are compared with an undisturbed pass within the reordering tolerance of the convolutions."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def test_cfg4_every_quantizer_matches_the_oracle(oracle):
    import bench
    from aimet_amd.v1 import tensor_quantizer as tq

    model, sim, x = bench.quantsim_resnet50_shaped(torch, batch=64)
    wrappers = list(sim.quant_wrappers())
    enabled_act = sum(q.enabled for _, w in wrappers for q in w.input_quantizers + w.output_quantizers)
    enabled_par = sum(q.enabled for _, w in wrappers for q in w.param_quantizers.values())
    assert enabled_par >= 54 and enabled_act >= 54           # 53 convolutions + the classifier; their outputs

    with torch.no_grad():
        plain = sim.model(x).cpu()

    # compute_encodings() left every weight quantized by ONE multi-tensor launch; those tensors are checked against the
    # oracle below, then dropped so that the checked pass sees every quantizer at work
    from_multi_launch = {}
    for _, w in wrappers:
        for name, (_, kept) in w.__dict__.get('_param_cache', {}).items():
            from_multi_launch[dict(w.get_named_parameters())[name].data_ptr()] = kept
        w.invalidate_param_cache()
    assert len(from_multi_launch) == enabled_par

    seen = {"per_tensor": 0, "per_channel": 0, "elements": 0}
    real = tq.StaticGridTensorQuantizer.quantize_dequantize

    def checked(self, tensor, round_mode):
        got = real(self, tensor, round_mode)
        if not (self.enabled and self.bitwidth != 32):
            return got
        host = tensor.detach().float().cpu().numpy()
        if isinstance(self, tq.StaticGridPerChannelQuantizer):
            encs = self._encoding                              # pylint: disable=protected-access
            c = tensor.shape[self.channel_axis]
            assert len(encs) == c and self.channel_axis == 0
            npc = tensor[0].numel()
            params = oracle.per_channel_params(np.array([e.min for e in encs]), np.array([e.max for e in encs]),
                                               self.bitwidth)
            want = oracle.qdq_per_channel(host, c, npc, params)
            seen["per_channel"] += 1
            kept = from_multi_launch[tensor.data_ptr()]
            assert np.array_equal(kept.cpu().numpy().view(np.uint32), want.view(np.uint32)), "multi-tensor launch"
        else:
            enc = self.encoding
            want = oracle.qdq_per_tensor(host, enc.min, enc.max, self.bitwidth)
            seen["per_tensor"] += 1
        seen["elements"] += host.size
        assert np.array_equal(got.cpu().numpy().view(np.uint32), want.view(np.uint32)), \
            f"{type(self).__name__} on a tensor of shape {tuple(tensor.shape)}"
        return torch.from_numpy(want).to(tensor.device)

    tq.StaticGridTensorQuantizer.quantize_dequantize = checked
    try:
        with torch.no_grad():
            through_oracle = sim.model(x).cpu()
    finally:
        tq.StaticGridTensorQuantizer.quantize_dequantize = real

    assert seen["per_channel"] == enabled_par and seen["per_tensor"] == enabled_act
    assert seen["elements"] > 5e8                               # the activations of 64 images went through the check
    print(f"cfg4: {seen['per_tensor']} activation + {seen['per_channel']} weight quantizers, "
          f"{seen['elements']} elements, every one bit-identical to the oracle")
    assert torch.isfinite(plain).all()
    # the convolutions (MIOpen) are not run-to-run deterministic in their summation order and every quantizer
    # downstream can turn an ulp into one grid step; logits are O(1) here
    scale = plain.abs().max().item()
    diff = (plain - through_oracle).abs()
    assert diff.max().item() <= 0.05 * scale
    assert diff.mean().item() <= 0.005 * scale


def test_quantized_parameters_are_kept_between_forwards():
    """In evaluation mode a wrapper keeps its quantized parameters while parameter and encoding stay the same, and
    compute_encodings() fills every wrapper from one multi-tensor launch: same outputs as quantizing in every forward,
    and every change that the key sees (in-place update of the parameter, a new encoding, training mode) is seen."""
    from aimet_amd.v1.qc_quantize_op import StaticGridQuantWrapper
    from aimet_amd.v1.quantsim import QuantizationSimModel
    torch.manual_seed(0)
    model = torch.nn.Sequential(torch.nn.Conv2d(3, 16, 3, padding=1), torch.nn.ReLU(), torch.nn.Conv2d(16, 32, 1),
                                torch.nn.ReLU(), torch.nn.AdaptiveAvgPool2d(1), torch.nn.Flatten(),
                                torch.nn.Linear(32, 10)).eval().cuda()
    x = torch.randn(4, 3, 16, 16).cuda()
    sim = QuantizationSimModel(model, dummy_input=x, quant_scheme='tf', default_param_bw=4)
    sim.compute_encodings(lambda m, a: m(a), x)
    layers = [w for _, w in sim.quant_wrappers() if w.param_quantizers]
    assert all('weight' in w.__dict__['_param_cache'] for w in layers)       # filled by compute_encodings
    assert sim.quantize_params_together() >= 3

    def forward(cached):
        StaticGridQuantWrapper.cache_quantized_params = cached
        try:
            with torch.no_grad():
                return sim.model(x)
        finally:
            StaticGridQuantWrapper.cache_quantized_params = True

    assert torch.equal(forward(True), forward(False))
    conv = layers[0]
    kept = conv.__dict__['_param_cache']['weight'][1]
    forward(True)
    assert conv.__dict__['_param_cache']['weight'][1] is kept               # used again, not recomputed
    with torch.no_grad():
        conv._module_to_wrap.weight.mul_(1.5)                                # in place on the parameter: version moves
    assert torch.equal(forward(True), forward(False))
    assert conv.__dict__['_param_cache']['weight'][1] is not kept
    q = conv.param_quantizers['weight']
    from aimet_amd.common import libpymo
    old = q.encoding if isinstance(q.encoding, list) else [q.encoding]
    new = [libpymo.TfEncoding(e.min * 0.5, e.max * 0.5, e.delta * 0.5, e.offset, e.bw) for e in old]
    q.encoding = new if isinstance(q.encoding, list) else new[0]             # a new encoding
    assert torch.equal(forward(True), forward(False))
    sim.model.train()
    out_train = sim.model(x)
    sim.model.eval()
    assert torch.isfinite(out_train).all() and torch.equal(forward(True), forward(False))
    # through a .data alias nothing moves: the documented way out
    conv._module_to_wrap.weight.data.mul_(2.0)
    for w in layers:
        w.invalidate_param_cache()
    assert torch.equal(forward(True), forward(False))


@pytest.mark.parametrize("scheme", ["tf", "tf_enhanced"])
@pytest.mark.parametrize("per_channel", [False, True])
def test_parameter_encodings_taken_ahead_of_the_batches(scheme, per_channel):
    """compute_encodings() observes the parameters before the calibration batches run.  The encodings are those of a
    quantizer fed with the parameter as the wrapper's first forward sees it: a weight changed by the callback before
    that forward is observed again, and a wrapper that never runs loses what was observed for it."""
    from aimet_amd.v1.quantsim import QuantizationSimModel
    from aimet_amd.v1.tensor_quantizer import StaticGridPerChannelQuantizer, StaticGridPerTensorQuantizer
    from aimet_amd.common import libpymo

    class Net(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.a = torch.nn.Conv2d(3, 8, 3, padding=1)
            self.b = torch.nn.Conv2d(8, 8, 1)
            self.spare = torch.nn.Conv2d(8, 8, 1)

        def forward(self, x):
            return self.b(torch.relu(self.a(x)))

    torch.manual_seed(3)
    model = Net().eval().cuda()
    x = torch.randn(2, 3, 12, 12).cuda()
    sim = QuantizationSimModel(model, dummy_input=x, quant_scheme=scheme, default_param_bw=8)
    if per_channel:
        for _, w in sim.quant_wrappers():
            if 'weight' in w.param_quantizers:
                w.enable_per_channel_quantization()

    def callback(m, _):
        with torch.no_grad():
            m.b._module_to_wrap.weight.mul_(3.0)          # after the parameters were observed, before b's forward
        m(x)

    sim.compute_encodings(callback, None)

    def fresh_encoding(like, weight):
        if isinstance(like, StaticGridPerChannelQuantizer):
            q = StaticGridPerChannelQuantizer(like.bitwidth, like.round_mode, like.quant_scheme,
                                              like.use_symmetric_encodings, weight.shape[0], True, ch_axis=0)
        else:
            q = StaticGridPerTensorQuantizer(like.bitwidth, like.round_mode, like.quant_scheme,
                                             like.use_symmetric_encodings, True)
        q.use_strict_symmetric, q.use_unsigned_symmetric = like.use_strict_symmetric, like.use_unsigned_symmetric
        q.update_encoding_stats(weight)
        q.compute_encoding()
        enc = q.encoding if isinstance(q.encoding, list) else [q.encoding]
        return [(e.min, e.max, e.delta, e.offset, e.bw) for e in enc]

    for name in ('a', 'b'):
        wrapper = getattr(sim.model, name)
        q = wrapper.param_quantizers['weight']
        assert q.enabled and not wrapper.__dict__.get('_param_encodings_ahead')
        enc = q.encoding if isinstance(q.encoding, list) else [q.encoding]
        assert [(e.min, e.max, e.delta, e.offset, e.bw) for e in enc] == \
            fresh_encoding(q, wrapper._module_to_wrap.weight.data)
    spare = sim.model.spare.param_quantizers['weight']
    assert not spare.enabled and not spare.encoding
