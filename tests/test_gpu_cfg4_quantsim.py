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
