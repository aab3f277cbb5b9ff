"""GPU tests of the grouped blockwise quantizer (block scales as small integers times one scale per group).

Cases follow the reference's own tests, TrainingExtensions/torch/test/python/v2/quantization/affine/
test_affine_quantizer.py:1017-1160 (same shapes, groupings, bitwidths and assertions, on GPU tensors), plus the scales
against a numpy restatement of the rule and the quantizer's output against the plain blockwise kernel fed those scales."""
import itertools

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def affine():
    from aimet_amd.v2.quantization import affine as a
    return a


def _calibrated(quantizer, tensor):
    quantizer = quantizer.cuda()
    with quantizer.compute_encodings():
        _ = quantizer(tensor)
    return quantizer


def test_largest_scale_of_a_channel_is_the_per_channel_scale(affine):
    # test_gbbq_sanity
    torch.manual_seed(0)
    tensor = torch.randn(8, 12).cuda()
    gbbq = _calibrated(affine.GroupedBlockQuantizeDequantize(shape=(8, 4), bitwidth=4, symmetric=True,
                                                             decompressed_bw=8, block_size=(-1, -1),
                                                             block_grouping=(1, -1)), tensor)
    pc = _calibrated(affine.QuantizeDequantize(shape=(8, 1), bitwidth=4, symmetric=True), tensor)
    assert gbbq.get_scale().shape == (8, 4)
    assert torch.equal(torch.amax(gbbq.get_scale(), dim=1, keepdim=True), pc.get_scale())
    assert not torch.equal(gbbq(tensor), pc(tensor))


@pytest.mark.parametrize('bitwidth, decompressed_bw', [[4, 8], [4, 16], [4, 12], [3, 5], [5, 9], [6, 6]])
def test_scales_of_every_group(affine, bitwidth, decompressed_bw):
    # test_gbbq_per_block_sanity
    torch.manual_seed(1)
    tensor = torch.randn(4, 8, 12).cuda()
    grouping = (2, 2, 3)
    gbbq = _calibrated(affine.GroupedBlockQuantizeDequantize(shape=(2, 4, 6), bitwidth=bitwidth, symmetric=True,
                                                             block_size=(2, 2, 2), decompressed_bw=decompressed_bw,
                                                             block_grouping=grouping), tensor)
    qdq = _calibrated(affine.QuantizeDequantize(shape=(2, 4, 6), bitwidth=bitwidth, symmetric=True,
                                                block_size=(2, 2, 2)), tensor)
    got, plain = gbbq.get_scale().cpu(), qdq.get_scale().cpu()
    for i, j, k in itertools.product(*(range(s // g) for s, g in zip(gbbq.shape, grouping))):
        where = tuple(slice(n * g, (n + 1) * g) for n, g in zip((i, j, k), grouping))
        gamma = torch.max(plain[where]) / 2 ** (decompressed_bw - bitwidth)
        want = torch.maximum(torch.tensor([1.0]), torch.round(plain[where] / gamma)) * gamma
        assert torch.equal(want, got[where])
    # the integers and gamma the scales expand to
    integers = gbbq.get_per_block_integer_scale().cpu()
    assert integers.dtype == torch.int32 and integers.shape == (2, 4, 6)
    assert int(integers.min()) >= 1 and int(integers.max()) <= 2 ** (decompressed_bw - bitwidth)
    gamma = gbbq.get_per_channel_scale().cpu()
    assert gamma.shape == (1, 1, 2, 1, 2, 1)
    rebuilt = (integers.view(1, 2, 2, 2, 2, 3).float() * gamma).view(2, 4, 6)
    assert torch.equal(rebuilt, got)


def test_scales_against_numpy_and_output_against_the_blockwise_kernel(affine):
    rng = np.random.default_rng(5)
    w = (rng.standard_normal((64, 256)) * np.exp(rng.standard_normal((64, 1)))).astype(np.float32)
    tensor = torch.from_numpy(w).cuda()
    bw, dbw, block = 4, 8, 32
    gbbq = _calibrated(affine.GroupedBlockQuantizeDequantize(shape=(64, 8), bitwidth=bw, symmetric=True,
                                                             decompressed_bw=dbw, block_size=(1, block),
                                                             block_grouping=(1, -1)), tensor)
    # symmetric min-max range of every block in float32 (delta = max(max / 7, -min / 8), range [-8 delta, 7 delta]),
    # its scale, then the grouping rule
    blocks = w.reshape(64, 8, block)
    pos, neg = np.float32(2 ** (bw - 1) - 1), np.float32(2 ** (bw - 1))
    delta = np.maximum(np.maximum(blocks.max(axis=2), 0) / pos, -np.minimum(blocks.min(axis=2), 0) / neg)
    lo, hi = (-neg * delta).astype(np.float32), (pos * delta).astype(np.float32)
    scale = ((hi - lo) / np.float32(2 ** bw - 1)).astype(np.float32)
    gamma = (scale.max(axis=1, keepdims=True) / np.float32(2 ** (dbw - bw))).astype(np.float32)
    integers = np.clip(np.rint((scale / gamma).astype(np.float32)), 1, 2 ** (dbw - bw)).astype(np.int32)
    # (torch divides a GPU tensor by a Python number through the number's reciprocal, so block scales and gamma may
    # sit one ulp from numpy's quotients; the integers are exact and the scales are exactly integer * gamma)
    got_gamma = gbbq.get_per_channel_scale().detach().cpu().numpy().reshape(64, 1)
    got_scale = gbbq.get_scale().detach().cpu().numpy()
    assert np.allclose(got_gamma, gamma, rtol=5e-7, atol=0)
    assert np.array_equal(gbbq.get_per_block_integer_scale().cpu().numpy(), integers)
    assert np.array_equal(got_scale, integers.astype(np.float32) * got_gamma)
    out = gbbq(tensor)
    direct = affine.quantize_dequantize(tensor, gbbq.get_scale(), torch.zeros(64, 8).cuda(), bw, True,
                                        block_size=(1, block))
    assert torch.equal(out, direct)


def test_default_grouping_keeps_every_block_scale(affine):
    # test_gbbq_quantizer_default_grouping
    torch.manual_seed(2)
    tensor = torch.randn(4, 8, 12).cuda()
    default = _calibrated(affine.GroupedBlockQuantizeDequantize(shape=(2, 4, 6), bitwidth=4, symmetric=True,
                                                                block_size=(2, 2, 2), decompressed_bw=8), tensor)
    ones = _calibrated(affine.GroupedBlockQuantizeDequantize(shape=(2, 4, 6), bitwidth=4, symmetric=True,
                                                             block_size=(2, 2, 2), decompressed_bw=8,
                                                             block_grouping=(1, 1, 1)), tensor)
    assert torch.equal(default.get_scale(), ones.get_scale())
    assert torch.equal(default(tensor), ones(tensor))


@pytest.mark.parametrize('gbbq_shape, decompressed_bw, block_size, grouping, qdq_shape, qdq_block_size',
                         [[(2, 4, 6), 8, (2, 2, 2), (1, 1, 1), (2, 4, 6), (2, 2, 2)],
                          [(2, 4, 6), 4, (2, 2, 2), (-1, -1, -1), (1, 1, 1), None],
                          [(2, 8, 6), 4, (2, 1, 2), (-1, 1, -1), (1, 8, 1), None]])
def test_equivalences(affine, gbbq_shape, decompressed_bw, block_size, grouping, qdq_shape, qdq_block_size):
    # test_gbbq_equivalences: groups of one block = blockwise; one group and no extra bits = per tensor; one group per
    # channel and no extra bits = per channel
    torch.manual_seed(3)
    tensor = torch.randn(4, 8, 12).cuda()
    gbbq = _calibrated(affine.GroupedBlockQuantizeDequantize(shape=gbbq_shape, bitwidth=4, symmetric=True,
                                                             block_size=block_size, decompressed_bw=decompressed_bw,
                                                             block_grouping=grouping), tensor)
    qdq = _calibrated(affine.QuantizeDequantize(shape=qdq_shape, bitwidth=4, symmetric=True,
                                                block_size=qdq_block_size), tensor)
    assert torch.equal(gbbq.get_scale(), qdq.get_scale().expand(gbbq.get_scale().shape))
    gbbq_out, qdq_out = gbbq(tensor), qdq(tensor)
    assert torch.equal(gbbq_out, qdq_out)
    if all(group == 1 for group in grouping):
        grad = torch.randn(gbbq_out.shape).cuda()
        gbbq_out.backward(grad)
        qdq_out.backward(grad)
        assert torch.equal(gbbq.min.grad, qdq.min.grad)
        assert torch.equal(gbbq.max.grad, qdq.max.grad)


def test_invalid_settings(affine):
    # test_invalid_gbbq_settings
    with pytest.raises(RuntimeError):
        affine.GroupedBlockQuantizeDequantize(shape=(2, 4, 6), bitwidth=4, symmetric=False, decompressed_bw=8)
    with pytest.raises(RuntimeError):
        affine.GroupedBlockQuantizeDequantize(shape=(2, 4, 6), bitwidth=4, symmetric=True, decompressed_bw=8,
                                              block_grouping=(-1, -1, -1, -1))
    with pytest.raises(RuntimeError):
        affine.GroupedBlockQuantizeDequantize(shape=(2, 4, 6), bitwidth=4, symmetric=True, decompressed_bw=3)
    with pytest.raises(RuntimeError):
        affine.GroupedBlockQuantizeDequantize(shape=(2, 4, 6), bitwidth=4, symmetric=True, decompressed_bw=8,
                                              block_grouping=(1, 3, 1))


class _ConvPoolLinear(torch.nn.Module):
    def __init__(self):
        super().__init__()
        self.conv, self.relu = torch.nn.Conv2d(3, 8, 3, padding=1), torch.nn.ReLU()
        self.pool, self.flatten = torch.nn.AdaptiveAvgPool2d(3), torch.nn.Flatten()
        self.fc = torch.nn.Linear(72, 10)

    def forward(self, x):
        return self.fc(self.flatten(self.pool(self.relu(self.conv(x)))))


def test_simulation_model_saves_and_loads_grouped_block_encodings(affine, tmp_path):
    # v2/quantsim/test_quantsim.py:743-795 (test_save_and_load_gbbq): a Linear weight of [10, 72] in blocks of 12 with
    # groups of 6 blocks; 60 encodings exported, loading them back restores the outputs
    import json
    from aimet_amd.v2.quantsim import QuantizationSimModel
    torch.manual_seed(0)
    model = _ConvPoolLinear().eval().cuda()
    dummy, other = torch.randn(1, 3, 28, 28).cuda(), torch.randn(1, 3, 28, 28).cuda()
    sim = QuantizationSimModel(model, dummy)
    sim.model.fc.param_quantizers['weight'] = affine.GroupedBlockQuantizeDequantize(
        shape=(10, 6), bitwidth=4, symmetric=True, decompressed_bw=8, block_size=(1, 12),
        block_grouping=(1, 6)).cuda()
    sim.compute_encodings(lambda m, _: m(dummy), None)
    quantizer = sim.model.fc.param_quantizers['weight']
    # every scale of a row is an integer in [1, 16] times the row's gamma
    integers = quantizer.get_per_block_integer_scale()
    assert int(integers.min()) >= 1 and int(integers.max()) == 16
    with torch.no_grad():
        out1 = sim.model(dummy)
    file = sim.export_encodings(str(tmp_path), 'grouped')
    with open(file) as f:
        exported = json.load(f)
    assert len(exported['param_encodings']['fc.weight']) == 60

    old_weight = sim.model.fc.weight
    old_max = quantizer.get_max()[0][0].item()
    sim.model.fc.weight = torch.nn.Parameter(torch.randn(old_weight.shape).cuda())
    sim.compute_encodings(lambda m, _: m(other), None)
    assert quantizer.get_max()[0][0].item() != old_max
    with torch.no_grad():
        assert not torch.equal(out1, sim.model(dummy))

    sim.model.fc.weight = old_weight
    sim.load_encodings(file)
    assert sim.model.fc.param_quantizers['weight'].get_max()[0][0].item() == pytest.approx(old_max, rel=1e-6)
    with torch.no_grad():
        out3 = sim.model(dummy)
    # (min / max come back through the exported scale and offset: the grid agrees to float rounding)
    assert torch.allclose(out1, out3, rtol=1e-5, atol=1e-6)
