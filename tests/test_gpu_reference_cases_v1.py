"""The cases of the reference's own v1 tensor-quantizer tests (TrainingExtensions/torch/test/python/
test_tensor_quantizer.py) that are not already part of tests/test_gpu_facade_v1.py, run on the GPU path: histogram
read-out, the unsigned-symmetric flag, bitwidth 32, fixed min / max values, non-contiguous inputs, extreme values."""
import pytest
import torch

pytestmark = pytest.mark.gpu

BUCKET_SIZE = 512


@pytest.fixture(scope="module")
def api():
    from aimet_amd.common import libpymo
    from aimet_amd.common.defs import QuantScheme
    from aimet_amd.v1 import tensor_quantizer as tq

    class Api:
        pass
    a = Api()
    a.libpymo, a.QuantScheme, a.tq = libpymo, QuantScheme, tq
    a.nearest = libpymo.RoundingMode.ROUND_NEAREST
    return a


def test_get_stats_histogram_per_tensor(api):
    # :60-75
    tensor = torch.randn(5, 5).cuda()
    quantizer = api.tq.StaticGridPerTensorQuantizer(8, api.nearest, api.QuantScheme.post_training_tf_enhanced,
                                                    use_symmetric_encodings=False, enabled_by_default=True)
    quantizer.update_encoding_stats(tensor)
    quantizer.compute_encoding()
    histograms = quantizer.get_stats_histogram()
    assert len(histograms) == 1
    for histogram in histograms:
        assert len(histogram) == BUCKET_SIZE
    assert sum(p for _, p in histograms[0]) == pytest.approx(1.0, abs=1e-9)       # a probability density


def test_get_stats_histogram_per_channel(api):
    # :77-92
    tensor = torch.randn(10, 5).cuda()
    quantizer = api.tq.StaticGridPerChannelQuantizer(8, api.nearest, api.QuantScheme.post_training_tf_enhanced,
                                                     use_symmetric_encodings=False, num_channels=10,
                                                     enabled_by_default=True)
    quantizer.update_encoding_stats(tensor)
    quantizer.compute_encoding()
    histograms = quantizer.get_stats_histogram()
    assert len(histograms) == 10
    for histogram in histograms:
        assert len(histogram) == BUCKET_SIZE


def test_get_stats_histogram_with_invalid_combination(api):
    # :94-110
    tensor = torch.randn(5, 5).cuda()
    tf_quantizer = api.tq.StaticGridPerTensorQuantizer(8, api.nearest, api.QuantScheme.post_training_tf,
                                                       use_symmetric_encodings=False, enabled_by_default=True)
    tf_quantizer.update_encoding_stats(tensor)
    tf_quantizer.compute_encoding()
    with pytest.raises(RuntimeError):
        tf_quantizer.get_stats_histogram()                          # TF keeps no histogram
    tfe_quantizer = api.tq.StaticGridPerTensorQuantizer(8, api.nearest, api.QuantScheme.post_training_tf_enhanced,
                                                        use_symmetric_encodings=False, enabled_by_default=True)
    with pytest.raises(RuntimeError):
        tfe_quantizer.get_stats_histogram()                         # no encoding computed yet


def test_is_unsigned_symmetric_flag(api):
    # :112-152: the flag follows the sign of the observed data and the quantizer's configuration
    def make(sym, unsigned):
        q = api.tq.StaticGridPerTensorQuantizer(8, api.nearest, api.QuantScheme.post_training_tf,
                                                use_symmetric_encodings=sym, enabled_by_default=True)
        q.use_unsigned_symmetric = unsigned
        return q

    positive, mixed = torch.rand(5, 5).cuda(), torch.randn(10, 5).cuda()
    q = make(True, True)
    q.update_encoding_stats(positive)
    q.compute_encoding()
    assert q.is_unsigned_symmetric and q.encoding.min == 0 and q.encoding.offset == 0
    q = make(True, True)
    q.update_encoding_stats(mixed)
    q.compute_encoding()
    assert not q.is_unsigned_symmetric and q.encoding.offset == -128
    q = make(True, False)
    q.update_encoding_stats(positive)
    q.compute_encoding()
    assert not q.is_unsigned_symmetric and q.encoding.offset == -128
    q = make(False, True)
    q.update_encoding_stats(positive)
    q.compute_encoding()
    assert not q.is_unsigned_symmetric


@pytest.mark.parametrize("per_channel", [False, True])
def test_tensor_quantizer_bitwidth_32(api, per_channel):
    # :154-193: statistics, encodings and quantization are all skipped
    if per_channel:
        quantizer = api.tq.StaticGridPerChannelQuantizer(32, api.nearest, api.QuantScheme.post_training_tf,
                                                         use_symmetric_encodings=False, num_channels=10,
                                                         enabled_by_default=True)
    else:
        quantizer = api.tq.StaticGridPerTensorQuantizer(32, api.nearest, api.QuantScheme.post_training_tf,
                                                        use_symmetric_encodings=False, enabled_by_default=True)
    tensor = torch.randn(10, 5).cuda()
    quantizer.update_encoding_stats(tensor)
    quantizer.compute_encoding()
    assert quantizer.encoding is None
    assert quantizer.enabled
    assert torch.equal(quantizer.quantize_dequantize(tensor, api.nearest), tensor)


@pytest.mark.parametrize("per_channel", [False, True])
def test_tensor_quantizer_fix_encoding_min_max_vals(api, per_channel):
    # :195-220: the fixed values replace the observed statistics
    if per_channel:
        quantizer = api.tq.StaticGridPerChannelQuantizer(8, api.nearest, api.QuantScheme.post_training_tf,
                                                         use_symmetric_encodings=False, num_channels=3,
                                                         enabled_by_default=True)
    else:
        quantizer = api.tq.StaticGridPerTensorQuantizer(8, api.nearest, api.QuantScheme.post_training_tf_enhanced,
                                                        use_symmetric_encodings=False, enabled_by_default=True)
    quantizer.encoding_min_max_fixed_vals = (0.0, 1.0)
    assert quantizer.quant_scheme == api.QuantScheme.post_training_tf
    quantizer.update_encoding_stats(torch.tensor([[-3.0, 7.0], [0.1, 0.2], [5.0, -9.0]]).cuda())
    quantizer.compute_encoding()
    encodings = quantizer.encoding if isinstance(quantizer.encoding, list) else [quantizer.encoding]
    assert len(encodings) == (3 if per_channel else 1)
    for enc in encodings:
        assert enc.min == pytest.approx(0.0, abs=1e-6) and enc.max == pytest.approx(1.0, abs=1e-6)
    with pytest.raises(AssertionError):
        quantizer.encoding_min_max_fixed_vals = (1.0, 0.5)


@pytest.mark.parametrize("kind", ["per_tensor", "per_channel_axis0", "per_channel_axis1"])
def test_non_contiguous_input_tensor(api, kind):
    # :354-398
    if kind == "per_tensor":
        quantizer = api.tq.StaticGridPerTensorQuantizer(8, api.nearest, api.QuantScheme.post_training_tf,
                                                        use_symmetric_encodings=False, enabled_by_default=True)
    else:
        quantizer = api.tq.StaticGridPerChannelQuantizer(8, api.nearest, api.QuantScheme.post_training_tf,
                                                         use_symmetric_encodings=True, enabled_by_default=True,
                                                         num_channels=5, ch_axis=0 if kind.endswith("0") else 1)
    tensor = torch.randn((5, 5, 100, 100)).cuda()
    quantizer.update_encoding_stats(tensor)
    quantizer.compute_encoding()
    out_contiguous = quantizer.quantize_dequantize(tensor.to(memory_format=torch.contiguous_format),
                                                   quantizer.round_mode)
    out_channels_last = quantizer.quantize_dequantize(tensor.to(memory_format=torch.channels_last),
                                                      quantizer.round_mode)
    assert torch.equal(out_contiguous, out_channels_last)
    tensor = tensor.view(*tensor.shape, 1)
    out_contiguous = quantizer.quantize_dequantize(tensor.to(memory_format=torch.contiguous_format),
                                                   quantizer.round_mode)
    out_channels_last_3d = quantizer.quantize_dequantize(tensor.to(memory_format=torch.channels_last_3d),
                                                         quantizer.round_mode)
    assert torch.equal(out_contiguous, out_channels_last_3d)
    if kind == "per_tensor":
        out_contiguous = quantizer.quantize_dequantize(tensor[..., ::2, :].contiguous(), quantizer.round_mode)
        out_strided = quantizer.quantize_dequantize(tensor[..., ::2, :], quantizer.round_mode)
        assert torch.equal(out_contiguous, out_strided)


@pytest.mark.parametrize("tensor", (torch.tensor([0, -3.4028e38, -3.4028e38]), torch.tensor([0, 3.4028e38]),
                                    torch.tensor([3.4028e38, 0, -3.4028e38])))
@pytest.mark.parametrize("scheme", ("post_training_tf", "post_training_tf_enhanced"))
@pytest.mark.parametrize("symmetric", (True, False))
def test_tensor_quantizer_extreme_values(api, scheme, tensor, symmetric):
    # :420-450: finite, ordered encodings for values at the edge of float32
    quantizer = api.tq.StaticGridPerTensorQuantizer(8, api.nearest, api.QuantScheme[scheme],
                                                    use_symmetric_encodings=symmetric, enabled_by_default=True)
    quantizer.update_encoding_stats(tensor.cuda())
    quantizer.compute_encoding()
    encoding = quantizer.encoding
    enc_min = torch.tensor(encoding.min, dtype=torch.float32)
    enc_max = torch.tensor(encoding.max, dtype=torch.float32)
    assert not torch.isinf(enc_min) and not torch.isnan(enc_min)
    assert not torch.isinf(enc_max) and not torch.isnan(enc_max)
    assert enc_min < enc_max
    assert encoding.delta > 0
