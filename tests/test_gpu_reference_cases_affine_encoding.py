"""AffineEncoding along the reference's TrainingExtensions/torch/test/python/v2/encodings/test_affine_encoding.py:
construction from (scale, offset, bitwidth[, signed]) and (scale, offset, qmin, qmax), the derived properties, moving
between devices and floating-point types, granularity, and blockwise quantize / dequantize against per-channel."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def _cls():
    from aimet_amd.v2.quantization.affine import AffineEncoding
    return AffineEncoding


def _tensors_of(encoding):
    return [encoding.min, encoding.max, encoding.scale, encoding.offset]


def test_asymmetric_from_scale_offset_bitwidth():
    offset = torch.tensor(-5)
    encoding = _cls()(torch.tensor(1.0), offset, bitwidth=8)
    for t in _tensors_of(encoding):
        assert isinstance(t, torch.Tensor) and t.shape == ()
    assert encoding.min == -5.0 and encoding.max == 2 ** 8 - 1 + offset and encoding.offset == -5
    assert encoding.bitwidth == 8 and encoding.num_steps == 255 and encoding.dtype == torch.uint8
    assert encoding.granularity == "pertensor" and encoding.mapping == "affine" and encoding.symmetry is False
    assert not encoding.signed


def test_signed_and_unsigned_symmetric():
    encoding = _cls()(torch.tensor(1.0), torch.tensor(0), bitwidth=8, signed=True, symmetry=True)
    assert (encoding.min, encoding.max, encoding.offset, encoding.scale) == (-128, 127, 0, 1.0)
    assert encoding.symmetry is True and encoding.dtype == torch.int8 and encoding.num_steps == 255
    encoding = _cls()(torch.tensor(0.5), torch.tensor(0), bitwidth=8, signed=False, symmetry=True)
    assert (encoding.min, encoding.max, encoding.offset, encoding.scale) == (0, 255.0 / 2, 0, 0.5)
    assert encoding.symmetry is True and encoding.dtype == torch.uint8 and encoding.num_steps == 255


def test_grid_forms_and_refusals():
    cls = _cls()
    by_grid = cls(torch.tensor(1.0), torch.tensor(0.), -8, 7)
    assert by_grid.bitwidth == 4 and by_grid.signed and by_grid.dtype == torch.int8
    assert cls(torch.tensor(1.0), torch.tensor(0.), qmin=0, qmax=65535).dtype == torch.int32
    assert cls(torch.tensor(1.0), torch.tensor(0.), 16, True).dtype == torch.int16
    odd = cls(torch.tensor(1.0), torch.tensor(0.), -3, 11)
    with pytest.raises(RuntimeError):
        _ = odd.bitwidth
    with pytest.raises(ValueError):
        cls(torch.tensor(1.0), torch.tensor(0.), 5, 5)
    with pytest.raises(TypeError):
        cls(torch.tensor(1.0), torch.tensor(0.), 8, nonsense=1)
    with pytest.raises(TypeError):
        cls(torch.tensor(1.0), torch.tensor(0.))


@pytest.mark.parametrize("device,new_device", (("cuda:0", "cpu"), ("cpu", "cuda:0")))
def test_device_of_the_encoding(device, new_device):
    encoding = _cls()(torch.ones([]).to(device), torch.ones([]).to(device), bitwidth=8)
    moved = encoding.to(new_device)
    assert all(t.device == torch.device(device) for t in _tensors_of(encoding))
    assert all(t.device == torch.device(new_device) for t in _tensors_of(moved))
    assert encoding.to(device) is encoding


@pytest.mark.parametrize("dtype,new_dtype", ((torch.float16, torch.float32), (torch.float32, torch.float16)))
def test_dtype_of_the_encoding(dtype, new_dtype):
    encoding = _cls()(torch.ones([]).to(dtype), torch.ones([]).to(dtype), bitwidth=8)
    changed = encoding.to(new_dtype)
    assert all(t.dtype == dtype for t in _tensors_of(encoding))
    assert all(t.dtype == new_dtype for t in _tensors_of(changed))
    for integer in (torch.uint8, torch.int32):
        with pytest.raises(RuntimeError):
            encoding.to(integer)


@pytest.mark.parametrize("shape", ((10, 1), (10,), (1,), ()))
def test_granularity(shape):
    encoding = _cls()(torch.randn(shape), torch.randn(shape), 8)
    assert all(t.shape == shape for t in _tensors_of(encoding))
    assert encoding.granularity == ("pertensor" if shape == () else "perchannel")
    assert encoding.mapping == "affine"
    if shape == (10, 1):
        assert _cls()(torch.randn(10, 4), torch.randn(10, 4), 8).granularity == "unknown"
        assert _cls()(torch.randn(10, 4), torch.randn(10, 4), 8, block_size=(1, 8)).granularity == "blockwise"


def test_blocks_of_one_element_equal_per_channel():
    torch.manual_seed(3)
    scale, offset = torch.randn(2, 2, 2, 2).cuda(), torch.zeros(2, 2, 2, 2).cuda()
    blockwise = _cls()(scale, offset, 8, block_size=[1, 1, 1, 1])
    per_channel = _cls()(scale, offset, 8)
    x = torch.randn(2, 2, 2, 2).cuda()
    on_blocks, on_channels = blockwise.quantize(x), per_channel.quantize(x)
    assert torch.equal(on_blocks, on_channels)
    assert torch.equal(on_blocks, torch.clamp(torch.round(x / scale) - offset, 0, 255))
    assert torch.equal(blockwise.dequantize(on_blocks), blockwise.dequantize(on_channels))
    assert torch.equal(per_channel.dequantize(on_channels), (on_channels + offset) * scale)


def test_the_quantizers_hand_out_this_class():
    from aimet_amd.v2.quantization.affine import QuantizeDequantize
    q = QuantizeDequantize((4, 1), 8, True).cuda()
    x = torch.randn(4, 32).cuda()
    with q.compute_encodings():
        q(x)
    encoding = q.get_encoding()
    assert isinstance(encoding, _cls()) and encoding.granularity == "perchannel" and encoding.symmetry
    assert torch.equal(encoding.dequantize(encoding.quantize(x)), q(x))
