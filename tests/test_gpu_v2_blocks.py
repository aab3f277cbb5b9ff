"""GPU tests of blockwise and multi-axis scales in the v2 backend and quantizer modules.

Cases follow the reference's own tests: TrainingExtensions/torch/test/python/v2/quantization/affine/backends/
test_backend.py:627-740 (shapes, the known-answer table of test_block_quant, block-versus-slice equality, invalid
block sizes) and .../affine/test_affine_quantizer.py:958-1001 (quantizer modules with block_size), plus parity with the
CPU oracle on the flattened channel layout and gradients against autograd of the textbook expression."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def affine():
    from aimet_amd.v2.quantization import affine as a
    return a


def test_block_size_shapes(affine):
    # test_backend.py:627-646
    torch.manual_seed(0)
    scale = (torch.rand(4, 3, 8, 1) + 0.05).cuda()
    offset = torch.randint(-128, 127, (4, 3, 8, 1)).float().cuda()
    inp = torch.randn(8, 6, 8, 3).cuda()
    block_size = [-1, 2, 1, 3]
    q = affine.quantize(inp, scale, offset, 8, True, block_size=block_size)
    dq = affine.dequantize(q, scale, offset, block_size=block_size)
    qdq = affine.quantize_dequantize(inp, scale, offset, 8, True, block_size=block_size)
    assert q.shape == dq.shape == qdq.shape == inp.shape
    assert torch.equal(dq, qdq)


@pytest.mark.parametrize('scale, offset, block_size, output', [
    [[[0.03, 0.02]], torch.zeros(1, 2), [2, 1], [[-40, 120], [-20, -9]]],
    [[[0.03, 0.02]], torch.zeros(1, 2), [-1, 1], [[-40, 120], [-20, -9]]],
    [[[0.03, 0.02]], torch.zeros(1, 2), None, [[-40, 120], [-20, -9]]],
    [[[0.03], [0.02]], torch.zeros(2, 1), [1, 2], [[-40, 80], [-30, -9]]],
    [[[0.03], [0.02]], torch.zeros(2, 1), [1, -1], [[-40, 80], [-30, -9]]],
    [[[0.03], [0.02]], torch.zeros(2, 1), None, [[-40, 80], [-30, -9]]],
    [[[0.03, 0.02], [0.01, 0.09]], torch.zeros(2, 2), [1, 1], [[-40, 120], [-60, -2]]],
])
def test_block_quant_known_answers(affine, scale, offset, block_size, output):
    # test_backend.py:648-667 (the reference's table)
    inp = torch.tensor([[-1.2, 2.4], [-.6, -.18]]).cuda()
    scale, offset, output = torch.tensor(scale).cuda(), offset.cuda(), torch.tensor(output).cuda()
    q = affine.quantize(inp, scale, offset, 8, True, block_size=block_size)
    assert torch.equal(q, output.to(q.dtype))
    dq = affine.dequantize(q, scale, offset, block_size=block_size)
    assert torch.allclose(dq, inp, atol=1e-6)
    qdq = affine.quantize_dequantize(inp, scale, offset, 8, True, block_size=block_size)
    assert torch.allclose(qdq, inp, atol=1e-6)


def test_every_block_equals_the_per_tensor_result_of_its_slice(affine):
    # test_backend.py:669-716, with leading axes that the block specification does not cover
    torch.manual_seed(1)
    inp = torch.randn(3, 5, 4, 6, 12, 9).cuda()
    scale = (torch.rand(2, 1, 4, 9) * 0.05 + 0.005).cuda()
    offset = torch.randint(-128, 127, (2, 1, 4, 9)).float().cuda()
    bs = [2, 6, 3, 1]
    q = affine.quantize(inp, scale, offset, 8, block_size=bs)
    dq = affine.dequantize(q, scale, offset, block_size=bs)
    qdq = affine.quantize_dequantize(inp, scale, offset, 8, block_size=bs)
    for i in range(2):
        for k in range(4):
            for l in range(0, 9, 4):
                sl = (Ellipsis, slice(i * 2, i * 2 + 2), slice(0, 6), slice(k * 3, k * 3 + 3), slice(l, l + 1))
                s, o = scale[i, 0, k, l], offset[i, 0, k, l]
                assert torch.equal(q[sl], affine.quantize(inp[sl], s, o, 8))
                assert torch.equal(dq[sl], affine.dequantize(q[sl], s, o))
                assert torch.equal(qdq[sl], affine.quantize_dequantize(inp[sl], s, o, 8))


def test_invalid_block_size(affine):
    # test_backend.py:718-740
    from aimet_amd.v2.quantization.affine.backends import hip_gfx950 as backend
    with pytest.raises(RuntimeError):
        backend._validate_arguments(torch.randn(4, 8), torch.randn(2, 2), torch.randn(2, 2), block_size=[2, 4, 1])
    backend._validate_arguments(torch.randn(4, 8), torch.randn(2, 2), torch.randn(2, 2), block_size=[2, 4])
    with pytest.raises(RuntimeError):
        backend._validate_arguments(torch.randn(1, 4), torch.randn(1, 3), torch.randn(1, 2), block_size=[1, -1])
    backend._validate_arguments(torch.randn(1, 4), torch.randn(1, 2), torch.randn(1, 2), block_size=[1, -1])
    with pytest.raises(RuntimeError):
        backend._validate_arguments(torch.randn(1, 4), torch.randn(1, 4), torch.randn(1, 2), block_size=[1, 3])
    backend._validate_arguments(torch.randn(1, 4), torch.randn(1, 2), torch.randn(1, 2), block_size=[1, 2])


@pytest.mark.parametrize("out_features,in_features,block", [(64, 512, 64), (48, 1024, 128), (16, 96, 16)])
def test_linear_weight_blocks_match_the_oracle_on_the_flat_channel_layout(affine, oracle, out_features, in_features,
                                                                          block):
    """[out, in] with scale [out, in / block]: no copy is made, and the result is the oracle's per-channel result
    with one channel per block."""
    torch.manual_seed(2)
    w = torch.randn(out_features, in_features) * 0.05
    nblk = in_features // block
    scale = w.reshape(out_features, nblk, block).abs().amax(dim=2) / 7
    offset = torch.zeros_like(scale)
    y = affine.quantize_dequantize(w.cuda(), scale.cuda(), offset.cuda(), -8, 7, block_size=(1, block))
    want, _, _ = oracle.v2_qdq(w.numpy().reshape(-1), out_features * nblk, block, scale.numpy().reshape(-1),
                               offset.numpy().reshape(-1), -8, 7)
    assert np.array_equal(y.cpu().numpy().reshape(-1).view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("shape,scale_shape,block_size", [
    ((32, 512), (32, 2), (1, 256)),            # runs of 256: the one-pass kernel
    ((8, 64), (8, 4), (1, 16)),                # short runs
    ((8, 6, 4), (4, 1, 2), (2, 6, 2)),         # blocks on several axes: permuted copy
    ((6, 5, 4), (6, 1, 4), None),              # scale varying along two non-adjacent axes, no blocks
])
def test_gradients_with_blocks_match_autograd(affine, shape, scale_shape, block_size):
    torch.manual_seed(3)
    x = torch.randn(*shape) * 2
    scale = torch.rand(scale_shape) * 0.02 + 0.01
    offset = torch.randint(-140, -110, scale_shape).float()
    g = torch.randn(*shape)
    xg, sg, og = (t.cuda().requires_grad_(True) for t in (x, scale, offset))
    y = affine.quantize_dequantize(xg, sg, og, 0, 255, block_size=block_size)
    y.backward(g.cuda())

    def expand(p):
        if block_size is None:
            return p
        for axis, d in enumerate(shape[len(shape) - len(scale_shape):]):
            p = p.repeat_interleave(d // scale_shape[axis], dim=axis)
        return p

    def ste_round(t):
        return t + (torch.round(t) - t).detach()
    xr, sr, orr = (t.double().requires_grad_(True) for t in (x, scale, offset))
    s_full, o_full = expand(sr), expand(orr)
    yr = (torch.clamp(ste_round(xr / s_full) - o_full, 0, 255) + o_full) * s_full
    yr.backward(g.double())
    assert torch.allclose(y.detach().cpu().double(), yr.detach(), rtol=1e-6, atol=1e-6)
    assert sg.grad.shape == scale.shape and og.grad.shape == offset.shape and xg.grad.shape == x.shape
    assert torch.equal(xg.grad.cpu() != 0, xr.grad != 0)
    assert torch.allclose(sg.grad.cpu().double(), sr.grad, rtol=1e-3, atol=1e-3)
    assert torch.allclose(og.grad.cpu().double(), orr.grad, rtol=1e-5, atol=1e-6)


def test_bq_compute_encodings_and_forward(affine):
    # test_affine_quantizer.py:958-977
    shape = (2, 2, 4)
    bq = affine.QuantizeDequantize(shape=shape, bitwidth=4, symmetric=True, block_size=(2, 4, 3)).cuda()
    assert bq.encoding_analyzer.observer.shape == (2, 1, 2, 1, 4, 1)
    bq.eval()
    torch.manual_seed(4)
    param_tensor = torch.randn(4, 8, 12).cuda()
    with bq.compute_encodings():
        _ = bq(param_tensor)
    out = bq(param_tensor)
    assert bq.get_min().shape == shape and out.shape == param_tensor.shape
    qdq_out = affine.quantize_dequantize(param_tensor, bq.get_scale(), bq.get_offset(), bq.qmin, bq.qmax,
                                         block_size=bq.block_size)
    assert torch.equal(out, qdq_out)
    # symmetric min-max calibration per block: the grid [-8, 7] * scale just covers the block's largest magnitude
    largest = param_tensor.reshape(2, 2, 2, 4, 4, 3).abs().amax(dim=(1, 3, 5))
    covered = torch.maximum(bq.get_max(), -bq.get_min())
    assert bool((covered >= largest * (1 - 1e-6)).all()) and bool((covered <= largest * (8 / 7) * (1 + 1e-6)).all())


@pytest.mark.parametrize('shape, block_sizes', [[(4, 1, 1), (1, 4, 4)], [(1, 4, 1), (4, 1, 4)], [(1, 1, 4), (4, 4, 1)]])
def test_bq_vs_per_channel_sanity(affine, shape, block_sizes):
    # test_affine_quantizer.py:979-1001
    bq = affine.QuantizeDequantize(shape=shape, bitwidth=4, symmetric=True, block_size=block_sizes).cuda().eval()
    pc = affine.QuantizeDequantize(shape=shape, bitwidth=4, symmetric=True).cuda().eval()
    torch.manual_seed(5)
    param_tensor = torch.randn(4, 4, 4).cuda()
    with bq.compute_encodings():
        _ = bq(param_tensor)
    with pc.compute_encodings():
        _ = pc(param_tensor)
    assert torch.equal(bq(param_tensor), pc(param_tensor))


def test_sqnr_analyzer_on_a_shape_that_is_not_made_of_slabs(oracle):
    """Histograms per channel along axis 1 of [N, C, H, W]: every channel's values are gathered by one copy."""
    from aimet_amd.v2.quantization.encoding_analyzer import SqnrEncodingAnalyzer
    from oracle import sqnr_oracle as sq
    torch.manual_seed(6)
    x = torch.randn(4, 3, 20, 20) * torch.tensor([1.0, 3.0, 0.2]).view(1, 3, 1, 1)
    an = SqnrEncodingAnalyzer((1, 3, 1, 1), num_bins=256)
    an.update_stats(x.cuda())
    mn, mx = an.compute_encodings(255, False)
    assert mn.shape == (1, 3, 1, 1)
    for c in range(3):
        ref = sq.SqnrAnalyzer(1, num_bins=256)
        ref.update_stats(x[:, c].contiguous())
        rmin, rmax, _ = ref.compute_encodings(255, False)
        assert torch.allclose(mn[0, c, 0, 0].cpu(), rmin.reshape(()), rtol=1e-6)
        assert torch.allclose(mx[0, c, 0, 0].cpu(), rmax.reshape(()), rtol=1e-6)
