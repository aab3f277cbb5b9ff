"""GPU tests of the v2 host-side interface: backend functions, QuantizeDequantize / Quantize modules and the min-max
encoding analyzer, against the CPU oracle and against textbook autograd of the straight-through formula.

Cases follow TrainingExtensions/torch/test/python/v2/quantization/affine/test_affine_quantizer.py and
.../backends/test_backend.py of the reference: error behaviour of the backend functions, forward values, gradients
w.r.t. input / scale / offset (min / max), dynamic quantization inside compute_encodings().
"""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def v2():
    from aimet_amd.v2.quantization import affine
    from aimet_amd.v2.quantization.affine import backends

    class V2:
        pass
    a = V2()
    a.affine, a.backends = affine, backends
    return a


def _ste_reference(x, scale, offset, qmin, qmax):
    """(clamp(ste_round(x / s) - ste_round(o), qmin, qmax) + o) * s with autograd's own derivative of every op."""
    def ste_round(t):
        return t + (torch.round(t) - t).detach()
    q = torch.clamp(ste_round(x / scale) - offset, qmin, qmax)
    return (q + offset) * scale


@pytest.mark.parametrize("shape,scale_shape", [((64, 33), ()), ((16, 24), (16, 1)), ((6, 5, 3, 3), (1, 5, 1, 1))])
def test_backend_quantize_dequantize_and_grads(v2, oracle, shape, scale_shape):
    torch.manual_seed(4)
    x = torch.randn(*shape) * 2
    scale = torch.rand(scale_shape) * 0.02 + 0.01
    offset = torch.randint(-140, -110, scale_shape).float()
    qmin, qmax = 0, 255
    xg = x.cuda().requires_grad_(True)
    sg = scale.cuda().requires_grad_(True)
    og = offset.cuda().requires_grad_(True)
    y = v2.backends.quantize_dequantize(xg, sg, og, qmin, qmax)
    # forward: identical to the oracle
    num_channel = max(1, scale.numel())
    axis = [i for i, d in enumerate(scale_shape) if d != 1]
    npc = int(np.prod(shape[axis[0] + 1:])) if axis else x.numel()
    want = oracle.v2_qdq(x.numpy().reshape(-1), num_channel, npc, scale.numpy().reshape(-1),
                         offset.numpy().reshape(-1), qmin, qmax)
    want = want[0] if isinstance(want, tuple) else want
    assert np.array_equal(y.detach().cpu().numpy().reshape(-1), want)
    g = torch.randn(*shape)
    y.backward(g.cuda())
    xr, sr, orr = x.clone().requires_grad_(True), scale.clone().requires_grad_(True), \
        offset.clone().requires_grad_(True)
    _ste_reference(xr, sr, orr, qmin, qmax).backward(g)
    # the kernel returns grad * mask exactly; autograd of the formula computes (grad * s) / s, one rounding off
    assert torch.equal(xg.grad.cpu() == 0, xr.grad == 0)
    assert torch.allclose(xg.grad.cpu(), xr.grad, rtol=3e-7, atol=0)
    assert torch.equal(xg.grad.cpu()[xr.grad != 0], g[xr.grad != 0])
    assert torch.allclose(sg.grad.cpu(), sr.grad, rtol=1e-4, atol=1e-4)
    assert torch.allclose(og.grad.cpu(), orr.grad, rtol=1e-4, atol=1e-5)


def test_backend_quantize_and_dequantize(v2):
    torch.manual_seed(6)
    x = (torch.randn(50, 20) * 3).cuda()
    scale = torch.tensor(0.05).cuda()
    offset = torch.tensor(-7.0).cuda()
    q = v2.backends.quantize(x, scale, offset, -8, 7)
    want = torch.clamp(torch.round(x / scale) - offset, -8, 7)
    assert torch.equal(q, want)
    dq = v2.backends.dequantize(q, scale, offset)
    assert torch.equal(dq, v2.backends.quantize_dequantize(x, scale, offset, -8, 7))


def test_backend_errors(v2):
    """test_backend.py of the reference: shape, device and grid checks raise RuntimeError."""
    x = torch.randn(4, 6).cuda()
    s, o = torch.tensor(0.1).cuda(), torch.tensor(0.0).cuda()
    with pytest.raises(RuntimeError):
        v2.backends.quantize_dequantize(x, torch.ones(5).cuda(), o, 0, 255)          # not expandable
    with pytest.raises(RuntimeError):
        v2.backends.quantize_dequantize(x, s.cpu(), o, 0, 255)                       # device mismatch
    with pytest.raises(RuntimeError):
        v2.backends.quantize_dequantize(x, s, o, 10, 5)                              # qmin > qmax
    with pytest.raises(RuntimeError):
        v2.backends.quantize(x.to(torch.bfloat16), s, o, 0, 2 ** 16 - 1)             # grid not representable
    with pytest.raises(RuntimeError):
        v2.backends.quantize_dequantize(x.cpu(), s.cpu(), o.cpu(), 0, 255)           # no CPU compute path
    with pytest.raises(RuntimeError):
        v2.backends.set_global_backend("torch_builtins")
    assert v2.backends.get_backend().__name__.endswith("hip_gfx950")


@pytest.mark.parametrize("symmetric", [False, True])
def test_quantize_dequantize_module(v2, symmetric):
    torch.manual_seed(8)
    qdq = v2.affine.QuantizeDequantize((), bitwidth=8, symmetric=symmetric).cuda()
    x = torch.randn(100, 30).cuda() * 1.7 + (0 if symmetric else 0.4)
    with pytest.raises(RuntimeError):
        qdq(x)                                   # not initialised
    with qdq.compute_encodings():
        y_dyn = qdq(x)                           # dynamic quantization with the batch's own statistics
    assert qdq.is_initialized()
    mn, mx = x.min().item(), x.max().item()
    if symmetric:
        # symmetric grid of 255 steps: scale = max(|min|, |max|) / 127.5 ... (MinMaxEncodingAnalyzer)
        assert qdq.get_max().item() > 0 and qdq.get_offset().item() == 0
    else:
        assert qdq.get_min().item() <= min(mn, 0) + qdq.get_scale().item()
        assert qdq.get_max().item() >= max(mx, 0) - qdq.get_scale().item()
    y = qdq(x)
    assert torch.equal(y, y_dyn)
    err = (y - x).abs().max().item()
    assert err <= qdq.get_scale().item() * 0.5 + 1e-6
    # gradients reach min and max (range learning)
    x.requires_grad_(True)
    qdq(x).sum().backward()
    assert qdq.min.grad is not None and qdq.max.grad is not None and x.grad is not None


def test_per_channel_module(v2, oracle):
    torch.manual_seed(9)
    w = torch.randn(12, 20).cuda() * torch.linspace(0.1, 2, 12).cuda().unsqueeze(1)
    qdq = v2.affine.QuantizeDequantize((12, 1), bitwidth=4, symmetric=True).cuda()
    with qdq.compute_encodings():
        qdq(w)
    y = qdq(w)
    scale, offset = qdq.get_scale().detach(), qdq.get_offset().detach()
    want = oracle.v2_qdq(w.cpu().numpy().reshape(-1), 12, 20, scale.cpu().numpy().reshape(-1),
                         offset.cpu().numpy().reshape(-1), qdq.qmin, qdq.qmax)
    want = want[0] if isinstance(want, tuple) else want
    assert np.array_equal(y.detach().cpu().numpy().reshape(-1), want)
    # every row uses its own grid
    assert torch.unique(scale).numel() == 12
