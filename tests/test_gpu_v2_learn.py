"""GPU parity of the one-pass v2 backward (input, scale and offset gradients) against the CPU oracle, through the
C ABI.  tensor_grad is bit-identical; the two parameter gradients are sums of float32 terms whose order the
reference leaves to autograd, so they are compared with the oracle's double-precision sum of the same terms at
rtol 2e-5 of the sum of the terms' magnitudes (float32 partial sums over at most 8192 elements)."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _gpu(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


@pytest.fixture(scope="module")
def ops():
    from aimet_amd import ops as o
    return o


def _case(seed, outer, c, npc, qmin, qmax):
    rng = np.random.default_rng(seed)
    n = outer * c * npc
    scale = (np.abs(rng.standard_normal(c)) * 0.01 + 2e-3).astype(np.float32)
    offset = -np.round(rng.uniform(0, qmax, c)).astype(np.float32) if qmin == 0 else np.zeros(c, np.float32)
    x = (rng.standard_normal(n) * 0.5).astype(np.float32)
    t = min(64, n)
    x[:t] = (scale[0] * (np.arange(t) - 32 + 0.5)).astype(np.float32)   # rounding ties
    g = rng.standard_normal(n).astype(np.float32)
    return x, g, scale, offset


def _check_sums(got, want, x, g, c, npc, scale, offset, qmin, qmax, oracle):
    # the yardstick of the tolerance: per channel, the sum of the magnitudes of the terms that were added
    xs = x.astype(np.float64).reshape(-1, c, npc)
    ga = np.abs(g.astype(np.float64)).reshape(-1, c, npc)
    s, o = scale.astype(np.float64).reshape(1, c, 1), offset.astype(np.float64).reshape(1, c, 1)
    with np.errstate(all="ignore"):
        q = xs / s
        r = np.rint(q)
        mask = (qmin <= r - o) & (r - o <= qmax)
        mag_s = np.nansum(ga * np.abs(np.clip(r, o + qmin, o + qmax) - np.where(mask, q, 0.0)), axis=(0, 2))
        mag_o = np.nansum(ga * np.where(mask, 0.0, s), axis=(0, 2))
    for k, (a, b, m) in enumerate(zip(got, want, (mag_s + 1e-3, mag_o + 1e-6))):
        assert np.all(np.abs(a.astype(np.float64) - b) <= 2e-5 * m), (k, np.abs(a - b).max(), m.min())


@pytest.mark.parametrize("qmin,qmax", [(0, 255), (-8, 7)])
@pytest.mark.parametrize("outer,c,npc", [
    (1, 1, 100003),        # per-tensor, odd length: scalar path
    (1, 1, 1 << 21),       # per-tensor, several spans
    (1, 1, 12),            # smaller than one vector step
    (1, 512, 4608),        # weight rows
    (1, 64, 1030),         # rows that are no multiple of the vector width
    (8, 32, 784),          # activations per channel: the sums run over the outer dimension
    (3, 7, 5),             # tiny rows
    (1, 4096, 128),        # blockwise weight: 32 lanes per row, sums stored directly
    (1, 8192, 64),         # 16 lanes per row
    (1, 1000, 16),         # 4 lanes per row, row count no multiple of the rows per workgroup
    (5, 300, 36),          # 3x3 kernels of 4 input channels, activations-style outer dimension
    (1, 333, 9),           # odd rows: one element per lane
    (2, 40, 2048),         # the longest row the lane-group kernel takes
    (2, 40, 2052),         # the shortest row the workgroup kernel takes
    (1, 3, 8192 + 2048 + 4),   # last span of a row much shorter than the others
])
def test_bwd_params_matches_oracle(ops, oracle, qmin, qmax, outer, c, npc):
    x, g, scale, offset = _case(qmax + c + npc, outer, c, npc, qmin, qmax)
    gin, sg, og = ops.v2_qdq_bwd_params(_gpu(x), _gpu(g), c, npc, _gpu(scale), _gpu(offset), qmin, qmax)
    want_gin, want_sg, want_og = oracle.v2_qdq_bwd_params(x, g, c, npc, scale, offset, qmin, qmax)
    assert np.array_equal(gin.cpu().numpy().view(np.uint32), want_gin.view(np.uint32))
    # and equal to the kernel that only forms tensor_grad
    only = ops.v2_qdq_bwd(_gpu(x), _gpu(g), c, npc, _gpu(scale), _gpu(offset), qmin, qmax)
    assert torch.equal(only, gin)
    _check_sums((sg.cpu().numpy(), og.cpu().numpy()), (want_sg, want_og), x, g, c, npc, scale, offset, qmin, qmax,
                oracle)
    # without tensor_grad the sums are the same bits
    none, sg2, og2 = ops.v2_qdq_bwd_params(_gpu(x), _gpu(g), c, npc, _gpu(scale), _gpu(offset), qmin, qmax,
                                           want_grad_in=False)
    assert none is None and torch.equal(sg, sg2) and torch.equal(og, og2)


def test_bwd_params_is_deterministic(ops):
    x, g, scale, offset = _case(5, 4, 16, 3000, -128, 127)
    a = ops.v2_qdq_bwd_params(_gpu(x), _gpu(g), 16, 3000, _gpu(scale), _gpu(offset), -128, 127)
    b = ops.v2_qdq_bwd_params(_gpu(x), _gpu(g), 16, 3000, _gpu(scale), _gpu(offset), -128, 127)
    assert all(torch.equal(u, v) for u, v in zip(a, b))


@pytest.mark.parametrize("c,npc", [(48, 2048), (24, 4096), (512, 64), (100, 24)])
def test_bwd_params_bf16(ops, oracle, c, npc):
    x, g, scale, offset = _case(11, 1, c, npc, -128, 127)
    xb, gb = torch.from_numpy(x).to(torch.bfloat16), torch.from_numpy(g).to(torch.bfloat16)
    gin, sg, og = ops.v2_qdq_bwd_params(xb.cuda(), gb.cuda(), c, npc, _gpu(scale), _gpu(offset), -128, 127)
    x32, g32 = xb.float().numpy(), gb.float().numpy()
    want_gin, want_sg, want_og = oracle.v2_qdq_bwd_params(x32, g32, c, npc, scale, offset, -128, 127)
    assert gin.dtype == torch.bfloat16
    assert np.array_equal(gin.float().cpu().numpy(), want_gin)          # grad * {0, 1} is exact in bf16
    _check_sums((sg.cpu().numpy(), og.cpu().numpy()), (want_sg, want_og), x32, g32, c, npc, scale, offset, -128, 127,
                oracle)


def test_bwd_params_non_finite_and_huge_values(ops, oracle):
    # the exact-division fast path is left for vectors holding huge values; NaN terms propagate into the sums
    c, npc = 2, 4096
    x, g, scale, offset = _case(2, 1, c, npc, 0, 255)
    x[5], x[9] = 3.0e30, -2.0e25                       # channel 0: finite sums, slow division path
    x[npc + 7] = np.nan                                # channel 1: NaN sums
    gin, sg, og = ops.v2_qdq_bwd_params(_gpu(x), _gpu(g), c, npc, _gpu(scale), _gpu(offset), 0, 255)
    want_gin, want_sg, want_og = oracle.v2_qdq_bwd_params(x, g, c, npc, scale, offset, 0, 255)
    assert np.array_equal(gin.cpu().numpy().view(np.uint32), want_gin.view(np.uint32))
    assert np.isnan(want_sg[1]) and torch.isnan(sg[1]).item()
    assert np.isclose(sg[0].item(), want_sg[0], rtol=2e-5) and np.isclose(og[0].item(), want_og[0], rtol=2e-5)
    assert og[1].item() == pytest.approx(want_og[1], rel=2e-5)     # NaN is outside the grid: the term is grad * scale


def test_bwd_params_empty_and_bad_arguments(ops):
    from aimet_amd._lib import MiqError
    e = torch.empty(0, device="cuda")
    one = torch.ones(1, device="cuda")
    gin, sg, og = ops.v2_qdq_bwd_params(e, e, 1, 1, one, one * 0, 0, 255)
    assert gin.numel() == 0 and sg.item() == 0.0 and og.item() == 0.0
    x = torch.randn(100, device="cuda")
    with pytest.raises(MiqError):
        ops.v2_qdq_bwd_params(x, x, 3, 7, torch.ones(3, device="cuda"), torch.zeros(3, device="cuda"), 0, 255)
    with pytest.raises(MiqError):
        ops.v2_qdq_bwd_params(x, x, 1, 100, one, one * 0, 5, 4)


@pytest.mark.parametrize("shape,scale_shape", [((4096,), ()), ((8, 512), (8, 1)), ((4, 6, 16, 16), (1, 6, 1, 1))])
def test_backend_routes_learnable_parameters_through_the_one_pass_kernel(shape, scale_shape):
    """quantize_dequantize with scale / offset that require grad: gradients against torch autograd of the textbook
    expression (the reference's own check, test_backend.py:598-625, rtol 1e-3)."""
    from aimet_amd.v2.quantization.affine import backends
    torch.manual_seed(8)
    x = torch.randn(*shape) * 2
    scale = torch.rand(scale_shape) * 0.02 + 0.01
    offset = torch.randint(-140, -110, scale_shape).float()
    g = torch.randn(*shape)
    xg, sg, og = (t.cuda().requires_grad_(True) for t in (x, scale, offset))
    backends.quantize_dequantize(xg, sg, og, 0, 255).backward(g.cuda())

    def ste_round(t):
        return t + (torch.round(t) - t).detach()
    xr, sr, orr = (t.double().requires_grad_(True) for t in (x, scale, offset))
    ((torch.clamp(ste_round(xr / sr) - orr, 0, 255) + orr) * sr).backward(g.double())
    assert sg.grad.shape == scale.shape and og.grad.shape == offset.shape
    assert torch.equal(xg.grad.cpu() != 0, xr.grad != 0)
    assert torch.allclose(sg.grad.cpu().double(), sr.grad, rtol=1e-3, atol=1e-3)
    assert torch.allclose(og.grad.cpu().double(), orr.grad, rtol=1e-5, atol=1e-6)
