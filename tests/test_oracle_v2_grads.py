"""Pins the restatement of the v2 quantize-dequantize backward (all three gradients) in the CPU oracle.

The reference's own check for these gradients is a comparison with torch autograd on the textbook expression
(TrainingExtensions/torch/test/python/v2/quantization/affine/backends/test_backend.py:200-215, 598-625, rtol 1e-3);
the same independent derivation is used here, in float64, plus cases whose answer is known in closed form."""
import numpy as np
import pytest
import torch

from oracle import lib as oracle


def _ste_round(t):
    return t + (torch.round(t) - t).detach()


def _autograd(x, g, scale, offset, qmin, qmax, shape):
    """Gradients of (clamp(round(x/s) - round(o), qmin, qmax) + round(o)) * s from autograd, in float64."""
    x = torch.tensor(x, dtype=torch.float64, requires_grad=True)
    s = torch.tensor(scale, dtype=torch.float64).reshape(shape).requires_grad_()
    o = torch.tensor(offset, dtype=torch.float64).reshape(shape).requires_grad_()
    y = (torch.clamp(_ste_round(x / s) - _ste_round(o), qmin, qmax) + _ste_round(o)) * s
    y.backward(torch.tensor(g, dtype=torch.float64))
    return x.grad.numpy(), s.grad.reshape(-1).numpy(), o.grad.reshape(-1).numpy()


def _round_safe(rng, shape, scale, lo, hi):
    """Values whose quotient by the scale stays away from rounding ties and from the edges of the clamp."""
    k = rng.integers(lo, hi, shape)
    frac = rng.uniform(-0.35, 0.35, shape)
    return ((k + frac) * scale).astype(np.float32)


@pytest.mark.parametrize("qmin,qmax", [(0, 255), (-128, 127), (-8, 7)])
@pytest.mark.parametrize("per_channel", [False, True])
def test_all_three_gradients_match_autograd(qmin, qmax, per_channel):
    rng = np.random.default_rng(qmax + per_channel)
    c, npc = (6, 40) if per_channel else (1, 240)
    shape = (c, 1) if per_channel else ()
    scale = rng.uniform(0.01, 0.2, c).astype(np.float32)
    offset = np.round(rng.uniform(-5, 5, c)).astype(np.float32)
    # a third of the values fall outside the grid on either side
    span = qmax - qmin
    x = _round_safe(rng, (c, npc), scale[:, None], qmin - span // 3, qmax + span // 3) + (offset * scale)[:, None]
    x = x.astype(np.float32)
    g = rng.standard_normal((c, npc)).astype(np.float32)
    gin, sg, og = oracle.v2_qdq_bwd_params(x, g, c, npc, scale, offset, qmin, qmax)
    egx, esg, eog = _autograd(x if per_channel else x.reshape(-1), g if per_channel else g.reshape(-1), scale, offset,
                              qmin, qmax, shape)
    assert 0.2 < (gin != 0).mean() < 0.9                        # both branches of the mask are exercised
    assert np.allclose(gin.reshape(egx.shape), egx, rtol=0, atol=0)
    assert np.allclose(sg, esg, rtol=1e-3, atol=1e-3)
    assert np.allclose(og, eog, rtol=1e-6, atol=1e-6)


def test_closed_forms():
    # every value inside the grid and exactly on it: x = k * s -> rounding residual 0, so scale_grad = 0 and
    # offset_grad = 0, whatever the incoming gradient
    s, o = np.array([0.25], np.float32), np.array([-3.0], np.float32)
    k = np.arange(-3, 13).astype(np.float32)
    g = np.linspace(-1, 1, k.size).astype(np.float32)
    gin, sg, og = oracle.v2_qdq_bwd_params(k * s, g, 1, k.size, s, o, 0, 15)
    assert np.array_equal(gin, g) and sg[0] == 0.0 and og[0] == 0.0
    # every value above the grid: y = (qmax + o) * s, so dy/ds = qmax + o, dy/do = s, dy/dx = 0
    x = np.full(8, 100.0, np.float32)
    g = np.arange(1, 9).astype(np.float32)
    gin, sg, og = oracle.v2_qdq_bwd_params(x, g, 1, 8, s, o, 0, 15)
    assert not gin.any() and sg[0] == g.sum() * (15 - 3) and og[0] == g.sum() * 0.25
    # every value below the grid: dy/ds = qmin + o
    gin, sg, og = oracle.v2_qdq_bwd_params(-x, g, 1, 8, s, o, 0, 15)
    assert not gin.any() and sg[0] == g.sum() * (0 - 3) and og[0] == g.sum() * 0.25
    # inside the grid, off the grid points: dy/ds = round(x/s) - x/s
    x = np.array([0.3, -0.6, 1.1], np.float32)
    g = np.ones(3, np.float32)
    _, sg, og = oracle.v2_qdq_bwd_params(x, g, 1, 3, s, o, 0, 15)
    q = x / s
    assert sg[0] == pytest.approx(float((np.rint(q) - q).astype(np.float64).sum()), abs=1e-12) and og[0] == 0.0


def test_channel_layout_with_outer_dimension():
    # [outer][channel][row]: the sums of a channel run over every outer index
    rng = np.random.default_rng(3)
    outer, c, npc = 4, 3, 10
    scale = np.array([0.1, 0.2, 0.05], np.float32)
    offset = np.array([-2.0, 0.0, 3.0], np.float32)
    x = rng.standard_normal((outer, c, npc)).astype(np.float32)
    g = rng.standard_normal((outer, c, npc)).astype(np.float32)
    gin, sg, og = oracle.v2_qdq_bwd_params(x, g, c, npc, scale, offset, -8, 7)
    for ch in range(c):
        gi, s1, o1 = oracle.v2_qdq_bwd_params(np.ascontiguousarray(x[:, ch]), np.ascontiguousarray(g[:, ch]), 1,
                                              outer * npc, scale[ch:ch + 1], offset[ch:ch + 1], -8, 7)
        assert np.array_equal(gi.reshape(outer, npc), gin.reshape(outer, c, npc)[:, ch])
        assert s1[0] == pytest.approx(sg[ch], rel=1e-12) and o1[0] == pytest.approx(og[ch], rel=1e-12)
