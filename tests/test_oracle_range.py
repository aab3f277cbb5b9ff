"""Pins oracle/range_oracle.py, the CPU restatement of range learning's parameter-sized arithmetic (runs without a GPU).

The v2 gradients: float64 autograd of the reference's own expressions (get_scale / get_offset with a straight-through
round, then the quantize-dequantize formula), the check the reference itself uses for gradients
(TrainingExtensions/torch/test/python/v2/ab_test/test_quantsim_qat.py:174-203).  A dropped term, a wrong sign or a
swapped min / max in the formulas fails it: min enters through scale and through offset, max through scale only.
The v1 grid: what get_computed_encodings exists for -- zero is a grid point and the grid covers [min, max] to within
one step.  The ordering of the range: its three stated invariants.
"""
import numpy as np
import pytest
import torch

from oracle import lib as oracle
from oracle import range_oracle


def _ste_round(t):
    return t + (torch.round(t) - t).detach()


def _autograd_v2(x, g, enc_min, enc_max, qmin, qmax, symmetric):
    """d/dmin, d/dmax of sum(g * qdq(x)) by autograd in float64, per channel (x, g: [C, N])."""
    x, g = torch.tensor(x, dtype=torch.float64), torch.tensor(g, dtype=torch.float64)
    mn = torch.tensor(enc_min, dtype=torch.float64).reshape(-1, 1).requires_grad_()
    mx = torch.tensor(enc_max, dtype=torch.float64).reshape(-1, 1).requires_grad_()
    scale = (mx - mn) / (qmax - qmin)
    offset = torch.zeros_like(mn) if symmetric else _ste_round(mn / scale) - qmin
    y = (torch.clamp(_ste_round(x / scale) - offset, qmin, qmax) + offset) * scale
    (y * g).sum().backward()
    return mn.grad.reshape(-1).numpy(), mx.grad.reshape(-1).numpy()


@pytest.mark.parametrize("symmetric", (False, True))
@pytest.mark.parametrize("qmin,qmax", ((0, 255), (-128, 127), (0, 15)))
@pytest.mark.parametrize("divide", (True, False))
def test_v2_range_gradients_match_autograd(symmetric, qmin, qmax, divide):
    rng = np.random.default_rng(qmax + 7 * symmetric)
    c, n = 5, 4000
    enc_min = -rng.uniform(0.5, 2.0, c).astype(np.float32)
    enc_max = rng.uniform(0.5, 2.0, c).astype(np.float32)
    if symmetric:
        enc_min = (-enc_max * np.float32(-qmin) / np.float32(qmax)).astype(np.float32) if qmin < 0 else -enc_max
    x = (rng.standard_normal((c, n)) * 1.2).astype(np.float32)     # a good part falls outside on both sides
    g = rng.standard_normal((c, n)).astype(np.float32)
    scale, offset = range_oracle.grid_v2(enc_min, enc_max, qmin, qmax, symmetric, divide)
    gin, sum_s, sum_o = oracle.v2_qdq_bwd_params(x, g, c, n, scale, offset, qmin, qmax)
    assert 0.3 < (gin != 0).mean() < 0.97
    got_min, got_max = range_oracle.range_grads_v2(sum_s, sum_o, enc_min, scale, qmin, qmax, symmetric, divide)
    want_min, want_max = _autograd_v2(x, g, enc_min, enc_max, qmin, qmax, symmetric)
    scale_of = np.abs(want_max).max()
    assert np.allclose(got_max, want_max, rtol=2e-3, atol=2e-3 * scale_of)
    assert np.allclose(got_min, want_min, rtol=2e-3, atol=2e-3 * scale_of)
    assert np.abs(want_min + want_max).max() > 1e-3 * scale_of or symmetric     # min is more than "minus max"


def test_v2_grid_forms():
    mn, mx = np.array([-1.0, -0.3, 0.25], np.float32), np.array([1.0, 2.25, 0.75], np.float32)
    scale, offset = range_oracle.grid_v2(mn, mx, 0, 255, False)
    assert np.array_equal(scale, ((mx - mn) / np.float32(255)).astype(np.float32))
    assert np.array_equal(offset, np.rint(mn / scale))
    # the range the grid spans starts at scale * offset: within half a step of min
    assert np.all(np.abs(scale * offset - mn) <= scale / 2 + 1e-7)
    scale_s, offset_s = range_oracle.grid_v2(-mx, mx, -128, 127, True)
    assert not offset_s.any() and np.array_equal(scale_s, ((mx + mx) / np.float32(255)).astype(np.float32))
    by_product, _ = range_oracle.grid_v2(mn, mx, 0, 255, False, divide=False)
    assert np.all(np.abs(by_product.view(np.int32) - scale.view(np.int32)) <= 1)       # one ulp apart at most


@pytest.mark.parametrize("bitwidth", (4, 8, 16))
def test_v1_grid_holds_zero_and_covers_the_range(bitwidth):
    rng = np.random.default_rng(bitwidth)
    mn = -rng.uniform(0.0, 3.0, 200).astype(np.float32)
    mx = rng.uniform(0.01, 3.0, 200).astype(np.float32)
    delta, offset, steps = range_oracle.grid_v1(mn, mx, bitwidth, False, False, False)
    assert steps == 2 ** bitwidth - 1
    assert np.array_equal(offset, np.rint(offset)) and np.all(offset <= 0) and np.all(offset >= -steps)   # zero point
    # (in float64; delta carries a float32 rounding of its own, which 65535 steps multiply)
    low, high = delta.astype(np.float64) * offset, delta.astype(np.float64) * (offset + float(steps))
    assert np.all(np.abs(low - mn) <= delta * 0.51) and np.all(np.abs(high - mx) <= delta * 0.51)
    # signed symmetric: max / floor(steps / 2), offset -ceil(steps / 2); strict symmetric has one step less
    delta, offset, steps = range_oracle.grid_v1(-mx, mx, bitwidth, True, False, False)
    assert np.array_equal(delta, (mx / np.float32(2 ** (bitwidth - 1) - 1)).astype(np.float32))
    assert np.all(offset == -(2 ** (bitwidth - 1)))
    delta, offset, steps = range_oracle.grid_v1(-mx, mx, bitwidth, True, True, False)
    assert steps == 2 ** bitwidth - 2 and np.all(offset == -(2 ** (bitwidth - 1) - 1))
    # unsigned symmetric: an unrounded offset min / delta
    delta, offset, _ = range_oracle.grid_v1(mn, mx, bitwidth, True, False, True)
    assert np.array_equal(offset, (mn / delta).astype(np.float32))


def test_v1_range_gradient_forms():
    s, o = np.array([3.0, -2.0], np.float32), np.array([0.5, 0.25], np.float32)
    mn, mx = np.array([-1.0, -2.0], np.float32), np.array([1.0, 2.0], np.float32)
    gmin, gmax = range_oracle.range_grads_v1(s, o, mn, mx, 255, True)
    assert np.array_equal(gmax, (s / np.float32(127)).astype(np.float32)) and np.array_equal(gmin, -gmax)
    gmin, gmax = range_oracle.range_grads_v1(s, o, mn, mx, 255, False)
    t1, t2 = s / np.float32(255), np.float32(255) / ((mx - mn) ** 2) * o
    assert np.allclose(gmin, -t1 + mx * t2, rtol=1e-6) and np.allclose(gmax, t1 - mn * t2, rtol=1e-6)
    # nothing clipped (sum_o = 0): the two gradients are opposite
    gmin, gmax = range_oracle.range_grads_v1(s, np.zeros(2, np.float32), mn, mx, 255, False)
    assert np.array_equal(gmin, -gmax)


def test_ordering_of_the_range():
    mn = np.array([-1.0, 0.5, -2.0, 0.0, -1e-7, np.nan, -3.0, 2.0], np.float32)
    mx = np.array([2.0, 1.5, -1.0, 0.0, 1e-7, 1.0, np.nan, 1.0], np.float32)
    got_min, got_max = range_oracle.ordered_range(mn, mx)
    ok = ~(np.isnan(got_min) | np.isnan(got_max))
    assert np.all(got_min[ok] <= 0) and np.all(got_max[ok] >= 0)
    assert np.all(got_max[ok] >= got_min[ok] + np.float32(1e-5))
    assert np.isnan(got_min[5]) and np.isnan(got_max[5]) and np.isnan(got_max[6]) and got_min[6] == -3.0
    untouched = [0, 2]
    assert got_min[0] == -1.0 and got_max[0] == 2.0 and got_min[2] == -2.0 and got_max[2] == 0.0 and untouched
