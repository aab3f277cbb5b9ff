"""Range learning without the parameter-sized tensor operations: the grid (scale, offset) made from a learnable encoding
min / max by one launch, and the gradients of min / max written by the backward's reduction kernel.

The checks: the grid against the tensor operations it replaces, on the same GPU, to the bit (v2:
QuantizeDequantize.get_scale() / get_offset(); v1: get_computed_encodings() and the wrappers' ordering of the range);
the encoding gradients against the formulas applied to the channel sums of miq_v2_qdq_bwd_params_*, to the bit, over
the layouts that take different kernels (one workgroup per channel, several, short rows, an outer dimension); and the
v2 quantizer modules and v1 wrappers with the fused path against themselves with it switched off.
"""
import numpy as np
import pytest
import torch
from torch import nn

pytestmark = pytest.mark.gpu


def _bits(t):
    return t.contiguous().view(torch.int32)


def _same(a, b):
    """Equal to the bit (signed zeros included) where they are numbers, NaN in the same places."""
    nan_a, nan_b = torch.isnan(a), torch.isnan(b)
    zero = torch.zeros_like(a)
    return a.shape == b.shape and torch.equal(nan_a, nan_b) and \
        torch.equal(_bits(torch.where(nan_a, zero, a)), _bits(torch.where(nan_b, zero, b)))


def _ranges(c, seed):
    g = torch.Generator().manual_seed(seed)
    mn = -torch.rand(c, generator=g) * 3 - 0.01
    mx = torch.rand(c, generator=g) * 3 + 0.01
    return mn.cuda(), mx.cuda()


# ------------------------------------------------------------------------------------------------------- the grid
@pytest.mark.parametrize("symmetric", (False, True))
@pytest.mark.parametrize("qmin,qmax", ((0, 255), (-128, 127), (-8, 7), (0, 65535)))
def test_v2_grid_equals_get_scale_and_get_offset(symmetric, qmin, qmax):
    from aimet_amd import ops
    from aimet_amd.v2.quantization.affine import QuantizeDequantize
    for c in (1, 7, 300):
        mn, mx = _ranges(c, 10 + c)
        if c == 7:
            mn[2], mx[2] = 0.25, 0.75                               # a range that does not hold zero
            mn[3] = mx[3]                                           # no width: scale 0, offset NaN
        q = QuantizeDequantize((c,), qmin, qmax, symmetric).cuda()
        q.set_range(mn, mx)
        mode = ops.RANGE_V2_SYMMETRIC if symmetric else ops.RANGE_V2_ASYMMETRIC
        grid = ops.range_to_grid(q.min.detach(), q.max.detach(), qmin, qmax, mode)
        assert _same(grid[0], q.get_scale().detach())
        assert _same(grid[1], q.get_offset().detach())
        assert _same(grid[2], mn) and _same(grid[3], mx)


@pytest.mark.parametrize("bitwidth", (4, 8, 16))
@pytest.mark.parametrize("symmetric,strict,unsigned", ((False, False, False), (True, False, False),
                                                       (True, True, False), (True, False, True)))
def test_v1_grid_equals_get_computed_encodings(bitwidth, symmetric, strict, unsigned):
    from aimet_amd import ops
    from aimet_amd.v1 import quantsim_straight_through_grad as ste
    steps = 2 ** bitwidth - 1 - (1 if symmetric and strict else 0)
    mode = ops.RANGE_V1_ASYMMETRIC if not symmetric else \
        (ops.RANGE_V1_UNSIGNED_SYMMETRIC if unsigned else ops.RANGE_V1_SIGNED_SYMMETRIC)
    for c in (1, 9, 513):
        mn, mx = _ranges(c, 20 + c)
        if c == 9:
            mn[1], mx[1] = 0.0, 0.0
            mn[2] = float("nan")
            mx[4] = float("inf")
        delta, offset, _ = ste.get_computed_encodings(bitwidth, mn, mx, symmetric, strict, unsigned)
        grid = ops.range_to_grid(mn.clone(), mx.clone(), 0, steps, mode)
        assert _same(grid[0], delta)
        assert _same(grid[1], offset)


def test_ordering_of_the_range_in_place():
    from aimet_amd import ops
    from aimet_amd.v1.tensor_quantizer import set_encoding_min_max_gating_threshold
    mn = torch.tensor([-1.0, 0.5, -2.0, 0.0, -1e-7, float("nan"), -3.0, 2.0]).cuda()
    mx = torch.tensor([2.0, 1.5, -1.0, 0.0, 1e-7, 1.0, float("nan"), 1.0]).cuda()
    want_min, want_max = nn.Parameter(mn.clone()), nn.Parameter(mx.clone())
    set_encoding_min_max_gating_threshold(want_min, want_max)
    got_min, got_max = nn.Parameter(mn.clone()), nn.Parameter(mx.clone())
    versions = got_min._version, got_max._version
    grid = ops.range_to_grid(got_min.detach(), got_max.detach(), 0, 255, ops.RANGE_V1_ASYMMETRIC, gate=True)
    assert _same(got_min.detach(), want_min.detach()) and _same(got_max.detach(), want_max.detach())
    assert got_min._version > versions[0] and got_max._version > versions[1]
    assert _same(grid[2], want_min.detach()) and _same(grid[3], want_max.detach())
    # without gate the tensors are left alone
    again_min, again_max = mn.clone(), mx.clone()
    ops.range_to_grid(again_min, again_max, 0, 255, ops.RANGE_V1_ASYMMETRIC)
    assert _same(again_min, mn) and _same(again_max, mx)


def test_grid_arguments_are_checked():
    from aimet_amd import ops
    mn, mx = _ranges(4, 1)
    with pytest.raises(Exception):
        ops.range_to_grid(mn, mx, 0, 255, 9)                        # no such mode
    with pytest.raises(Exception):
        ops.range_to_grid(mn, mx, -128, 127, ops.RANGE_V1_ASYMMETRIC)       # the v1 grids start at 0
    with pytest.raises(Exception):
        ops.range_to_grid(mn, mx, 5, 5, ops.RANGE_V2_ASYMMETRIC)
    with pytest.raises(ValueError):
        ops.range_to_grid(mn.double(), mx.double(), 0, 255, ops.RANGE_V2_ASYMMETRIC)
    with pytest.raises(ValueError):
        ops.range_to_grid(mn, mx[:3], 0, 255, ops.RANGE_V2_ASYMMETRIC)


# ---------------------------------------------------------------------------------------------- the range gradients
def _expected_range_grads(ops, mode, sum_s, sum_o, grid, qmin, qmax):
    """The header's formulas in float32 tensor operations, one rounding per operation as in the kernel."""
    scale, mn, mx = grid[0], grid[2], grid[3]
    steps = float(qmax - qmin)
    steps_t = torch.full_like(sum_s, steps)
    rcp = float(np.float32(1.0) / np.float32(steps))
    if mode == ops.RANGE_V2_ASYMMETRIC:
        s = sum_s + (-sum_o) * ((mn / scale) / scale)
        gmax = s * rcp
        return sum_o / scale + (-gmax), gmax
    if mode == ops.RANGE_V2_SYMMETRIC:
        gmax = sum_s * rcp
        return -gmax, gmax
    if mode == ops.RANGE_V1_ASYMMETRIC:
        t1 = sum_s / steps_t
        d = mx - mn
        t2 = steps_t / (d * d) * sum_o
        return -t1 + mx * t2, t1 - mn * t2
    gmax = sum_s / torch.full_like(sum_s, float((qmax - qmin) // 2))
    return -gmax, gmax


_LAYOUTS = [  # (outer, channels, elements per channel)
    (1, 1, 300000),      # per tensor, many workgroups and the reduction kernel
    (1, 1, 4096),        # per tensor, one workgroup: no second launch
    (1, 64, 4608),       # a weight: one workgroup per channel
    (1, 16, 40000),      # several workgroups per channel
    (1, 384, 27),        # short rows (3 x 3 kernels of 3 channels)
    (8, 32, 196),        # activations per channel: an outer dimension
    (4, 6, 5000),        # outer dimension, long rows
]


@pytest.mark.parametrize("outer,channels,per_channel", _LAYOUTS)
@pytest.mark.parametrize("mode_name", ("RANGE_V2_ASYMMETRIC", "RANGE_V2_SYMMETRIC", "RANGE_V1_ASYMMETRIC",
                                       "RANGE_V1_SIGNED_SYMMETRIC", "RANGE_V1_UNSIGNED_SYMMETRIC"))
@pytest.mark.parametrize("dtype", (torch.float32, torch.bfloat16))
def test_range_gradients_equal_the_formulas_on_the_channel_sums(outer, channels, per_channel, mode_name, dtype):
    from aimet_amd import ops
    mode = getattr(ops, mode_name)
    v2 = mode in (ops.RANGE_V2_ASYMMETRIC, ops.RANGE_V2_SYMMETRIC)
    qmin, qmax = (-128, 127) if mode == ops.RANGE_V2_SYMMETRIC else (0, 255)
    torch.manual_seed(outer * 1000 + channels + per_channel)
    x = (torch.randn(outer, channels, per_channel) * 1.5).cuda().to(dtype)
    g = torch.randn(outer, channels, per_channel).cuda().to(dtype)
    mn, mx = _ranges(channels, channels)
    if not v2 and mode != ops.RANGE_V1_ASYMMETRIC:
        mn = -mx                                                    # the symmetric v1 quantizers learn with min = -max
    grid = ops.range_to_grid(mn, mx, qmin, qmax, mode)
    for want_grad_in in (True, False):
        gin, gmin, gmax = ops.qdq_bwd_range(x, g, channels, per_channel, grid, qmin, qmax, mode, want_grad_in)
        ref_in, sum_s, sum_o = ops.v2_qdq_bwd_params(x, g, channels, per_channel, grid[0], grid[1], qmin, qmax,
                                                     want_grad_in=want_grad_in)
        want_min, want_max = _expected_range_grads(ops, mode, sum_s, sum_o, grid, qmin, qmax)
        assert torch.equal(_bits(gmin), _bits(want_min)) and torch.equal(_bits(gmax), _bits(want_max))
        assert (gin is None) == (not want_grad_in)
        if want_grad_in:
            assert torch.equal(gin, ref_in)
    assert torch.isfinite(gmin).all() and gmin.abs().max() > 0


# ------------------------------------------------------------------------------------------------ the v2 quantizers
@pytest.mark.parametrize("shape,param_shape,block_size", [((32, 64, 14, 14), (), None),
                                                          ((64, 32, 3, 3), (64, 1, 1, 1), None),
                                                          ((48, 256), (48, 1), None),
                                                          ((16, 8, 5, 5), (1, 8, 1, 1), None),
                                                          ((32, 128), (32, 4), (1, 32))])
@pytest.mark.parametrize("symmetric", (False, True))
@pytest.mark.parametrize("dtype", (torch.float32, torch.bfloat16))
def test_v2_quantizer_with_and_without_the_fused_range_path(shape, param_shape, block_size, symmetric, dtype,
                                                            monkeypatch):
    from aimet_amd.v2.quantization.affine import QuantizeDequantize
    torch.manual_seed(len(shape) * 17 + int(symmetric))
    x = torch.randn(shape).cuda().to(dtype)
    upstream = torch.randn(shape).cuda().to(dtype)
    results = []
    for fused in (True, False):
        monkeypatch.setattr(QuantizeDequantize, "fuse_range_learning", fused)
        q = QuantizeDequantize(param_shape, 4, symmetric, block_size=block_size).cuda()
        with q.compute_encodings():
            q(x.float() * 0.6)                                      # a range that clips part of x
        for p in q.parameters():
            p.requires_grad_(True)
        xin = x.clone().requires_grad_(True)
        out = q(xin)
        out.backward(upstream)
        results.append((out.detach(), xin.grad, q.min.grad, q.max.grad))
    fused, plain = results
    assert torch.equal(fused[0], plain[0]) and torch.equal(fused[1], plain[1])
    for got, want in zip(fused[2:], plain[2:]):
        assert got.shape == want.shape
        assert torch.allclose(got, want, rtol=1e-5, atol=1e-6 * float(want.abs().max()))
    assert fused[2].abs().max() > 0 and fused[3].abs().max() > 0


def test_v2_fused_range_path_only_while_the_range_learns(monkeypatch):
    """Frozen ranges, inference and calibration do not take it; a range with only one learnable end does."""
    from aimet_amd.v2.quantization.affine import QuantizeDequantize
    from aimet_amd.v2.quantization.affine.backends import hip_gfx950
    calls = []
    original = hip_gfx950.quantize_dequantize_learned_range
    monkeypatch.setattr(hip_gfx950, "quantize_dequantize_learned_range",
                        lambda *a, **k: (calls.append(1), original(*a, **k))[1])
    q = QuantizeDequantize((), 8, False).cuda()
    x = torch.randn(64, 64).cuda()
    with q.compute_encodings():
        q(x)
    with torch.no_grad():
        q(x)
    assert not calls                                                # neither calibration nor inference
    q(x)
    assert len(calls) == 1                                          # min / max are created learnable
    calls.clear()
    q.requires_grad_(False)
    q(x.requires_grad_(True)).sum().backward()
    assert not calls
    q.max.requires_grad_(True)
    q(x).sum().backward()
    assert len(calls) == 1 and q.max.grad is not None and q.min.grad is None


# ------------------------------------------------------------------------------------------------- the v1 wrappers
@pytest.mark.parametrize("symmetric", (False, True))
@pytest.mark.parametrize("per_channel", (False, True))
def test_v1_learned_grid_wrapper_with_and_without_the_library_grid(symmetric, per_channel, monkeypatch):
    from aimet_amd.common.defs import QuantScheme
    from aimet_amd.v1 import quantsim_straight_through_grad as ste
    from aimet_amd.v1.quantsim import QuantizationSimModel

    class Net(nn.Module):
        def __init__(self):
            super().__init__()
            self.conv1, self.relu1 = nn.Conv2d(3, 8, 3, padding=1), nn.ReLU()
            self.conv2, self.flat, self.fc = nn.Conv2d(8, 8, 3, stride=2), nn.Flatten(), nn.Linear(8 * 7 * 7, 10)

        def forward(self, x):
            return self.fc(self.flat(self.conv2(self.relu1(self.conv1(x)))))

    config = {"defaults": {"ops": {"is_output_quantized": "True"},
                           "params": {"is_quantized": "True", "is_symmetric": str(symmetric)},
                           "per_channel_quantization": str(per_channel)},
              "params": {"bias": {"is_quantized": "False"}}, "op_type": {}, "supergroups": [],
              "model_input": {"is_input_quantized": "True"}, "model_output": {}}
    torch.manual_seed(5)
    model = Net().cuda()
    x = torch.randn(8, 3, 16, 16).cuda()
    results = []
    for library_grid in (True, False):
        if not library_grid:
            monkeypatch.setattr(ste, "grid_in_one_launch", lambda *_: False)
        sim = QuantizationSimModel(model, x, quant_scheme=QuantScheme.training_range_learning_with_tf_init,
                                   default_param_bw=4, default_output_bw=8, config_file=config)
        sim.compute_encodings(lambda m, _: m(x), None)
        # a range pushed out of order is put back by the forward pass
        with torch.no_grad():
            sim.model.relu1.output0_encoding_min.fill_(0.25)
        out = sim.model(x * 1.7)
        out.square().mean().backward()
        named = dict(sim.model.named_parameters())
        results.append((out.detach(), {n: p.grad for n, p in named.items() if p.grad is not None},
                        {n: p.detach().clone() for n, p in named.items() if "encoding" in n}))
    (out_a, grads_a, ranges_a), (out_b, grads_b, ranges_b) = results
    assert torch.equal(out_a, out_b)
    assert ranges_a.keys() == ranges_b.keys() and len(ranges_a) >= 10
    for name, value in ranges_a.items():
        assert torch.equal(value, ranges_b[name]), name
    assert float(ranges_a["relu1.output0_encoding_min"]) == 0.0
    assert grads_a.keys() == grads_b.keys()
    checked = 0
    for name, grad in grads_a.items():
        if "encoding" in name:
            assert torch.allclose(grad, grads_b[name], rtol=1e-5, atol=1e-6 * float(grads_b[name].abs().max())), name
            checked += 1
        else:
            # weight gradients come out of convolution kernels that add in no fixed order
            assert torch.allclose(grad, grads_b[name], rtol=1e-4, atol=1e-6), name
    assert checked >= 10


# ------------------------------------------------------------------------------------------------- against the oracle
@pytest.mark.parametrize("mode_name", ("RANGE_V2_ASYMMETRIC", "RANGE_V2_SYMMETRIC", "RANGE_V1_ASYMMETRIC",
                                       "RANGE_V1_SIGNED_SYMMETRIC", "RANGE_V1_UNSIGNED_SYMMETRIC"))
def test_grid_and_range_gradients_against_the_cpu_oracle(mode_name):
    """The CPU restatement (numpy float32, one rounding per operation) gives the same grid, ordered range and range
    gradients to the bit -- the v2 modes with "/ steps" as the product with float32(1 / steps), as the device kernels
    of torch form it; with a division, as torch's CPU kernels do, scale is at most one ulp away."""
    from aimet_amd import ops
    from oracle import lib as oracle
    from oracle import range_oracle
    mode = getattr(ops, mode_name)
    c, n = 24, 3000
    rng = np.random.default_rng(mode)
    enc_min = (-rng.uniform(0.2, 2.0, c)).astype(np.float32)
    enc_max = rng.uniform(0.2, 2.0, c).astype(np.float32)
    enc_min[3], enc_max[5] = 0.125, -0.5                                # out of order: put right by the gate
    if mode == ops.RANGE_V1_SIGNED_SYMMETRIC:
        enc_max[5] = 0.5                                                # (a max of 0 would be a step of 0 here)
    qmin, qmax = (-128, 127) if mode == ops.RANGE_V2_SYMMETRIC else (0, 255)
    want_min, want_max = range_oracle.ordered_range(enc_min, enc_max)
    if mode in (ops.RANGE_V2_ASYMMETRIC, ops.RANGE_V2_SYMMETRIC):
        symmetric = mode == ops.RANGE_V2_SYMMETRIC
        scale, offset = range_oracle.grid_v2(want_min, want_max, qmin, qmax, symmetric, divide=False)
        divided, _ = range_oracle.grid_v2(want_min, want_max, qmin, qmax, symmetric, divide=True)
        assert np.all(np.abs(divided.view(np.int32) - scale.view(np.int32)) <= 1)
    else:
        symmetric = mode != ops.RANGE_V1_ASYMMETRIC
        scale, offset, steps = range_oracle.grid_v1(want_min, want_max, 8, symmetric, False,
                                                    mode == ops.RANGE_V1_UNSIGNED_SYMMETRIC)
        assert steps == qmax
    dev_min, dev_max = torch.from_numpy(enc_min).cuda(), torch.from_numpy(enc_max).cuda()
    grid = ops.range_to_grid(dev_min, dev_max, qmin, qmax, mode, gate=True)
    assert np.array_equal(dev_min.cpu().numpy(), want_min) and np.array_equal(dev_max.cpu().numpy(), want_max)
    got = grid.cpu().numpy()
    assert np.array_equal(got[0].view(np.int32), scale.view(np.int32))
    assert np.array_equal(got[1], offset)           # (by value: max(0, -0) may be either zero, here and in torch)

    x = (rng.standard_normal((c, n)) * 1.3).astype(np.float32)
    g = rng.standard_normal((c, n)).astype(np.float32)
    _, sum_s, sum_o = oracle.v2_qdq_bwd_params(x, g, c, n, scale, offset, qmin, qmax)
    if mode in (ops.RANGE_V2_ASYMMETRIC, ops.RANGE_V2_SYMMETRIC):
        want_gmin, want_gmax = range_oracle.range_grads_v2(sum_s, sum_o, want_min, scale, qmin, qmax, symmetric,
                                                           divide=False)
    else:
        want_gmin, want_gmax = range_oracle.range_grads_v1(sum_s, sum_o, want_min, want_max, qmax, symmetric)
    _, gmin, gmax = ops.qdq_bwd_range(torch.from_numpy(x).cuda(), torch.from_numpy(g).cuda(), c, n, grid, qmin, qmax,
                                      mode, want_grad_in=False)
    # the sums are float32 sums in another order: the bar of the scale / offset gradients (2e-5 of their magnitude)
    for got_grad, want_grad in ((gmin, want_gmin), (gmax, want_gmax)):
        bar = 2e-5 * max(float(np.abs(want_gmin).max()), float(np.abs(want_gmax).max()))
        assert np.allclose(got_grad.cpu().numpy(), want_grad, rtol=2e-5, atol=bar)
