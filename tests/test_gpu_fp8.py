"""8-bit float simulation: the HIP kernel against the reference's torch expression (aimet_torch/fp_quantization.py:
133-209), evaluated by torch in float32 on the same GPU.  Both sides use the device's library log2 / pow, but torch and
this library are built with different releases of it, so single results may differ in the last bit: the bar is a
relative error of 1e-6, and the share of bit-identical elements is checked to be overwhelming.  Independently of that
expression, test_nearest_point_of_the_enumerated_grid pins the kernel to the format's own definition: nearest point of
the enumerated grid (to the few ulp the device's pow() leaves).
"""
import pytest
import torch

pytestmark = pytest.mark.gpu


def _reference(x_float, maxval, mantissa_bits, ch_axis=0):
    """torch float32 statement of the fake cast, op for op."""
    m = torch.tensor([float(mantissa_bits)], device=x_float.device)
    exponent_bits = 7 - m
    if maxval.dim() and maxval.shape[0] != 1:
        shape = [1] * x_float.dim()
        shape[ch_axis] = -1
        maxval = maxval.view(shape)
    bias = 2 ** exponent_bits - torch.log2(maxval) + torch.log2(2 - 2 ** (-m)) - 1
    x_clipped = x_float.clamp(-maxval, maxval)
    log_scales = torch.clamp(torch.floor(torch.log2(torch.abs(x_clipped)) + bias), 1.)
    scales = 2. ** (log_scales - m - bias)
    return torch.round(x_clipped / scales) * scales


def _check(got, want):
    assert got.shape == want.shape
    nan = torch.isnan(want)
    assert torch.equal(torch.isnan(got), nan)
    torch.testing.assert_close(got[~nan], want[~nan], rtol=1e-6, atol=0.0)
    assert (got[~nan] == want[~nan]).float().mean().item() > 0.999


@pytest.mark.parametrize("mantissa_bits", [3, 2, 4])
@pytest.mark.parametrize("shape", [(4096, 1024), (3, 7, 5), (1,), (64, 3, 3, 3)])
def test_per_tensor(shape, mantissa_bits):
    from aimet_amd import ops
    g = torch.Generator(device='cuda').manual_seed(5)
    x = torch.randn(shape, device='cuda', generator=g) * 3
    maxval = x.abs().max() * 0.7                      # part of the tensor clips
    _check(ops.fp8_fake_cast(x, maxval, mantissa_bits), _reference(x, maxval, mantissa_bits))


def test_grid_properties():
    """What the format fixes: at most 2^8 distinct values, symmetric, idempotent, maxval itself representable, zero
    and the subnormal range on a uniform grid."""
    from aimet_amd import ops
    g = torch.Generator(device='cuda').manual_seed(6)
    x = torch.randn(1 << 20, device='cuda', generator=g) * torch.logspace(-6, 1, 1 << 20, device='cuda')
    maxval = torch.tensor(7.5, device='cuda')         # 1.875 * 2^2: the grid is the unscaled E4M3-shaped one
    y = ops.fp8_fake_cast(x, maxval)
    assert torch.unique(y).numel() <= 256
    assert torch.equal(ops.fp8_fake_cast(-x, maxval), -y)
    torch.testing.assert_close(ops.fp8_fake_cast(y, maxval), y, rtol=1e-6, atol=0.0)
    assert y.abs().max().item() == pytest.approx(7.5, rel=1e-6)
    assert ops.fp8_fake_cast(torch.zeros(8, device='cuda'), maxval).abs().sum().item() == 0
    # steps of 2^-1 in [4, 8), 2^-2 in [2, 4), ...; the step itself comes out of pow() and is exact to a few ulp
    probe = torch.tensor([4.3, 7.4, 2.1, 100.0, -100.0, 1.06], device='cuda')
    assert ops.fp8_fake_cast(probe, maxval).tolist() == pytest.approx([4.5, 7.5, 2.0, 7.5, -7.5, 1.0], rel=1e-6)
    small = ops.fp8_fake_cast(torch.linspace(0, 2.0 ** -11, 4097, device='cuda'), maxval)
    steps = torch.unique(small)
    assert steps.numel() > 2
    assert torch.allclose(steps[1:] - steps[:-1], (steps[1] - steps[0]).expand(steps.numel() - 1))


def _enumerated_grid(k, mantissa_bits):
    """Every non-negative value of the 8-bit float format with `mantissa_bits` mantissa bits whose largest value is
    maxval = (2 - 2^-m) 2^k, written down from the format itself (sign, 7 - m exponent bits, m mantissa bits, subnormals,
    no infinities; aimet_torch/fp_quantization.py:133-209 chooses the exponent bias so that maxval is the top code):
    exponent bias b = 2^(7 - m) - k - 1; subnormals and the first binade j 2^(1 - m - b), j = 0 .. 2^(m + 1) - 1;
    binade p >= 2 - b: (2^m + j) 2^(p - m), j = 0 .. 2^m - 1; nothing above maxval."""
    m = mantissa_bits
    bias = 2 ** (7 - m) - k - 1
    maxval = (2.0 - 2.0 ** -m) * 2.0 ** k
    vals = [j * 2.0 ** (1 - m - bias) for j in range(2 ** (m + 1))]
    for p in range(2 - bias, k + 1):
        vals += [(2 ** m + j) * 2.0 ** (p - m) for j in range(2 ** m)]
    vals = sorted(v for v in set(vals) if v <= maxval)
    return vals, maxval


@pytest.mark.parametrize("mantissa_bits,k", [(3, 2), (3, 8), (3, -3), (2, 0), (4, 5), (5, 1)])
def test_nearest_point_of_the_enumerated_grid(mantissa_bits, k):
    """Closed-form check that does not go through the reference's log2 / pow expression: for a maxval that is the top
    code of an unscaled format, the grid is enumerated from the format's definition and the kernel must return, for
    every input, the nearest grid point (brute force in float64), the clipped value outside, and every grid point
    unchanged.  The step of a binade comes out of the device's pow() in the kernel as in the reference, a few float32
    ulp from the power of two, so values are compared to 2e-6 relative, and inputs closer than 1e-5 (relative to the
    step) to the middle between two grid points -- whose side those ulp decide -- are left out."""
    import numpy as np
    from aimet_amd import ops
    grid, maxval = _enumerated_grid(k, mantissa_bits)
    assert len(grid) == 2 ** 7 and grid[-1] == maxval                # 128 codes per sign, the largest is maxval
    g = np.array(grid)
    rng = np.random.default_rng(mantissa_bits * 100 + k + 50)
    x = np.concatenate([rng.uniform(-1.3 * maxval, 1.3 * maxval, 3000),
                        rng.uniform(-1, 1, 3000) * g[8],             # subnormal range and first binades
                        rng.standard_normal(2000) * g[40], g, -g])
    x = x.astype(np.float32).astype(np.float64)
    mag = np.minimum(np.abs(x), maxval)
    hi = np.searchsorted(g, mag, side='left').clip(1, len(g) - 1)
    lo = hi - 1
    d_lo, d_hi = mag - g[lo], g[hi] - mag
    decided = np.abs(d_lo - d_hi) > 1e-5 * (g[hi] - g[lo])
    assert decided.mean() > 0.99
    want = (np.sign(x) * np.where(d_lo < d_hi, g[lo], g[hi]))[decided]
    got = ops.fp8_fake_cast(torch.from_numpy(x.astype(np.float32)).cuda(), torch.tensor(maxval, device='cuda'),
                            mantissa_bits).cpu().numpy().astype(np.float64)[decided]
    assert np.allclose(got, want, rtol=2e-6, atol=0.0)


@pytest.mark.parametrize("shape, axis", [((16, 8, 3, 3), 0), ((8, 16, 3, 3), 1), ((32, 100), 0), ((5, 7), 1),
                                         ((6, 4, 8), 1),
                                         # rows of 1024 elements and more take the row-wise kernel: a ragged row, rows
                                         # inside an outer dimension, several workgroups per row, the shortest such row
                                         ((12, 4100), 0), ((3, 5, 2048), 1), ((64, 8192), 0), ((2, 3, 1024), 1),
                                         ((3, 20000), 0)])
def test_per_channel(shape, axis):
    from aimet_amd import ops
    g = torch.Generator(device='cuda').manual_seed(7)
    x = torch.randn(shape, device='cuda', generator=g)
    x = x * torch.logspace(-2, 2, shape[axis], device='cuda').view([-1 if a == axis else 1 for a in range(len(shape))])
    reduce_dims = [a for a in range(len(shape)) if a != axis]
    maxval = x.abs().amax(dim=reduce_dims) * 0.9
    _check(ops.fp8_fake_cast(x, maxval, 3, axis), _reference(x, maxval, 3, axis))


def test_special_values_and_errors():
    from aimet_amd import ops
    x = torch.tensor([float('nan'), float('inf'), -float('inf'), 0.0, -0.0, 1e-30, -1e-30, 3.0], device='cuda')
    maxval = torch.tensor(2.0, device='cuda')
    _check(ops.fp8_fake_cast(x, maxval), _reference(x, maxval, 3))
    with pytest.raises(RuntimeError):
        ops.fp8_fake_cast(torch.zeros(4, 4, device='cuda'), torch.ones(3, device='cuda'))
    with pytest.raises(RuntimeError):
        ops.fp8_fake_cast(torch.zeros(4), torch.tensor(1.0))
    with pytest.raises(RuntimeError):
        ops.fp8_fake_cast(torch.zeros(4, device='cuda'), torch.tensor(1.0, device='cuda'), mantissa_bits=0)


# ------------------------------------------------------------------------- through the tensor quantizers and the sim
def _quantizer(per_channel, scheme, channels=8, axis=0):
    from aimet_amd.common.defs import QuantizationDataType
    from aimet_amd.v1.tensor_quantizer import StaticGridPerChannelQuantizer, StaticGridPerTensorQuantizer
    if per_channel:
        return StaticGridPerChannelQuantizer(8, 'nearest', scheme, False, channels, True, ch_axis=axis,
                                             data_type=QuantizationDataType.float)
    return StaticGridPerTensorQuantizer(8, 'nearest', scheme, False, True, data_type=QuantizationDataType.float)


def test_tensor_quantizer_minmax_init_and_running_maxval():
    """TF scheme: maxval is the largest magnitude, then 0.9 old + 0.1 new (reference tensor_quantizer.py:393-400)."""
    from aimet_amd.common import libpymo
    from aimet_amd.common.defs import QuantScheme
    q = _quantizer(False, QuantScheme.post_training_tf)
    x = torch.randn(64, 64, device='cuda')
    with pytest.raises(ValueError):
        q.quantize_dequantize(x, libpymo.RoundingMode.ROUND_NEAREST)       # no maxval yet
    q.update_encoding_stats(x)
    first = x.abs().max()
    assert torch.equal(q.fp8_maxval, first)
    q.update_encoding_stats(2 * x)
    assert torch.allclose(q.fp8_maxval, 0.9 * first + 0.1 * 2 * first)
    q.compute_encoding()
    assert q.encoding.max == pytest.approx(float(q.fp8_maxval)) and q.encoding.min == -q.encoding.max
    out = q.quantize_dequantize(x, libpymo.RoundingMode.ROUND_NEAREST)
    _check(out, _reference(x, q.fp8_maxval, 3))
    # pass-through gradient
    xg = x.clone().requires_grad_(True)
    q.quantize_dequantize(xg, libpymo.RoundingMode.ROUND_NEAREST).sum().backward()
    assert torch.equal(xg.grad, torch.ones_like(x))


@pytest.mark.parametrize("per_channel", [False, True])
def test_tensor_quantizer_mse_init(per_channel):
    """TF-Enhanced scheme: the candidate among 111 in [0.1, 1.2] x largest magnitude with the least squared error
    (reference fp_quantization.py:78-110), checked against the same search written with the torch expression."""
    from aimet_amd.common import libpymo
    from aimet_amd.common.defs import QuantScheme
    g = torch.Generator(device='cuda').manual_seed(11)
    x = torch.randn(8, 4, 3, 3, device='cuda', generator=g)
    x[:, 0, 0, 0] *= 6                               # an outlier per channel
    q = _quantizer(per_channel, QuantScheme.post_training_tf_enhanced)
    q.update_encoding_stats(x)
    largest = x.abs().amax(dim=(1, 2, 3)) if per_channel else x.abs().max()
    fractions = torch.linspace(0.1, 1.2, 111, device='cuda')
    errors = torch.stack([((x - _reference(x, largest * f, 3)) ** 2).mean(dim=(1, 2, 3) if per_channel else None)
                          for f in fractions])
    # a tie or a last-bit difference in an error may pick the neighbouring candidate
    picked = q.fp8_maxval / largest
    assert torch.all((picked - fractions[errors.argmin(0)]).abs() <= 0.0101)
    assert len(q.encoding) == 8 if per_channel else q.encoding.max == pytest.approx(float(q.fp8_maxval))
    out = q.quantize_dequantize(x, libpymo.RoundingMode.ROUND_NEAREST)
    _check(out, _reference(x, q.fp8_maxval, 3))


def test_percentile_scheme_is_refused():
    from aimet_amd.common.defs import QuantScheme
    q = _quantizer(False, QuantScheme.post_training_percentile)
    with pytest.raises(NotImplementedError):
        q.update_encoding_stats(torch.randn(16, device='cuda'))


@pytest.mark.parametrize("per_channel", [False, True])
def test_simulation_model_with_8_bit_float(per_channel, tmp_path):
    import json
    from torch import nn
    from aimet_amd.common.defs import QuantizationDataType, QuantScheme
    from aimet_amd.v1.quantsim import QuantizationSimModel
    torch.manual_seed(3)
    model = nn.Sequential(nn.Conv2d(3, 8, 3), nn.ReLU(), nn.Flatten(), nn.Linear(8 * 6 * 6, 10)).cuda().eval()
    x = torch.rand(4, 3, 8, 8, device='cuda')
    sim = QuantizationSimModel(model, x, quant_scheme=QuantScheme.post_training_tf, default_output_bw=8,
                               default_param_bw=8, default_data_type=QuantizationDataType.float)
    if per_channel:
        for _, wrapper in sim.quant_wrappers():
            wrapper.enable_per_channel_quantization()
    sim.compute_encodings(lambda m, _: m(x), None)
    with torch.no_grad():
        out, ref = sim.model(x), model(x)
    assert torch.isfinite(out).all()
    assert not torch.equal(out, ref)
    assert (out - ref).abs().max() < 0.25 * ref.abs().max()          # 3 mantissa bits: a few percent
    weight_quantizer = getattr(sim.model, '0').param_quantizers['weight']
    assert weight_quantizer.fp8_maxval.numel() == (8 if per_channel else 1)
    # the last module's output goes through the fake cast with the calibrated maxval
    last = getattr(sim.model, '3').output_quantizers[0]
    _check(out, _reference(out, last.fp8_maxval, 3))
    sim.export_encodings(str(tmp_path), 'fp8')
    with open(tmp_path / 'fp8.encodings') as f:
        encodings = json.load(f)
    assert encodings['param_encodings']['0.weight'] == [{'bitwidth': 8, 'dtype': 'float'}]
    assert encodings['activation_encodings']['3']['output']['0'] == {'bitwidth': 8, 'dtype': 'float'}
    # training-mode pass: parameters are re-observed, gradients pass straight through
    sim.model.train()
    sim.model(x).sum().backward()
    assert getattr(sim.model, '0')._module_to_wrap.weight.grad is not None
