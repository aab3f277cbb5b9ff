"""GPU parity of the stochastic rounding mode (DlQuantization/src/trim_functions.cpp:141-166, ROUND_STOCHASTIC) through
the C ABI.  The restated formula is pinned against the reference's CPU loop, and the generator against its published
recipe, in tests/test_oracle_stochastic.py; here the kernel must equal formula(generator) bit for bit, for every
launch path (16-byte vectors, tails, misaligned pointers, rows shorter than a vector, bf16 storage), for grid positions
outside the float fast path (negative, >= 2^23), and at the host interface of the v1 quantizers."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

STOCHASTIC = 1


def _bits(a):
    return np.ascontiguousarray(a, np.float32).view(np.uint32)


def _gpu(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def _inputs(seed, n, scale):
    rng = np.random.default_rng(seed)
    x = (rng.standard_normal(n) * scale).astype(np.float32)
    if n >= 16:
        x[:8] = [np.nan, np.inf, -np.inf, 0.0, -0.0, 1e-42, -1e-42, 3.4e38]
    return x


@pytest.fixture(scope="module")
def ops():
    from aimet_amd import ops as o
    return o


@pytest.mark.parametrize("n", [1, 3, 5, 4096, 1_000_003])
@pytest.mark.parametrize("bw,mnmx", [(8, (-0.46, 0.72)), (4, (0.0, 6.0)), (16, (-3.0, 3.0))])
def test_per_tensor(ops, oracle, n, bw, mnmx):
    x = _inputs(n + bw, n, 1.5)
    seed = 1000 + n % 97
    ops.set_stochastic_seed(seed)
    assert ops.stochastic_state() == (seed, 0)
    xg = _gpu(x)
    for call in range(3):
        got = ops.qdq_per_tensor(xg, *mnmx, bw, STOCHASTIC).cpu().numpy()
        want = oracle.stochastic_per_tensor(x, *mnmx, bw, oracle.stochastic_uniforms(seed, call, n))
        assert np.array_equal(_bits(got), _bits(want)), call
    assert ops.stochastic_state() == (seed, 3)
    for call, shift in ((3, False), (4, True)):
        got = ops.quantize_per_tensor(xg, *mnmx, bw, shift, STOCHASTIC).cpu().numpy()
        want = oracle.stochastic_per_tensor(x, *mnmx, bw, oracle.stochastic_uniforms(seed, call, n), dequant=False,
                                            shift_to_signed=shift)
        assert np.array_equal(_bits(got), _bits(want))
    # the same seed gives the same numbers again; nearest rounding does not consume a call
    ops.set_stochastic_seed(seed)
    ops.qdq_per_tensor(xg, *mnmx, bw)
    again = ops.qdq_per_tensor(xg, *mnmx, bw, STOCHASTIC).cpu().numpy()
    want = oracle.stochastic_per_tensor(x, *mnmx, bw, oracle.stochastic_uniforms(seed, 0, n))
    assert np.array_equal(_bits(again), _bits(want))


def test_per_tensor_misaligned_and_empty(ops, oracle):
    n = 100_001
    x = _inputs(5, n + 1, 1.0)
    xg = _gpu(x)[1:]                       # 4 bytes off a 16-byte boundary: the element-wise kernel
    ops.set_stochastic_seed(9)
    got = ops.qdq_per_tensor(xg, -1.0, 2.0, 8, STOCHASTIC).cpu().numpy()
    want = oracle.stochastic_per_tensor(x[1:], -1.0, 2.0, 8, oracle.stochastic_uniforms(9, 0, n))
    assert np.array_equal(_bits(got), _bits(want))
    empty = ops.qdq_per_tensor(torch.empty(0, device='cuda'), -1.0, 2.0, 8, STOCHASTIC)
    assert empty.numel() == 0 and ops.stochastic_state() == (9, 1)


@pytest.mark.parametrize("outer,c,npc", [(1, 37, 513), (2, 5, 3), (3, 4, 1), (1, 64, 4096), (2, 3, 6)])
def test_per_channel(ops, oracle, outer, c, npc):
    rng = np.random.default_rng(c * npc)
    x = _inputs(c + npc, outer * c * npc, 0.05)
    enc_min = -np.abs(rng.standard_normal(c)) * 0.1
    enc_max = np.abs(rng.standard_normal(c)) * 0.1
    for bw in (4, 8):
        params = oracle.per_channel_params(enc_min, enc_max, bw)
        gp = [_gpu(p) for p in params]
        ops.set_stochastic_seed(bw)
        for call in range(2):
            got = ops.qdq_per_channel(_gpu(x), c, npc, *gp, rounding_mode=STOCHASTIC).cpu().numpy()
            want = oracle.stochastic(x, c, npc, params, oracle.stochastic_uniforms(bw, call, x.size))
            assert np.array_equal(_bits(got), _bits(want))
        # misaligned input: element-wise kernel
        xs = np.concatenate([[0.0], x]).astype(np.float32)
        got = ops.qdq_per_channel(_gpu(xs)[1:], c, npc, *gp, rounding_mode=STOCHASTIC).cpu().numpy()
        want = oracle.stochastic(x, c, npc, params, oracle.stochastic_uniforms(bw, 2, x.size))
        assert np.array_equal(_bits(got), _bits(want))


def test_grid_positions_outside_the_float_path(ops, oracle):
    """Parameters a caller may pass directly: a minimum that is not on the grid gives negative grid positions at the
    lower clamp, a tiny delta gives positions >= 2^23 where float32 has no fraction bits left; both take the double
    arithmetic of the reference."""
    c, npc = 5, 50_000
    mn = np.array([-0.33, -0.05, 0.0, -1.0, -1e-21], np.float32)
    mx = np.array([0.5, 0.05, 1.0, 1.0, 1e-21], np.float32)
    delta = np.array([0.1, 0.1, 1e-8, 3e-9, 1.7e-25], np.float32)      # the last one is below the fast division's range
    offset = np.array([-3.0, 0.0, 0.0, -7.0, -5882.0], np.float32)
    x = _inputs(77, c * npc, 0.5)
    x[4 * npc:] *= 1e-21
    params = (mn, mx, delta, offset)
    ops.set_stochastic_seed(31)
    got = ops.qdq_per_channel(_gpu(x), c, npc, *[_gpu(p) for p in params], rounding_mode=STOCHASTIC).cpu().numpy()
    want = oracle.stochastic(x, c, npc, params, oracle.stochastic_uniforms(31, 0, x.size))
    assert np.array_equal(_bits(got), _bits(want))
    t = (np.clip(x.reshape(c, npc), mn[:, None], mx[:, None]) / delta[:, None] - offset[:, None])
    assert (t[0] < 0).any() and (t[2] >= 2 ** 23).any()


def test_bf16_storage(ops, oracle):
    n = 300_001
    x = _inputs(8, n, 1.0)
    bits = oracle.f32_to_bf16_bits(x)
    xf = oracle.bf16_bits_to_f32(bits)
    xb = _gpu(bits.view(np.int16)).view(torch.bfloat16)
    ops.set_stochastic_seed(4)
    got = ops.qdq_per_tensor(xb, -2.0, 1.5, 8, STOCHASTIC).view(torch.int16).cpu().numpy().view(np.uint16)
    want = oracle.f32_to_bf16_bits(oracle.stochastic_per_tensor(xf, -2.0, 1.5, 8, oracle.stochastic_uniforms(4, 0, n)))
    assert np.array_equal(got, want)
    c, npc = 7, 1001
    x = _inputs(9, 2 * c * npc, 0.05)
    bits = oracle.f32_to_bf16_bits(x)
    xf = oracle.bf16_bits_to_f32(bits)
    params = oracle.per_channel_params(-np.linspace(0.05, 0.1, c), np.linspace(0.04, 0.12, c), 4)
    got = ops.qdq_per_channel(_gpu(bits.view(np.int16)).view(torch.bfloat16), c, npc, *[_gpu(p) for p in params],
                              rounding_mode=STOCHASTIC).view(torch.int16).cpu().numpy().view(np.uint16)
    want = oracle.f32_to_bf16_bits(oracle.stochastic(xf, c, npc, params, oracle.stochastic_uniforms(4, 1, x.size)))
    assert np.array_equal(got, want)


def test_unbiased_and_one_step(ops, oracle):
    """What stochastic rounding is for: E[q] = t.  A constant input between two grid points comes out as the two
    neighbours in the proportion of its position; and no output is further than one step from the input."""
    e = oracle.fill_encoding_info(8, -1.0, 1.0)
    n = 1 << 22
    for frac in (0.1, 0.5, 0.9):
        value = np.float32(e.delta * (140 + frac + e.offset))
        x = torch.full((n,), float(value), device='cuda')
        ops.set_stochastic_seed(int(frac * 10))
        y = ops.qdq_per_tensor(x, -1.0, 1.0, 8, STOCHASTIC)
        q = torch.round(y / e.delta - e.offset).long()
        assert set(q.unique().tolist()) == {140, 141}
        up = (q == 141).double().mean().item()
        assert abs(up - frac) < 5 * np.sqrt(frac * (1 - frac) / n) + 1e-6
    x = torch.randn(n, device='cuda') * 0.3
    y = ops.qdq_per_tensor(x, -1.0, 1.0, 8, STOCHASTIC)
    inside = (x > e.min) & (x < e.max)
    assert (y - x)[inside].abs().max().item() < e.delta * (1 + 1e-5)
    assert abs((y - x)[inside].double().mean().item()) < 5 * e.delta / np.sqrt(n)


def test_v1_quantizers_with_stochastic_rounding(ops, oracle):
    from aimet_amd.common import libpymo
    from aimet_amd.common.defs import QuantScheme
    from aimet_amd.v1 import tensor_quantizer as tq
    stochastic = libpymo.RoundingMode.ROUND_STOCHASTIC
    x = _gpu(_inputs(3, 65_536, 1.0)[8:])
    q = tq.StaticGridPerTensorQuantizer(8, stochastic, QuantScheme.post_training_tf, False, enabled_by_default=True)
    q.update_encoding_stats(x)
    q.compute_encoding()
    e = q.encoding
    ops.set_stochastic_seed(21)
    y = q.quantize_dequantize(x, stochastic).cpu().numpy()
    want = oracle.stochastic_per_tensor(x.cpu().numpy(), e.min, e.max, e.bw, oracle.stochastic_uniforms(21, 0, x.numel()))
    assert np.array_equal(_bits(y), _bits(want))
    codes = q.quantize(x, stochastic).cpu().numpy()
    want = oracle.stochastic_per_tensor(x.cpu().numpy(), e.min, e.max, e.bw, oracle.stochastic_uniforms(21, 1, x.numel()),
                                        dequant=False, shift_to_signed=True)   # signed range by default
    assert np.array_equal(codes, want)
    # per channel
    w = _gpu(_inputs(4, 16 * 72, 0.1).reshape(16, 8, 3, 3))
    pc = tq.StaticGridPerChannelQuantizer(4, stochastic, QuantScheme.post_training_tf, True, num_channels=16,
                                          enabled_by_default=True, ch_axis=0)
    pc.update_encoding_stats(w)
    pc.compute_encoding()
    ops.set_stochastic_seed(22)
    y = pc.quantize_dequantize(w, stochastic).cpu().numpy()
    params = oracle.per_channel_params(np.array([e.min for e in pc.encoding]), np.array([e.max for e in pc.encoding]), 4)
    want = oracle.stochastic(w.cpu().numpy(), 16, 72, params, oracle.stochastic_uniforms(22, 0, w.numel()))
    assert np.array_equal(_bits(y), _bits(want.reshape(-1)).reshape(_bits(y).shape))
    # the straight-through gradient does not depend on the rounding mode
    xr = x.clone().requires_grad_(True)
    q.quantize_dequantize(xr, stochastic).sum().backward()
    assert torch.equal(xr.grad, ((xr >= e.min) & (xr <= e.max)).float())
