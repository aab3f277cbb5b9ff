"""Stochastic rounding (DlQuantization/src/trim_functions.cpp:141-166, ROUND_STOCHASTIC): q = floor(t + u).

Two things are pinned here on the CPU:
* the restated formula (oracle.stochastic, uniform numbers as an argument) against the reference's own CPU loop, which
  draws from libc rand(): srand(seed) before the reference call, the same rand() sequence replayed for the restatement;
  bit-identical results, per tensor (quantize-dequantize and quantize with and without the signed shift) and per
  channel;
* the product's documented generator (restated in oracle.stochastic_uniforms): a known-answer vector computed by hand
  from the published recipe in pure Python, range, mean / variance, independence of seeds and of calls.
The GPU kernel is then compared bit for bit with `formula(generator)` in tests/test_gpu_stochastic.py.
"""
import numpy as np
import pytest


def _bits(a):
    return np.asarray(a, np.float32).view(np.uint32)


def _inputs(rng, n, scale):
    x = (rng.standard_normal(n) * scale).astype(np.float32)
    x[:8] = [np.nan, np.inf, -np.inf, 0.0, -0.0, 1e-42, -1e-42, 3.4e38]
    return x


@pytest.mark.parametrize("bw", [4, 8, 16])
@pytest.mark.parametrize("mnmx", [(-0.46, 0.72), (0.0, 6.0), (-3.0, 3.0), (-1e-7, 2e-7), (0.5, 1.0)])
def test_formula_against_reference_per_tensor(oracle, ref, bw, mnmx):
    rng = np.random.default_rng(bw + int(mnmx[1] * 10))
    x = _inputs(rng, 50000, 1.5)
    for seed in (1, 77):
        u = ref.libc_uniforms(seed, x.size)
        assert u.min() >= 0.0 and u.max() < 1.0
        want = ref.qdq_per_tensor_stochastic(x, *mnmx, bw, seed)
        got = oracle.stochastic_per_tensor(x, *mnmx, bw, u)
        assert np.array_equal(_bits(got), _bits(want))
        for shift in (False, True):
            want = ref.quantize_per_tensor_stochastic(x, *mnmx, bw, shift, seed)
            got = oracle.stochastic_per_tensor(x, *mnmx, bw, u, dequant=False, shift_to_signed=shift)
            assert np.array_equal(_bits(got), _bits(want))
    # the rounding really is stochastic: it differs from nearest somewhere, by at most one step, and is unbiased
    e = oracle.fill_encoding_info(bw, *mnmx)
    near = oracle.quantize_per_tensor(x[8:], *mnmx, bw, False)
    stoch = oracle.stochastic_per_tensor(x[8:], *mnmx, bw, ref.libc_uniforms(5, x.size - 8), dequant=False)
    assert np.abs(near - stoch).max() <= 1.0
    inside = (x[8:] > e.min) & (x[8:] < e.max)
    if inside.sum() > 1000:
        assert (near != stoch).any()
        t = x[8:][inside].astype(np.float64) / e.delta - e.offset
        assert abs((stoch[inside] - t).mean()) < 0.02


def test_formula_against_reference_per_channel(oracle, ref):
    rng = np.random.default_rng(3)
    c, npc = 19, 257
    x = _inputs(rng, 2 * c * npc, 0.05)
    enc_min = -np.abs(rng.standard_normal(c)) * 0.1
    enc_max = np.abs(rng.standard_normal(c)) * 0.1
    for bw in (4, 8):
        params = oracle.per_channel_params(enc_min, enc_max, bw)
        u = ref.libc_uniforms(9, x.size)
        want = ref.qdq_per_channel_stochastic(x, c, npc, params, 9)
        got = oracle.stochastic(x, c, npc, params, u)
        assert np.array_equal(_bits(got), _bits(want))


# ------------------------------------------------------------------------------------------------- the generator
M32, M64 = 0xFFFFFFFF, 0xFFFFFFFFFFFFFFFF


def _mix32(x):
    x ^= x >> 16
    x = (x * 0x7feb352d) & M32
    x ^= x >> 15
    x = (x * 0x846ca68b) & M32
    x ^= x >> 16
    return x


def _uniform(seed, call, i):
    z = (seed + 0x9E3779B97F4A7C15 * (call + 1)) & M64
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & M64
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & M64
    z ^= z >> 31
    k0, k1 = z & M32, z >> 32
    r = _mix32((i + k0) & M32) ^ k1 ^ ((i >> 32) & M32)
    return (r >> 8) / 2.0 ** 24


def test_generator_known_answers(oracle):
    for seed, call in ((0, 0), (1234, 0), (1234, 7), (2 ** 64 - 1, 3)):
        for first in (0, 1000, 2 ** 32 - 2, 2 ** 40 + 5):
            got = oracle.stochastic_uniforms(seed, call, 5, first)
            want = [_uniform(seed, call, first + j) for j in range(5)]
            assert got.tolist() == want
    # mix32 is a bijection of the 32-bit integers with mix32(0) == 0: the key added to the counter is what moves the zero
    assert _mix32(0) == 0 and len({_mix32(i) for i in range(1 << 16)}) == 1 << 16


def test_generator_statistics(oracle):
    n = 1 << 20
    u = oracle.stochastic_uniforms(42, 0, n)
    assert u.min() >= 0.0 and u.max() < 1.0
    assert abs(u.mean() - 0.5) < 4 * np.sqrt(1 / 12 / n)
    assert abs(u.var() - 1 / 12) < 1e-3
    counts = np.bincount((u * 256).astype(np.int64), minlength=256)
    chi2 = ((counts - n / 256) ** 2 / (n / 256)).sum()
    assert chi2 < 400                      # 255 degrees of freedom: mean 255, sigma 22.6
    # neighbouring elements, other calls and other seeds are uncorrelated
    others = [u[1:], oracle.stochastic_uniforms(42, 1, n)[:-1], oracle.stochastic_uniforms(43, 0, n)[:-1]]
    for v in others:
        assert abs(np.corrcoef(u[:-1], v)[0, 1]) < 5 / np.sqrt(n)
