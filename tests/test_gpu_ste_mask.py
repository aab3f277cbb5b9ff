"""The forward that saves a one-bit-per-element straight-through mask and the backward that reads it, through the C ABI.

Bar: the forward's output equals the plain forward's bit for bit, the mask bits equal the CPU oracle's comparison
(decoded on the host from the documented layout), and grad_out * bit equals the oracle's straight-through backward bit
for bit (sign of zero included), float32 and bfloat16 storage, per tensor / per channel / v2, ragged sizes, unaligned
pointers, the configured shapes.  Reference: aimet_torch/v1/quantsim_straight_through_grad.py:100-118,
aimet_torch/v2/quantization/affine/backends/torch_builtins.py:303-327.
"""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    from aimet_amd import ops as o
    return o


def _bits(a):
    return np.ascontiguousarray(a, np.float32).view(np.uint32)


def _bf16_bits(t):
    return t.contiguous().view(torch.int16).cpu().numpy().view(np.uint16)


def _gpu(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def _normal(seed, n, scale=1.0, special=True):
    rng = np.random.default_rng(seed)
    x = (rng.standard_normal(n) * scale).astype(np.float32)
    if special and n >= 16:
        x[:8] = [np.nan, np.inf, -np.inf, 0.0, -0.0, 1e-42, -1e-42, 3.4e38]
    return x


def decode_mask(mask, n, vec):
    """Flags of the n elements from the words: group g = 64 * vec elements owns words g * vec .. + vec - 1, bit t of
    word j is element 64 * vec * g + vec * t + j; the n % vec trailing elements sit in one more word."""
    words = mask.cpu().numpy().view(np.uint64)
    nvec = n // vec
    groups = (nvec + 63) // 64
    assert words.size == groups * vec + 1
    t = np.arange(64, dtype=np.uint64)
    bits = ((words[:groups * vec].reshape(groups, vec, 1) >> t) & np.uint64(1)).astype(bool)   # [g, j, t]
    flags = bits.transpose(0, 2, 1).reshape(-1)[:nvec * vec]                                   # element order
    tail = ((words[-1] >> np.arange(n - nvec * vec, dtype=np.uint64)) & np.uint64(1)).astype(bool)
    return np.concatenate([flags, tail])


@pytest.mark.parametrize("n", [1, 3, 4, 5, 255, 256, 257, 1023, 4096, 4097, 65537, (1 << 20) + 3])
def test_per_tensor_sizes(ops, oracle, n):
    x = _normal(n, n, 1.5)
    grad = _normal(n + 1, n, 1.0, special=False)
    grad[:4] = [-1.0, np.inf, -0.0, 2.0][:min(4, n)]     # grad * 0 keeps the sign / gives NaN for inf, as the product does
    mn, mx = -2.1, 3.3
    y, mask = ops.qdq_mask_per_tensor(_gpu(x), mn, mx, 8)
    assert np.array_equal(_bits(y.cpu().numpy()), _bits(oracle.qdq_per_tensor(x, mn, mx, 8)))
    with np.errstate(invalid="ignore"):
        want = (np.float32(mn) <= x) & (x <= np.float32(mx))
    assert np.array_equal(decode_mask(mask, n, 4), want)
    gin = ops.ste_bwd_mask(mask, _gpu(grad)).cpu().numpy()
    assert np.array_equal(_bits(gin), _bits(oracle.ste_bwd_per_tensor(x, grad, np.float32(mn), np.float32(mx))))
    assert torch.equal(ops.ste_bwd_per_tensor(_gpu(x), _gpu(grad), mn, mx).cpu().view(torch.int32),
                       torch.from_numpy(gin).view(torch.int32))


def test_per_tensor_unaligned_and_empty(ops, oracle):
    x = _normal(5, 10001)
    grad = _normal(6, 10001, special=False)
    base, gbase = _gpu(x), _gpu(grad)
    for off in (1, 2, 3):
        y, mask = ops.qdq_mask_per_tensor(base[off:], -1.0, 2.0, 8)
        assert np.array_equal(_bits(y.cpu().numpy()), _bits(oracle.qdq_per_tensor(x[off:], -1.0, 2.0, 8)))
        want = oracle.ste_bwd_per_tensor(x[off:], grad[off:], np.float32(-1.0), np.float32(2.0))
        assert np.array_equal(_bits(ops.ste_bwd_mask(mask, gbase[off:]).cpu().numpy()), _bits(want))
        # a mask written by the tile kernel read by the fallback and the other way round
        y2, mask2 = ops.qdq_mask_per_tensor(base[off:].clone(), -1.0, 2.0, 8)
        assert torch.equal(mask2, mask)
        assert np.array_equal(_bits(ops.ste_bwd_mask(mask, gbase[off:].clone()).cpu().numpy()), _bits(want))
    y, mask = ops.qdq_mask_per_tensor(torch.empty(0, device="cuda"), -1, 1, 8)
    assert y.numel() == 0 and mask.numel() == 1
    assert ops.ste_bwd_mask(mask, torch.empty(0, device="cuda")).numel() == 0
    with pytest.raises(RuntimeError, match="mask"):
        ops.ste_bwd_mask(mask, torch.zeros(100, device="cuda"))


def test_cfg1_activation(ops, oracle):
    """[32,64,56,56] ~N(0,1) with its min/max encoding: forward, mask and backward at the configured size."""
    shape = (32, 64, 56, 56)
    x = torch.randn(shape, generator=torch.Generator().manual_seed(1001))
    grad = torch.randn(shape, generator=torch.Generator().manual_seed(1101))
    xn = x.numpy()
    enc = oracle.tf_compute_encoding(*map(float, oracle.minmax(xn)), 8)
    # a narrower range too, so that a good share of the mask is zero
    for mn, mx in ((enc.min, enc.max), (-0.5, 1.25)):
        y, mask = ops.qdq_mask_per_tensor(x.cuda(), mn, mx, 8)
        assert torch.equal(y, ops.qdq_per_tensor(x.cuda(), mn, mx, 8))
        gin = ops.ste_bwd_mask(mask, grad.cuda()).cpu().numpy()
        assert np.array_equal(_bits(gin), _bits(oracle.ste_bwd_per_tensor(xn, grad.numpy(), np.float32(mn),
                                                                          np.float32(mx))))
    assert mask.numel() * 8 == x.numel() // 8 + 8


def test_per_tensor_bf16(ops, oracle):
    for n in (200003, 8, 7, 513 * 8):
        x = torch.from_numpy(_normal(9, n, 2.0)).to(torch.bfloat16)
        g = torch.from_numpy(_normal(10, n, 1.0, special=False)).to(torch.bfloat16)
        y, mask = ops.qdq_mask_per_tensor(x.cuda(), -3.0, 2.5, 8)
        assert np.array_equal(_bf16_bits(y), oracle.qdq_per_tensor_bf16(_bf16_bits(x), -3.0, 2.5, 8))
        xf = x.float().numpy()
        with np.errstate(invalid="ignore"):
            assert np.array_equal(decode_mask(mask, n, 8), (np.float32(-3.0) <= xf) & (xf <= np.float32(2.5)))
        gin = ops.ste_bwd_mask(mask, g.cuda())
        assert np.array_equal(_bf16_bits(gin), _bf16_bits(ops.ste_bwd_per_tensor(x.cuda(), g.cuda(), -3.0, 2.5)))
        want = oracle.ste_bwd_per_tensor(xf, g.float().numpy(), np.float32(-3.0), np.float32(2.5))
        assert np.array_equal(gin.float().cpu().numpy(), want)


def _laplace_outliers(seed, shape):
    rng = np.random.default_rng(seed)
    u = rng.random(shape) - 0.5
    w = (-0.02 * np.sign(u) * np.log(1 - 2 * np.abs(u))).astype(np.float32)
    w[rng.random(shape) < 0.001] *= 20
    return w


@pytest.mark.parametrize("shape", [(512, 512, 3, 3), (4096, 4096), (11008, 4096)])
@pytest.mark.parametrize("bw", [8, 4])
def test_cfg2_weight_shapes(ops, oracle, shape, bw):
    """Per-output-channel symmetric weights at the configured shapes; the stored encoding is narrower than the data in
    every tenth channel so that the mask has zeros."""
    seed = 1002 + {512: 0, 4096: 1, 11008: 2}[shape[0]]
    w = _laplace_outliers(seed, shape)
    c, npc = shape[0], int(np.prod(shape[1:]))
    rows = w.reshape(c, npc)
    amax = np.abs(rows).max(axis=1).astype(np.float64)
    amax[::10] *= 0.02
    encs = [oracle.tf_compute_encoding(-a, a, bw, sym=True) for a in amax]
    enc_min, enc_max = np.array([e.min for e in encs]), np.array([e.max for e in encs])
    steps = 2 ** bw - 1 - (1 if enc_min[0] == -enc_max[0] else 0)
    raw = [_gpu(enc_min.astype(np.float32)), _gpu(enc_max.astype(np.float32))]
    gp = ops.per_channel_params(raw[0], raw[1], steps)
    grad = _normal(seed + 50, w.size, 1.0, special=False).reshape(shape)
    wg = _gpu(w)
    y, mask = ops.qdq_mask_per_channel(wg, c, npc, *gp, *raw)
    assert torch.equal(y, ops.qdq_per_channel(wg, c, npc, *gp))
    gin = ops.ste_bwd_mask(mask, _gpu(grad)).cpu().numpy()
    want = oracle.ste_bwd_per_channel(w, grad, c, npc, enc_min.astype(np.float32), enc_max.astype(np.float32))
    assert np.array_equal(_bits(gin), _bits(want))
    assert 0.005 < (want == 0).mean() < 0.5
    wb, gb = torch.from_numpy(w).to(torch.bfloat16).cuda(), torch.from_numpy(grad).to(torch.bfloat16).cuda()
    yb, maskb = ops.qdq_mask_per_channel(wb, c, npc, *gp, *raw)
    assert torch.equal(yb.view(torch.int16), ops.qdq_per_channel(wb, c, npc, *gp).view(torch.int16))
    assert np.array_equal(_bf16_bits(ops.ste_bwd_mask(maskb, gb)),
                          _bf16_bits(ops.ste_bwd_per_channel(wb, gb, c, npc, *raw)))


@pytest.mark.parametrize("c,npc,outer", [(4, 6, 1), (7, 1, 3), (5, 9, 4), (3, 17, 5), (16, 20, 2), (33, 4100, 2),
                                         (8, 4096, 1), (64, 1030, 1), (2, 100003, 1)])
def test_per_channel_ragged(ops, oracle, c, npc, outer):
    n = outer * c * npc
    x = _normal(c * 1000 + npc, n, 0.3)
    rng = np.random.default_rng(c + npc)
    enc_min = -np.abs(rng.standard_normal(c)) * 0.4
    enc_max = np.abs(rng.standard_normal(c)) * 0.4
    params = oracle.per_channel_params(enc_min, enc_max, 8)
    gp = [_gpu(p) for p in params]
    raw = [_gpu(enc_min.astype(np.float32)), _gpu(enc_max.astype(np.float32))]
    y, mask = ops.qdq_mask_per_channel(_gpu(x), c, npc, *gp, *raw)
    assert np.array_equal(_bits(y.cpu().numpy()), _bits(oracle.qdq_per_channel(x, c, npc, params)))
    grad = _normal(n, n, 1.0, special=False)
    gin = ops.ste_bwd_mask(mask, _gpu(grad)).cpu().numpy()
    want = oracle.ste_bwd_per_channel(x, grad, c, npc, enc_min.astype(np.float32), enc_max.astype(np.float32))
    assert np.array_equal(_bits(gin), _bits(want))
    xb, gb = torch.from_numpy(x).to(torch.bfloat16).cuda(), torch.from_numpy(grad).to(torch.bfloat16).cuda()
    yb, maskb = ops.qdq_mask_per_channel(xb, c, npc, *gp, *raw)
    assert torch.equal(yb.view(torch.int16), ops.qdq_per_channel(xb, c, npc, *gp).view(torch.int16))
    assert np.array_equal(_bf16_bits(ops.ste_bwd_mask(maskb, gb)),
                          _bf16_bits(ops.ste_bwd_per_channel(xb, gb, c, npc, *raw)))


@pytest.mark.parametrize("qmin,qmax", [(0, 255), (-128, 127), (-8, 7)])
@pytest.mark.parametrize("c,npc,outer", [(1, 100003, 1), (512, 4608, 1), (64, 1030, 1), (7, 5, 3)])
def test_v2(ops, oracle, qmin, qmax, c, npc, outer):
    n = outer * c * npc
    x = _normal(qmax + c, n, 0.5)
    rng = np.random.default_rng(qmax * 7 + c)
    scale = (np.abs(rng.standard_normal(c)) * 0.01 + 1e-3).astype(np.float32)
    offset = -np.round(rng.uniform(0, qmax, c)).astype(np.float32) if qmin == 0 else np.zeros(c, np.float32)
    y, mask = ops.v2_qdq_mask(_gpu(x), c, npc, _gpu(scale), _gpu(offset), qmin, qmax)
    plain = ops.v2_qdq(_gpu(x), c, npc, _gpu(scale), _gpu(offset), qmin, qmax)
    assert torch.equal(y.view(torch.int32), plain.view(torch.int32))
    grad = _normal(n + 1, n, 1.0, special=False)
    gin = ops.ste_bwd_mask(mask, _gpu(grad)).cpu().numpy()
    assert np.array_equal(_bits(gin), _bits(oracle.v2_qdq_bwd(x, grad, c, npc, scale, offset, qmin, qmax)))
    _, _, omask = oracle.v2_qdq(x, c, npc, scale, offset, qmin, qmax)
    assert np.array_equal(decode_mask(mask, n, 4), np.asarray(omask).reshape(-1).astype(bool))
    xb, gb = torch.from_numpy(x).to(torch.bfloat16).cuda(), torch.from_numpy(grad).to(torch.bfloat16).cuda()
    yb, maskb = ops.v2_qdq_mask(xb, c, npc, _gpu(scale), _gpu(offset), qmin, qmax)
    assert torch.equal(yb.view(torch.int16), ops.v2_qdq(xb, c, npc, _gpu(scale), _gpu(offset), qmin, qmax)
                       .view(torch.int16))
    assert np.array_equal(_bf16_bits(ops.ste_bwd_mask(maskb, gb)),
                          _bf16_bits(ops.v2_qdq_bwd(xb, gb, c, npc, _gpu(scale), _gpu(offset), qmin, qmax)))


def test_v1_autograd_function_saves_the_mask(ops, oracle):
    """QuantizeDequantize keeps the mask instead of the input when the input wants a gradient: same output and same
    gradient as with save_mask = False, per tensor and per channel, float32 and bfloat16 (whose per-tensor bounds the
    reference's comparison rounds to bfloat16)."""
    from aimet_amd.common import libpymo
    from aimet_amd.common.defs import QuantScheme
    from aimet_amd.v1.tensor_quantizer import (QuantizeDequantize, StaticGridPerChannelQuantizer,
                                               StaticGridPerTensorQuantizer)
    nearest = libpymo.RoundingMode.ROUND_NEAREST
    torch.manual_seed(3)
    x = torch.randn(6, 32, 9, 9).cuda()
    pt = StaticGridPerTensorQuantizer(8, nearest, QuantScheme.post_training_tf, False, True)
    pt.update_encoding_stats(x * 0.6)
    pt.compute_encoding()
    # bounds that bfloat16 cannot hold: -0.4997 rounds to -0.5, so x = -0.5 is inside for the reference
    pt.encoding = libpymo.TfEncoding(-0.4997, 1.003, pt.encoding.delta, pt.encoding.offset, 8)
    pc = StaticGridPerChannelQuantizer(8, nearest, QuantScheme.post_training_tf, True, 32, True, ch_axis=1)
    pc.update_encoding_stats(x * 0.5)
    pc.compute_encoding()
    for q in (pt, pc):
        for dtype in (torch.float32, torch.bfloat16):
            xin = x.to(dtype)
            xin.view(-1)[:4] = torch.tensor([-0.5, 1.0, -0.4997, 1.003]).to(dtype)
            grad = torch.randn_like(xin)
            results = []
            for save in (True, False):
                QuantizeDequantize.save_mask = save
                try:
                    leaf = xin.clone().requires_grad_(True)
                    out = q.quantize_dequantize(leaf, nearest)
                    saved = out.grad_fn.saved_tensors
                    assert (saved[0].dtype == torch.int64) == save
                    out.backward(grad)
                    results.append((out.detach(), leaf.grad))
                finally:
                    QuantizeDequantize.save_mask = True
            for a, b in zip(*results):
                assert torch.equal(a.float().view(torch.int32), b.float().view(torch.int32))
            assert (results[0][1] == 0).float().mean() > 0.01
    # no gradient wanted: no mask is written
    with torch.no_grad():
        assert torch.equal(pt.quantize_dequantize(x, nearest), ops.qdq_per_tensor(x, -0.4997, 1.003, 8))
    # stochastic rounding keeps the input
    leaf = x.clone().requires_grad_(True)
    out = pt.quantize_dequantize(leaf, libpymo.RoundingMode.ROUND_STOCHASTIC)
    assert out.grad_fn.saved_tensors[0].dtype == torch.float32


def test_v2_backend_saves_the_mask():
    from aimet_amd.v2.quantization.affine.backends import hip_gfx950 as backend
    torch.manual_seed(4)
    x = torch.randn(40, 24, 5).cuda()
    scale = (torch.rand(24, 1) * 0.01 + 2e-3).cuda()
    offset = torch.zeros(24, 1).cuda()
    grad = torch.randn_like(x)
    results = []
    for save in (True, False):
        backend._QuantDequantFunc.save_mask = save          # pylint: disable=protected-access
        try:
            leaf = x.clone().requires_grad_(True)
            out = backend.quantize_dequantize(leaf, scale, offset, -8, 7)
            out.backward(grad)
            results.append((out.detach(), leaf.grad))
        finally:
            backend._QuantDequantFunc.save_mask = True      # pylint: disable=protected-access
    for a, b in zip(*results):
        assert torch.equal(a.view(torch.int32), b.view(torch.int32))
    assert 0.01 < (results[0][1] == 0).float().mean() < 0.99
    # learnable scale: the recomputing backward with the parameter sums
    s = scale.clone().requires_grad_(True)
    leaf = x.clone().requires_grad_(True)
    backend.quantize_dequantize(leaf, s, offset, -8, 7).backward(grad)
    assert torch.equal(leaf.grad.view(torch.int32), results[0][1].view(torch.int32)) and s.grad is not None
