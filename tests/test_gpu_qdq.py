"""GPU parity of the quantize-dequantize kernels against the CPU oracle, through the C ABI (aimet_amd.ops is a thin
ctypes layer).  Integer codes, dequantized float32 values and gradient masks must be bit-identical."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _bits(a):
    return np.ascontiguousarray(a, np.float32).view(np.uint32)


def _gpu(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def _normal(seed, shape, scale=1.0, special=True):
    rng = np.random.default_rng(seed)
    x = (rng.standard_normal(shape) * scale).astype(np.float32)
    if special and x.size >= 16:
        f = x.reshape(-1)
        f[:8] = [np.nan, np.inf, -np.inf, 0.0, -0.0, 1e-42, -1e-42, 3.4e38]
    return x


def _laplace_outliers(seed, shape):
    rng = np.random.default_rng(seed)
    u = rng.random(shape) - 0.5
    w = (-0.02 * np.sign(u) * np.log(1 - 2 * np.abs(u))).astype(np.float32)
    w[rng.random(shape) < 0.001] *= 20
    return w


@pytest.fixture(scope="module")
def ops():
    from aimet_amd import ops as o
    return o


# ------------------------------------------------------------------------------------------------- golden vectors
def test_golden_vectors_on_gpu(ops, vectors):
    for v in vectors["v1_per_tensor_qdq"]:
        y = ops.qdq_per_tensor(_gpu(np.array(v["x"], np.float32)), v["min"], v["max"], v["bw"]).cpu().numpy()
        assert np.allclose(y, np.array(v["y"], np.float32), rtol=5e-7, atol=0), v["source"]
    for v in vectors["v1_per_tensor_quantize"]:
        q = ops.quantize_per_tensor(_gpu(np.array(v["x"], np.float32)), v["min"], v["max"], v["bw"],
                                    v["shift_to_signed"]).cpu().numpy()
        assert np.array_equal(q, np.array(v["q"], np.float32)), v["source"]
    for v in vectors["v2_backend"]:
        x = np.array(v["tensor"], np.float32)
        scale = np.array(v["delta"], np.float32).reshape(-1)
        offset = np.array(v["offset"], np.float32).reshape(-1)
        c = scale.size
        npc = x.shape[1] if c > 1 else x.size
        y, q = ops.v2_qdq(_gpu(x), c, npc, _gpu(scale), _gpu(offset), v["qmin"], v["qmax"], want_codes=True)
        assert np.array_equal(q.cpu().numpy(), np.array(v["tensor_q"], np.int32)), v["name"]
        assert np.allclose(y.cpu().numpy(), np.array(v["tensor_qdq"], np.float32)), v["name"]
        g = ops.v2_qdq_bwd(_gpu(x), torch.ones_like(_gpu(x)), c, npc, _gpu(scale), _gpu(offset), v["qmin"],
                           v["qmax"]).cpu().numpy()
        clipped = np.array(v["clipped"], bool)
        assert np.all(g[clipped] == 0) and np.all(g[~clipped] == 1), v["name"]


# ---------------------------------------------------------------------------------------------------- per-tensor
@pytest.mark.parametrize("n", [1, 3, 4, 5, 1023, 4096, 4097, 65537, 1 << 20])
@pytest.mark.parametrize("bw", [4, 8, 16])
def test_per_tensor_sizes(ops, oracle, n, bw):
    x = _normal(n * 7 + bw, n, 1.5)
    mn, mx = -2.1, 3.3
    y = ops.qdq_per_tensor(_gpu(x), mn, mx, bw).cpu().numpy()
    assert np.array_equal(_bits(y), _bits(oracle.qdq_per_tensor(x, mn, mx, bw)))
    for shift in (False, True):
        q = ops.quantize_per_tensor(_gpu(x), mn, mx, bw, shift).cpu().numpy()
        assert np.array_equal(_bits(q), _bits(oracle.quantize_per_tensor(x, mn, mx, bw, shift)))


def test_per_tensor_empty_and_unaligned(ops, oracle):
    assert ops.qdq_per_tensor(torch.empty(0, device="cuda"), -1, 1, 8).numel() == 0
    x = _normal(5, 10001)
    base = _gpu(x)
    for off in (1, 2, 3):                       # views whose data pointer is not 16-byte aligned
        y = ops.qdq_per_tensor(base[off:], -1.0, 2.0, 8).cpu().numpy()
        assert np.array_equal(_bits(y), _bits(oracle.qdq_per_tensor(x[off:], -1.0, 2.0, 8)))


def test_per_tensor_ties_and_degenerate_ranges(ops, oracle):
    for (mn, mx) in ((-0.46, 0.72), (0.5, 1.0), (0.5, 0.5), (-0.5, -0.1), (-1e-7, 2e-7), (-3.0, 3.0), (0.0, 0.0)):
        for bw in (4, 8):
            e = oracle.fill_encoding_info(bw, mn, mx)
            k = np.arange(-3, 2 ** bw + 3)
            x = np.concatenate([(np.float32(e.delta) * (k + 0.5 + e.offset)).astype(np.float32),
                                (np.float32(e.delta) * (k + e.offset)).astype(np.float32),
                                _normal(bw, 5000, float(e.delta) * 60)])
            y = ops.qdq_per_tensor(_gpu(x), mn, mx, bw).cpu().numpy()
            assert np.array_equal(_bits(y), _bits(oracle.qdq_per_tensor(x, mn, mx, bw))), (mn, mx, bw)


def test_cfg1_activation_codes_and_mask(ops, oracle):
    """Per-tensor asymmetric int8 QDQ forward + STE backward on [32,64,56,56] ~N(0,1) with the min/max encoding."""
    shape = (32, 64, 56, 56)
    g = torch.Generator(device="cpu").manual_seed(1001)
    x = torch.randn(shape, generator=g)
    grad = torch.randn(shape, generator=torch.Generator().manual_seed(1101))
    xn = x.numpy()
    mnmx = ops.minmax(x.cuda()).cpu().numpy()
    omn, omx = oracle.minmax(xn)
    assert mnmx[0] == omn and mnmx[1] == omx
    enc = oracle.tf_compute_encoding(float(omn), float(omx), 8)
    y, codes = ops.qdq_codes_per_tensor(x.cuda(), enc.min, enc.max, 8, shift_to_signed=False)
    _, scodes = ops.qdq_codes_per_tensor(x.cuda(), enc.min, enc.max, 8, shift_to_signed=True, want_dequant=False)
    oq = oracle.quantize_per_tensor(xn, enc.min, enc.max, 8, False)
    assert np.array_equal(codes.cpu().numpy(), oq.astype(np.uint8))
    assert np.array_equal(scodes.cpu().numpy(), (oq - 128).astype(np.int8))
    assert np.array_equal(_bits(y.cpu().numpy()), _bits(oracle.qdq_per_tensor(xn, enc.min, enc.max, 8)))
    y2 = ops.qdq_per_tensor(x.cuda(), enc.min, enc.max, 8)
    assert torch.equal(y, y2)
    gin = ops.ste_bwd_per_tensor(x.cuda(), grad.cuda(), enc.min, enc.max).cpu().numpy()
    ogin = oracle.ste_bwd_per_tensor(xn, grad.numpy(), np.float32(enc.min), np.float32(enc.max))
    assert np.array_equal(_bits(gin), _bits(ogin))
    mask = gin != 0
    assert np.array_equal(mask, (np.float32(enc.min) <= xn) & (xn <= np.float32(enc.max)) & (grad.numpy() != 0))


def test_per_tensor_bf16(ops, oracle):
    x = torch.from_numpy(_normal(9, 200003, 2.0)).to(torch.bfloat16)
    bits = x.view(torch.int16).numpy().view(np.uint16)
    y = ops.qdq_per_tensor(x.cuda(), -3.0, 2.5, 8).cpu()
    assert np.array_equal(y.view(torch.int16).numpy().view(np.uint16), oracle.qdq_per_tensor_bf16(bits, -3.0, 2.5, 8))
    # STE backward in bf16 storage
    g = torch.from_numpy(_normal(10, 200003, 1.0, special=False)).to(torch.bfloat16)
    gin = ops.ste_bwd_per_tensor(x.cuda(), g.cuda(), -3.0, 2.5).cpu()
    xf, gf = x.float().numpy(), g.float().numpy()
    expect = oracle.ste_bwd_per_tensor(xf, gf, np.float32(-3.0), np.float32(2.5))
    assert np.array_equal(gin.float().numpy(), expect)


def test_unknown_rounding_mode_is_refused(ops):
    with pytest.raises(RuntimeError, match="rounding mode"):
        ops.qdq_per_tensor(torch.zeros(16, device="cuda"), -1, 1, 8, rounding_mode=2)


# --------------------------------------------------------------------------------------------------- per-channel
def _channel_case(oracle, w, c, npc, bw, sym=True):
    rows = w.reshape(c, npc)          # channel axis 0, no outer dimension
    enc_min = rows.min(axis=1).astype(np.float64)
    enc_max = rows.max(axis=1).astype(np.float64)
    encs = [oracle.tf_compute_encoding(enc_min[i], enc_max[i], bw, sym=sym) for i in range(c)]
    return np.array([e.min for e in encs]), np.array([e.max for e in encs])


@pytest.mark.parametrize("shape,axis_c", [((512, 512, 3, 3), 512), ((4096, 4096), 4096), ((11008, 4096), 11008)])
@pytest.mark.parametrize("bw", [8, 4])
def test_cfg2_weight_shapes(ops, oracle, shape, axis_c, bw):
    """Per-output-channel symmetric weight QDQ, int8/int4, fp32 and bf16, on the configured weight shapes."""
    seed = 1002 + {512: 0, 4096: 1, 11008: 2}[axis_c]
    w = _laplace_outliers(seed, shape)
    c, npc = shape[0], int(np.prod(shape[1:]))
    enc_min, enc_max = _channel_case(oracle, w, c, npc, bw)
    params = oracle.per_channel_params(enc_min, enc_max, bw)
    steps = 2 ** bw - 1 - (1 if enc_min[0] == -enc_max[0] else 0)
    gp = ops.per_channel_params(_gpu(enc_min.astype(np.float32)), _gpu(enc_max.astype(np.float32)), steps)
    for a, b in zip(gp, params):
        assert np.array_equal(_bits(a.cpu().numpy()), _bits(b))
    wg = _gpu(w)
    y, codes = ops.qdq_codes_per_channel(wg, c, npc, *gp, bw=bw)
    oy = oracle.qdq_per_channel(w, c, npc, params)
    oq = oracle.qdq_per_channel(w, c, npc, params, quantize_only=True)
    assert np.array_equal(codes.cpu().numpy().reshape(-1), oq.reshape(-1).astype(np.uint8))
    assert np.array_equal(_bits(y.cpu().numpy()), _bits(oy))
    assert torch.equal(ops.qdq_per_channel(wg, c, npc, *gp), y)
    # backward mask
    grad = _normal(seed + 50, shape, 1.0, special=False)
    emn, emx = enc_min.astype(np.float32), enc_max.astype(np.float32)
    gin = ops.ste_bwd_per_channel(wg, _gpu(grad), c, npc, _gpu(emn), _gpu(emx)).cpu().numpy()
    assert np.array_equal(_bits(gin), _bits(oracle.ste_bwd_per_channel(w, grad, c, npc, emn, emx)))
    # bf16 storage
    wb = torch.from_numpy(w).to(torch.bfloat16)
    bits = wb.view(torch.int16).numpy().view(np.uint16)
    yb = ops.qdq_per_channel(wb.cuda(), c, npc, *gp).cpu()
    assert np.array_equal(yb.view(torch.int16).numpy().view(np.uint16),
                          oracle.qdq_per_channel_bf16(bits, c, npc, params))
    _check_bf16_channel_backward(ops, oracle, wb, grad, c, npc, emn, emx)


def _bf16_bits(t):
    return t.contiguous().view(torch.int16).numpy().view(np.uint16)


def _check_bf16_channel_backward(ops, oracle, xb, grad, c, npc, emn, emx):
    """STE backward with bf16 storage: both inputs widen exactly to float32, grad * {0, 1} is exact, so the expected
    bf16 words are the oracle's float32 result on the widened inputs, narrowed (sign of zero included)."""
    gb = torch.from_numpy(np.ascontiguousarray(grad)).to(torch.bfloat16).reshape(xb.shape)
    gin = ops.ste_bwd_per_channel(xb.cuda(), gb.cuda(), c, npc, _gpu(emn), _gpu(emx)).cpu()
    want = oracle.ste_bwd_per_channel(xb.float().numpy(), gb.float().numpy(), c, npc, emn, emx)
    want_b = torch.from_numpy(np.ascontiguousarray(want)).to(torch.bfloat16).reshape(xb.shape)
    assert np.array_equal(_bf16_bits(gin), _bf16_bits(want_b))


@pytest.mark.parametrize("c,npc,outer", [(4, 6, 1), (7, 1, 3), (5, 9, 4), (3, 17, 5), (16, 20, 2), (33, 4100, 2),
                                         (8, 4096, 1), (64, 1030, 1), (2, 100003, 1)])
def test_per_channel_ragged(ops, oracle, c, npc, outer):
    """channel(i) = (i / npc) % C for every geometry: tiny channels, channels that are not a multiple of the vector
    width, an outer dimension in front of the channel axis."""
    n = outer * c * npc
    x = _normal(c * 1000 + npc, n, 0.3)
    rng = np.random.default_rng(c + npc)
    enc_min = -np.abs(rng.standard_normal(c)) * 0.4
    enc_max = np.abs(rng.standard_normal(c)) * 0.4
    params = oracle.per_channel_params(enc_min, enc_max, 8)
    gp = [_gpu(p) for p in params]
    y = ops.qdq_per_channel(_gpu(x), c, npc, *gp).cpu().numpy()
    assert np.array_equal(_bits(y), _bits(oracle.qdq_per_channel(x, c, npc, params)))
    grad = _normal(n, n, 1.0, special=False)
    gin = ops.ste_bwd_per_channel(_gpu(x), _gpu(grad), c, npc, gp[0], gp[1]).cpu().numpy()
    assert np.array_equal(_bits(gin), _bits(oracle.ste_bwd_per_channel(x, grad, c, npc, params[0], params[1])))
    xb = torch.from_numpy(x).to(torch.bfloat16)
    yb = ops.qdq_per_channel(xb.cuda(), c, npc, *gp).cpu()
    assert np.array_equal(yb.view(torch.int16).numpy().view(np.uint16),
                          oracle.qdq_per_channel_bf16(xb.view(torch.int16).numpy().view(np.uint16), c, npc, params))
    _check_bf16_channel_backward(ops, oracle, xb, grad, c, npc, params[0], params[1])


def test_reference_per_channel_vectors(ops, oracle, vectors):
    for v in vectors["v1_per_channel_qdq"]:
        x = np.array(v["x"], np.float32)
        steps = 255 - (1 if v["enc_min"][0] == -v["enc_max"][0] else 0)
        gp = ops.per_channel_params(_gpu(np.array(v["enc_min"], np.float32)),
                                    _gpu(np.array(v["enc_max"], np.float32)), steps)
        y = ops.qdq_per_channel(_gpu(x), 4, 6, *gp).cpu().numpy()
        assert np.allclose(y, np.array(v["y"], np.float32), atol=v["atol"], rtol=0), v["source"]


def test_broadcast(ops, oracle):
    rng = np.random.default_rng(21)
    shape = (3, 8, 5, 4)
    x = _normal(22, int(np.prod(shape)))
    strides = [160, 20, 4, 1]
    for enc_shape in ((1, 8, 1, 1), (3, 1, 1, 4), (1, 1, 1, 1), (1, 8, 5, 1)):
        n_enc = int(np.prod(enc_shape))
        est, acc = [], 1
        for d in reversed(enc_shape):
            est.append(acc if d > 1 else 0)
            acc *= d
        est = est[::-1]
        params = oracle.per_channel_params(-np.abs(rng.standard_normal(n_enc)), np.abs(rng.standard_normal(n_enc)), 8)
        y = ops.qdq_broadcast(_gpu(x), strides, est, *[_gpu(p) for p in params]).cpu().numpy()
        assert np.array_equal(_bits(y), _bits(oracle.qdq_broadcast(x, strides, est, params)))


@pytest.mark.parametrize("shape,enc_shape", [
    ((6, 64, 7, 9), (1, 64, 1, 1)),        # per channel on axis 1 with an outer axis: (e / run) % channels
    ((96, 33, 3, 3), (96, 1, 1, 1)),       # per output channel
    ((48, 4, 128), (48, 4, 1)),            # blocks of 128 along the last axis of a [48, 512] tensor
    ((5, 12, 10, 6), (1, 12, 10, 1)),      # two adjacent varying axes
    ((4, 6, 10, 8), (4, 1, 10, 1)),        # varying axes that are not adjacent: the general kernel
    ((7, 1, 5, 3), (1, 1, 5, 3)),          # the encoding covers the trailing axes
    ((1000,), (1,)),
])
def test_broadcast_layouts(ops, oracle, shape, enc_shape):
    """Broadcast layouts that the library maps onto its [outer, channel, run] vector kernel, and one that it cannot:
    the result is the restatement's, bit for bit, either way (reference DlQuantization/src/trim_functions.cpp:634-660)."""
    rng = np.random.default_rng(len(shape) * 100 + shape[0])
    x = (rng.standard_normal(int(np.prod(shape))) * 1.5).astype(np.float32)
    strides, acc = [], 1
    for d in reversed(shape):
        strides.append(acc)
        acc *= d
    strides = strides[::-1]
    est, acc = [], 1
    for d in reversed(enc_shape):
        est.append(acc if d > 1 else 0)
        acc *= d
    est = est[::-1]
    n_enc = int(np.prod(enc_shape))
    params = oracle.per_channel_params(-np.abs(rng.standard_normal(n_enc)) - 0.1, np.abs(rng.standard_normal(n_enc)) + 0.1,
                                       8)
    y = ops.qdq_broadcast(_gpu(x), strides, est, *[_gpu(p) for p in params]).cpu().numpy()
    assert np.array_equal(_bits(y), _bits(oracle.qdq_broadcast(x, strides, est, params)))


# ------------------------------------------------------------------------------------------------------------ v2
@pytest.mark.parametrize("qmin,qmax", [(0, 255), (-128, 127), (-8, 7), (0, 15)])
@pytest.mark.parametrize("c,npc,outer", [(1, 100003, 1), (512, 4608, 1), (64, 1030, 1), (7, 5, 3)])
def test_v2_qdq_fwd_bwd(ops, oracle, qmin, qmax, c, npc, outer):
    n = outer * c * npc
    x = _normal(qmax + c, n, 0.5)
    rng = np.random.default_rng(qmax * 7 + c)
    scale = (np.abs(rng.standard_normal(c)) * 0.01 + 1e-3).astype(np.float32)
    offset = -np.round(rng.uniform(0, qmax, c)).astype(np.float32) if qmin == 0 else np.zeros(c, np.float32)
    x[100:100 + min(64, n - 100)] = (scale[0] * (np.arange(min(64, n - 100)) - 32 + 0.5)).astype(np.float32)  # ties
    y, q = ops.v2_qdq(_gpu(x), c, npc, _gpu(scale), _gpu(offset), qmin, qmax, want_codes=True)
    oy, oq, om = oracle.v2_qdq(x, c, npc, scale, offset, qmin, qmax)
    yn = y.cpu().numpy()
    nan = np.isnan(oy)
    assert np.array_equal(np.isnan(yn), nan)
    assert np.array_equal(_bits(yn)[~nan], _bits(oy)[~nan])
    assert np.array_equal(q.cpu().numpy()[~nan], oq[~nan].astype(np.int32))
    grad = _normal(n + 1, n, 1.0, special=False)
    gin = ops.v2_qdq_bwd(_gpu(x), _gpu(grad), c, npc, _gpu(scale), _gpu(offset), qmin, qmax).cpu().numpy()
    assert np.array_equal(_bits(gin), _bits(oracle.v2_qdq_bwd(x, grad, c, npc, scale, offset, qmin, qmax)))
    xb = torch.from_numpy(x).to(torch.bfloat16)
    yb = ops.v2_qdq(xb.cuda(), c, npc, _gpu(scale), _gpu(offset), qmin, qmax).cpu()
    ob, _ = oracle.v2_qdq_bf16(xb.view(torch.int16).numpy().view(np.uint16), c, npc, scale, offset, qmin, qmax)
    assert np.array_equal(yb.view(torch.int16).numpy().view(np.uint16), ob)


def test_v2_rejects_bad_grid(ops):
    x = torch.zeros(16, device="cuda")
    s, o = torch.ones(1, device="cuda"), torch.zeros(1, device="cuda")
    with pytest.raises(RuntimeError, match="qmin"):
        ops.v2_qdq(x, 1, 16, s, o, 5, 3)
    with pytest.raises(RuntimeError, match="represent"):
        ops.v2_qdq(x, 1, 16, s, o, 0, 1 << 25)


# ---------------------------------------------------------------------------------------- properties at full size
def test_idempotence_and_grid_membership_full_size(ops):
    """Size-independent properties at the largest configured weight shape: QDQ is idempotent and every output is
    delta * integer with the integer inside the grid."""
    c, npc = 11008, 4096
    w = torch.from_numpy(_laplace_outliers(3, (c, npc))).cuda()
    mm = ops.minmax_per_channel(w, c, npc)
    amax = torch.maximum(mm[0].abs(), mm[1].abs())
    delta = amax / 127
    gp = ops.per_channel_params(-128 * delta, 127 * delta, 255)
    y = ops.qdq_per_channel(w, c, npc, *gp)
    assert torch.equal(ops.qdq_per_channel(y, c, npc, *gp), y)
    k = (y.double() / gp[2].double().unsqueeze(1))
    assert torch.all((k - k.round()).abs() < 1e-3)
    assert k.round().min() >= -128 and k.round().max() <= 127
    assert torch.equal(mm[0], w.min(dim=1).values) and torch.equal(mm[1], w.max(dim=1).values)


def test_more_than_2_31_elements(ops, oracle):
    """Maximum sizes: 2^31 + 4099 elements (64-bit indexing in the kernels and in the channel arithmetic); slices at
    the start, across the 2^31 boundary and at the end are compared with the oracle."""
    n = (1 << 31) + 4099
    free, _ = torch.cuda.mem_get_info()
    if free < 3 * 4 * n:
        pytest.skip("not enough device memory for a 2^31-element round trip")
    g = torch.Generator(device="cuda").manual_seed(9)
    x = torch.empty(n, device="cuda")
    chunk = 1 << 28
    for s in range(0, n, chunk):
        x[s:s + chunk].normal_(generator=g)
    spans = [(0, 100000), ((1 << 31) - 50000, (1 << 31) + 4099), (n - 70001, n)]
    y = ops.qdq_per_tensor(x, -2.5, 3.0, 8)
    for a, b in spans:
        xs = x[a:b].cpu().numpy()
        assert np.array_equal(y[a:b].cpu().numpy().view(np.uint32), oracle.qdq_per_tensor(xs, -2.5, 3.0, 8).view(np.uint32))
    gx = ops.ste_bwd_per_tensor(x, y, -2.5, 3.0)
    for a, b in spans:
        assert np.array_equal(gx[a:b].cpu().numpy(),
                              oracle.ste_bwd_per_tensor(x[a:b].cpu().numpy(), y[a:b].cpu().numpy(),
                                                        np.float32(-2.5), np.float32(3.0)))
    del y, gx
    # per-channel: 7 channels of 613 consecutive elements, repeating (channel = (i / 613) % 7)
    C, npc = 7, 613
    emin = np.linspace(-3, -1, C).astype(np.float32)
    emax = np.linspace(1, 3.5, C).astype(np.float32)
    params = oracle.per_channel_params(emin, emax, 8)
    gp = ops.per_channel_params(torch.from_numpy(emin).cuda(), torch.from_numpy(emax).cuda(), 255)
    yc = ops.qdq_per_channel(x, C, npc, *gp)
    for a, b in spans:
        a0 = a - a % (C * npc)                      # start on a channel-0 boundary so the oracle sees the same phase
        xs = x[a0:b].cpu().numpy()
        want = oracle.qdq_per_channel(xs, C, npc, params)
        assert np.array_equal(yc[a0:b].cpu().numpy().view(np.uint32), want.view(np.uint32))


def test_kernels_run_on_torch_current_stream(ops, oracle):
    """The entry points take a stream; the Python layer passes torch's current one.  On a side stream the input is
    written after a long sleep kernel: a launch on any other stream would read the tensor before that write."""
    n = 1 << 20
    side = torch.cuda.Stream()
    x = torch.zeros(n, device="cuda")
    g = torch.ones(n, device="cuda")
    torch.cuda.synchronize()
    with torch.cuda.stream(side):
        torch.cuda._sleep(100_000_000)                   # tens of milliseconds on this stream only
        x.fill_(0.7)
        y = ops.qdq_per_tensor(x, -1.0, 1.0, 8)
        gin = ops.ste_bwd_per_tensor(x * 2, g, -1.0, 1.0)
        an = ops.Analyzer(1)
        an.update_stats(x)
        mm = ops.minmax(x)
    assert not side.query()                              # nothing above waited for the device
    side.synchronize()
    want = oracle.qdq_per_tensor(np.full(4, 0.7, np.float32), -1.0, 1.0, 8)[0]
    assert torch.equal(y, torch.full_like(y, float(want)))
    assert gin.sum().item() == 0                         # 1.4 lies outside [-1, 1]
    assert mm.tolist() == [pytest.approx(0.7), pytest.approx(0.7)]
    xl, pdf = an.get_stats_histogram()
    assert pdf.sum() == pytest.approx(1.0) and (pdf > 0).sum() == 1


# ------------------------------------------------------------------------------------- several tensors in one launch
def test_multi_tensor_launch(ops, oracle):
    """One launch over a table of tensors: every tensor's result is that of its own per-channel call (and the
    oracle's), for ragged shapes, a per-tensor encoding (one channel), an outer axis, bf16; what cannot take part is
    refused."""
    rng = np.random.default_rng(77)
    shapes = [((64, 3, 7, 7), 64, 147), ((256, 64, 1, 1), 256, 64), ((96, 33, 3, 3), 96, 297), ((1000, 2048), 1000, 2048),
              ((5, 4099), 5, 4099), ((3, 8, 50), 8, 50), ((7, 6001), 1, 42007), ((16, 9), 16, 9)]
    entries, want = [], []
    for k, (shape, c, npc) in enumerate(shapes):
        x = _normal(300 + k, shape, 0.3)
        enc_min = -np.abs(rng.standard_normal(c)) * 0.4
        enc_max = np.abs(rng.standard_normal(c)) * 0.4
        params = oracle.per_channel_params(enc_min, enc_max, 8 if k % 2 else 4)
        entries.append((_gpu(x), c, npc, *[_gpu(p) for p in params]))
        want.append(oracle.qdq_per_channel(x, c, npc, params))
    multi = ops.QdqMulti(entries)
    for _ in range(2):                       # the prepared launch is reusable
        outs = multi()
        for e, out, w in zip(entries, outs, want):
            assert np.array_equal(_bits(out.cpu().numpy()), _bits(w))
            assert torch.equal(out, ops.qdq_per_channel(e[0], e[1], e[2], *e[3:7]))
        for out in outs:
            out.zero_()
    # bf16 storage
    bentries = [(e[0].to(torch.bfloat16), *e[1:]) for e in entries[:-1]]    # 9 elements per channel: too few for bf16
    bouts = ops.QdqMulti(bentries)()
    for e, out in zip(bentries, bouts):
        assert torch.equal(out.view(torch.int16), ops.qdq_per_channel(e[0], e[1], e[2], *e[3:7]).view(torch.int16))
    # tiny channels / unaligned data cannot take part
    x = _gpu(_normal(1, (40, 4), 1.0))
    p4 = [_gpu(p) for p in oracle.per_channel_params(-np.ones(40), np.ones(40), 8)]
    with pytest.raises(RuntimeError, match="multi-tensor"):
        ops.QdqMulti([(x, 40, 4, *p4)])
    base = _gpu(_normal(2, 4097, 1.0))
    p1 = [_gpu(p) for p in oracle.per_channel_params(-np.ones(1), np.ones(1), 8)]
    with pytest.raises(RuntimeError, match="multi-tensor"):
        ops.QdqMulti([(base[1:], 1, 4096, *p1)])
