"""Pins the CPU oracle (oracle/miq_oracle.c) to the known answers the reference's own tests hold.

Every expected value here comes from tests/golden/reference_vectors.json (transcribed data, with the reference
file:line of each vector) or from a closed form the mathematics fixes; nothing re-types the oracle's formulas.
"""
import math

import numpy as np
import pytest


def _ulp_diff(a, b):
    a = np.asarray(a, np.float32).view(np.int32).astype(np.int64)
    b = np.asarray(b, np.float32).view(np.int32).astype(np.int64)
    a = np.where(a < 0, -(a & 0x7fffffff), a)
    b = np.where(b < 0, -(b & 0x7fffffff), b)
    return np.abs(a - b)


# ---------------------------------------------------------------------------------------------------- per-tensor
def test_v1_per_tensor_qdq_golden(oracle, vectors):
    for v in vectors["v1_per_tensor_qdq"]:
        y = oracle.qdq_per_tensor(np.array(v["x"], np.float32), v["min"], v["max"], v["bw"])
        # the reference asserts EXPECT_FLOAT_EQ, i.e. within 4 ulp
        assert _ulp_diff(y, np.array(v["y"], np.float32)).max() <= v["ulp"], v["source"]


def test_v1_per_tensor_qdq_first_vector_bits(oracle, vectors):
    # Bit patterns observed from the compiled reference for the first vector set (min -0.46, max 0.72, bw 8).
    v = vectors["v1_per_tensor_qdq"][0]
    y = oracle.qdq_per_tensor(np.array(v["x"], np.float32), v["min"], v["max"], v["bw"])
    assert [hex(b) for b in y.view(np.uint32)] == ["0xbeea8e65", "0xbe7fe128", "0x0", "0x3e7fe128", "0x3effe128",
                                                   "0x3f38cd48"]


def test_v1_per_tensor_quantize_golden(oracle, vectors):
    for v in vectors["v1_per_tensor_quantize"]:
        q = oracle.quantize_per_tensor(np.array(v["x"], np.float32), v["min"], v["max"], v["bw"],
                                       v["shift_to_signed"])
        assert np.array_equal(q, np.array(v["q"], np.float32)), v["source"]


def test_fill_encoding_info_golden(oracle, vectors):
    for v in vectors["fill_encoding_info"]:
        e = oracle.fill_encoding_info(v["bw"], v["min"], v["max"])
        # EXPECT_DOUBLE_EQ = 4 ulp of double
        assert e.min == pytest.approx(v["exp_min"], rel=1e-15)
        assert e.max == pytest.approx(v["exp_max"], rel=1e-15)


def test_tf_encoding_then_quantize_golden(oracle, vectors):
    v = vectors["tf_encoding_quantize"]
    x = np.array(v["x"], np.float32)
    mn, mx = oracle.minmax(x)
    enc = oracle.tf_compute_encoding(float(mn), float(mx), v["bw"])
    # expected encoding is the reference helper getTfEncoding(-50, 80, 8): closed form, not the oracle's code
    lo, hi = v["encoding_from"]
    delta = (hi - lo) / 255.0
    offset = float(np.round(lo / delta))
    assert enc.delta == pytest.approx(delta, rel=1e-15)
    assert enc.offset == offset
    assert enc.min == pytest.approx(delta * offset, rel=1e-15)
    assert enc.max == pytest.approx(delta * 255 + delta * offset, rel=1e-14)
    q = oracle.quantize_per_tensor(x, enc.min, enc.max, v["bw"], False)
    assert np.array_equal(q, np.array(v["codes"], np.float32))
    y = oracle.qdq_per_tensor(x, enc.min, enc.max, v["bw"])
    assert np.allclose(y, np.array(v["dequant"], np.float32), atol=v["dequant_atol"])


def _data2():
    return (-15 + 0.5 * np.arange(60)).astype(np.float32).reshape(1, 4, 5, 3)


def test_tf_per_slice_qdq_golden(oracle, vectors):
    g = vectors["tf_per_slice_qdq"]
    x = _data2()
    # asymmetric, one TF encoding per slice along the axis
    for key, sym in (("asymmetric", False), ("symmetric", True)):
        v = g[key]
        out = np.empty_like(x)
        for c in range(x.shape[v["axis"]]):
            sl = np.take(x, c, axis=v["axis"])
            mn, mx = oracle.minmax(sl)
            enc = oracle.tf_compute_encoding(float(mn), float(mx), 8, sym=sym, strict=sym, unsigned_sym=False)
            y = oracle.qdq_per_tensor(sl, enc.min, enc.max, 8)
            idx = [slice(None)] * 4
            idx[v["axis"]] = c
            out[tuple(idx)] = y
        assert np.allclose(out.reshape(-1), np.array(v["y"], np.float32), atol=v["atol"]), v["source"]


def test_tf_per_slice_packed_codes_golden(oracle, vectors):
    g = vectors["tf_per_slice_qdq"]
    x = _data2()
    v = g["packed_asymmetric_codes"]
    codes = []
    for c in range(4):
        sl = np.ascontiguousarray(x[:, c])
        mn, mx = oracle.minmax(sl)
        enc = oracle.tf_compute_encoding(float(mn), float(mx), 8)
        assert (enc.min, enc.max) == pytest.approx(_tf_helper(*v["slice_minmax"][c]), rel=1e-12)
        codes.append(oracle.quantize_per_tensor(sl, enc.min, enc.max, 8, False).reshape(-1))
    assert np.array_equal(np.concatenate(codes), np.array(v["q"], np.float32)), v["source"]
    v = g["packed_symmetric_codes"]
    codes = []
    for c in range(4):
        sl = np.ascontiguousarray(x[:, c])
        mn, mx = oracle.minmax(sl)
        enc = oracle.tf_compute_encoding(float(mn), float(mx), 8, sym=True, strict=True)
        # getTfSymmetricEncoding(absmax, 8): delta = absmax / 127, offset -127
        assert enc.delta == pytest.approx(v["slice_absmax"][c] / 127.0, rel=1e-15)
        assert enc.offset == -127
        codes.append(oracle.quantize_per_tensor(sl, enc.min, enc.max, 8, False).reshape(-1))
    # The reference's packed signed path stores grid index + offset (offset = -127 on the strict-symmetric grid),
    # so the vector pins the unsigned grid index of the hot-path quantizer, not its 2^(bw-1) shift.
    assert np.array_equal(np.concatenate(codes) - 127, np.array(v["q"], np.float32)), v["source"]


def _tf_helper(lo, hi, bw=8):
    steps = 2 ** bw - 1
    delta = (hi - lo) / steps
    offset = float(np.round(lo / delta)) if lo / delta % 1 != 0.5 else math.copysign(math.floor(abs(lo / delta) + 0.5),
                                                                                    lo)
    mn = delta * offset
    return mn, delta * steps + mn


# --------------------------------------------------------------------------------------------------- per-channel
def test_v1_per_channel_qdq_golden(oracle, vectors):
    for v in vectors["v1_per_channel_qdq"]:
        x = np.array(v["x"], np.float32)
        params = oracle.per_channel_params(v["enc_min"], v["enc_max"], v["bw"])
        y = oracle.qdq_per_channel(x, x.shape[0], x.shape[1], params)
        assert np.allclose(y, np.array(v["y"], np.float32), atol=v["atol"], rtol=0), v["source"]


def test_v1_per_channel_params_closed_form(oracle, vectors):
    v = vectors["v1_per_channel_qdq"][0]
    mn, mx, delta, offset = oracle.per_channel_params(v["enc_min"], v["enc_max"], 8)
    # the reference test states delta 0.03 / 0.05 and offset -128 for these encodings
    assert np.allclose(delta, [0.03, 0.03, 0.03, 0.05], atol=1e-7)
    assert np.array_equal(offset, np.full(4, -128, np.float32))
    v = vectors["v1_per_channel_qdq"][1]
    mn, mx, delta, offset = oracle.per_channel_params(v["enc_min"], v["enc_max"], 8)
    assert np.array_equal(offset, np.array([-153, -153, -153, -182], np.float32))


def test_tf_per_channel_encodings_golden(oracle, vectors):
    v = vectors["tf_per_channel_encodings"]
    x = np.array(v["x"], np.float32)
    encs = []
    for sym in (True, False):
        row = []
        for c in range(4):
            mn, mx = oracle.minmax(x[c])
            row.append(oracle.tf_compute_encoding(float(mn), float(mx), 8, sym=sym))
        encs.append(row)
    s, a = encs
    assert s[0].max == v["symmetric"]["ch0_max"] and round(s[0].min, 2) == v["symmetric"]["ch0_min_round2"]
    assert s[3].max == v["symmetric"]["ch3_max"] and round(s[3].min, 2) == v["symmetric"]["ch3_min_round2"]
    assert round(a[0].max, 3) == v["asymmetric"]["ch0_max_round3"]
    assert round(a[0].min, 3) == v["asymmetric"]["ch0_min_round3"]
    assert round(a[3].max, 3) == v["asymmetric"]["ch3_max_round3"]
    assert round(a[3].min, 3) == v["asymmetric"]["ch3_min_round3"]


# -------------------------------------------------------------------------------------------------- STE backward
def test_ste_backward_golden(oracle, vectors):
    v = vectors["ste_backward"]
    for case in v["cases"]:
        x = np.array(case["x"], np.float32)
        g = np.ones_like(x)
        got = oracle.ste_bwd_per_tensor(x, g, v["min"], v["max"])
        assert np.array_equal(got, np.array(case["grad"], np.float32))
        got = oracle.ste_bwd_per_channel(x, g, 2, 2, [v["min"]] * 2, [v["max"]] * 2)
        assert np.array_equal(got, np.array(case["grad"], np.float32))


# ---------------------------------------------------------------------------------------------------- TF / TF-Enh
def test_tf_encoding_bw6_golden(oracle, vectors):
    v = vectors["tf_encoding_bw6"]
    e = oracle.tf_compute_encoding(v["min"], v["max"], v["bw"])
    assert e.delta == pytest.approx(v["delta"], abs=v["atol"])
    assert e.offset == v["offset"]
    assert e.min == pytest.approx(v["exp_min"], abs=v["atol"])
    assert e.max == pytest.approx(v["exp_max"], abs=v["atol"])


def test_tf_symmetric_invariants(oracle):
    # DLQT/TestTfEncodingAnalyzer.cpp:55-295: offsets -128 / -127 / 0 and zero exactly representable
    rng = np.random.default_rng(0)
    for _ in range(50):
        lo, hi = sorted(rng.normal(0, 5, 2))
        e = oracle.tf_compute_encoding(lo, hi, 8, sym=True)
        if lo < 0:
            assert e.offset == -128 and e.delta == pytest.approx(max(abs(lo), abs(hi), 0.0) / 127) or hi - lo < 0.01
        e = oracle.tf_compute_encoding(lo, hi, 8, sym=True, strict=True)
        assert e.offset == -127 and e.min == -e.max
        e = oracle.tf_compute_encoding(abs(lo), abs(lo) + abs(hi), 8, sym=True, unsigned_sym=True)
        assert e.offset == 0 and e.min == 0
        e = oracle.tf_compute_encoding(lo, hi, 8)
        assert abs(e.min + e.delta * (-e.offset)) < 1e-7


def test_tf_enhanced_n22_golden(oracle, vectors, n22):
    v = vectors["tf_enhanced_n22"]
    pdf = oracle.new_pdf()
    hist = pdf.update(n22)
    assert int(hist.sum()) == n22.size           # widened range: nothing dropped on the first batch
    enc, costs, best = pdf.compute_encoding(v["bw"])
    assert enc.min == pytest.approx(v["exp_min"], abs=v["atol"])
    assert enc.max == pytest.approx(v["exp_max"], abs=v["atol"])
    y = oracle.qdq_per_tensor(np.array([5.0], np.float32), enc.min, enc.max, 8)
    assert float(y[0]) == pytest.approx(v["qdq_of_5"], abs=1e-3)
    # values observed from the compiled reference (float results, so exact in binary32)
    assert np.float32(enc.min) == np.float32(-6.52710772)
    assert np.float32(enc.max) == np.float32(8.88411903)
    assert np.float32(enc.delta) == np.float32(0.0604361817)
    assert enc.offset == -108
    assert np.float32(pdf.x_left()[0]) == np.float32(-22.0508747)
    assert np.float32(pdf.x_left()[1]) == np.float32(-21.9602204)
    assert pdf.pdf().sum() == pytest.approx(1.0, abs=1e-12)


def test_tf_enhanced_all_zeros_golden(oracle, vectors):
    v = vectors["tf_enhanced_all_zeros"]
    pdf = oracle.new_pdf()
    pdf.update(np.zeros(1000, np.float32))
    assert not pdf.initialized
    enc, _, _ = pdf.compute_encoding(v["bw"])
    assert enc.min == pytest.approx(v["exp_min"], abs=v["atol"])
    assert enc.max == pytest.approx(v["exp_max"], abs=v["atol"])
    assert enc.offset == v["offset"]


def test_tf_enhanced_no_stats_is_invalid(oracle):
    enc, _, _ = oracle.new_pdf().compute_encoding(8)
    assert enc.astuple() == (0, 0, 0, 0, 0)


def test_tf_enhanced_constant_tensors(oracle):
    # DLQT/TestTfEnhancedEncodingAnalyzer.cpp:141-174
    pdf = oracle.new_pdf()
    pdf.update(np.full(100, 4.0, np.float32))
    enc, _, _ = pdf.compute_encoding(8)
    assert enc.max >= 3.5 and enc.min <= 0
    pdf = oracle.new_pdf()
    pdf.update(np.full(100, -5.0, np.float32))
    enc, _, _ = pdf.compute_encoding(8)
    assert enc.min <= -4.5


def test_tf_enhanced_symmetric_modes(oracle, n22):
    # DLQT/TestTfEnhancedEncodingAnalyzer.cpp:199-345
    pdf = oracle.new_pdf()
    pdf.update(n22)
    e, _, _ = pdf.compute_encoding(8, sym=True)
    assert e.offset == -128 and e.delta == pytest.approx((e.max - e.min) / 255, rel=1e-6)
    e, _, _ = pdf.compute_encoding(8, sym=True, strict=True)
    assert e.offset == -127 and e.min == -e.max and e.delta == pytest.approx((e.max - e.min) / 254, rel=1e-6)
    pdf = oracle.new_pdf()
    pos = np.abs(n22)
    pdf.update(pos)
    e, _, _ = pdf.compute_encoding(8, sym=True, unsigned_sym=True)
    assert e.min == 0 and e.offset == 0
    d, o = pdf.candidates(8, sym=True)
    assert len(d) == 101      # float accumulation of 0.01 yields 101 deltas
    d, o = pdf.candidates(8)
    assert len(d) <= 17 * 21 + 1


def test_tf_enhanced_cost_brute_force(oracle):
    """The cost of one candidate, recomputed from its definition by expanding the PDF into samples.

    With gamma = 3 the cost is sum_i pdf_i * w_i * (mid_i - qdq(mid_i))^2, where saturated buckets use the middle of
    the clip bucket; build it with plain float64 numpy on a 512-bucket PDF whose range makes all quantities exact
    enough for a 1e-9 relative comparison."""
    x = np.linspace(-1.0, 3.0, 4001, dtype=np.float32)
    pdf = oracle.new_pdf()
    pdf.update(x)
    xl, p = pdf.x_left(), pdf.pdf()
    step = xl[1] - xl[0]
    start = float(np.float32(xl[0]))
    mids = start + np.arange(512) * step + step / 2
    delta, offset, bw = np.float32(0.01), -60, 8
    lo, hi = float(delta) * offset, float(delta) * (offset + 255)
    min_ind = int(np.clip(math.floor((np.float32(lo) - np.float32(start)) / step), 0, 511))
    max_ind = int(np.clip(math.floor((np.float32(np.float32(delta) * np.float32(offset + 255)) - np.float32(start)) / step), 0, 511))
    cost = 0.0
    for i in range(512):
        if i < min_ind:
            cost += 3 * p[i] * (mids[i] - float(np.float32(start + min_ind * step + step / 2))) ** 2
        elif i >= max_ind:
            cost += 3 * p[i] * (mids[i] - float(np.float32(start + max_ind * step + step / 2))) ** 2
        else:
            fv = np.float32(mids[i])
            q = np.floor(np.abs(fv / delta - np.float32(offset)) + np.float32(0.5)) * np.sign(fv / delta - np.float32(offset))
            dq = delta * np.float32(q + offset)
            cost += p[i] * float(fv - dq) ** 2
    assert pdf.cost(bw, delta, offset) == pytest.approx(cost, rel=1e-9)


def test_histogram_invariants(oracle):
    rng = np.random.default_rng(3)
    x = rng.normal(0, 1, 100000).astype(np.float32)
    pdf = oracle.new_pdf()
    h1 = pdf.update(x)
    assert h1.sum() == x.size
    # a second batch with outliers beyond the 3x widened range: those samples are dropped
    y = x.copy()
    y[:10] = 1e6
    y[10:15] = np.nan
    h2 = pdf.update(y)
    assert h2.sum() == x.size - 15
    # bin counts do not depend on element order
    h3 = oracle.new_pdf()
    h3.update(x)
    perm = rng.permutation(x.size)
    h4 = oracle.new_pdf()
    assert np.array_equal(h4.update(x[perm]), h1)
    # direct numpy restatement of the bucket index with the same float32 operations
    bucket = np.float32(pdf.x_left()[1] - pdf.x_left()[0])
    off = np.float32(pdf.x_left()[0]) / bucket
    t = x / bucket - off
    idx = (np.sign(t) * np.floor(np.abs(t) + np.float32(0.5))).astype(np.int64)
    ref = np.bincount(idx[(idx >= 0) & (idx < 512)], minlength=512)
    assert np.array_equal(ref.astype(np.uint32), h1)


# ------------------------------------------------------------------------------------------------------------ v2
def test_v2_backend_golden(oracle, vectors):
    for v in vectors["v2_backend"]:
        x = np.array(v["tensor"], np.float32)
        scale = np.array(v["delta"], np.float32).reshape(-1)
        offset = np.array(v["offset"], np.float32).reshape(-1)
        c = scale.size
        npc = x.shape[1] if c > 1 else x.size
        y, q, mask = oracle.v2_qdq(x, c, npc, scale, offset, v["qmin"], v["qmax"])
        assert np.array_equal(q, np.array(v["tensor_q"], np.float32)), v["name"]
        assert np.allclose(y, np.array(v["tensor_qdq"], np.float32)), v["name"]
        # the reference's `mask` field marks CLIPPED positions: gradient must be zero exactly there
        clipped = np.array(v["clipped"], bool)
        g = oracle.v2_qdq_bwd(x, np.ones_like(x), c, npc, scale, offset, v["qmin"], v["qmax"])
        assert np.all(g[clipped] == 0) and np.all(g[~clipped] == 1), v["name"]
        assert np.array_equal(mask.astype(bool), ~clipped), v["name"]
        if v["bf16_exact"]:
            xb = oracle.f32_to_bf16_bits(x)
            assert np.array_equal(oracle.bf16_bits_to_f32(xb), x)
            yb, _ = oracle.v2_qdq_bf16(xb, c, npc, scale, offset, v["qmin"], v["qmax"])
            assert np.array_equal(oracle.bf16_bits_to_f32(yb), np.array(v["tensor_qdq"], np.float32)), v["name"]


def test_v2_docstring_example(oracle):
    # TORCH/v2/quantization/affine/backends/__init__.py:297-323: scale 1/15, 4-bit unsigned, x = arange(-0.5..1.5)
    import torch
    x = torch.arange(start=-0.3, end=1.3, step=0.05)
    scale, offset = np.float32(1 / 15), np.float32(0)
    y, q, _ = oracle.v2_qdq(x.numpy(), 1, x.numel(), [scale], [offset], 0, 15)
    expect = ((torch.round(x / torch.tensor(1 / 15)) - 0).clamp(0, 15) + 0) * torch.tensor(1 / 15)
    assert np.array_equal(y, expect.numpy())


def test_v2_matches_torch_ops(oracle):
    """torch.round / clamp on CPU as the library oracle for the v2 formula (ties included)."""
    import torch
    g = torch.Generator().manual_seed(5)
    x = torch.randn(4, 1000, generator=g) * 3
    scale = torch.tensor([[0.05], [0.125], [0.031], [0.5]])
    offset = torch.tensor([[-128.], [-3.], [0.], [-7.]])
    x[1, :16] = (torch.arange(16) - 8 + 0.5) * 0.125      # exact ties: half-to-even decides
    for qmin, qmax in ((0, 255), (-8, 7), (-128, 127), (0, 15)):
        r = torch.round(x / scale) - offset
        m = (qmin <= r) & (r <= qmax)
        y = (r.clamp(qmin, qmax) + offset) * scale
        yo, qo, mo = oracle.v2_qdq(x.numpy(), 4, 1000, scale.reshape(-1).numpy(), offset.reshape(-1).numpy(), qmin,
                                   qmax)
        assert np.array_equal(yo, y.numpy())
        assert np.array_equal(mo.astype(bool), m.numpy())


def test_bf16_roundtrip_matches_torch(oracle):
    import torch
    g = torch.Generator().manual_seed(7)
    x = torch.randn(10000, generator=g) * 100
    x[:4] = torch.tensor([float("inf"), -float("inf"), 0.0, -0.0])
    bits = oracle.f32_to_bf16_bits(x.numpy())
    tb = x.to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(bits, tb)
    for v in x[:200].numpy():
        assert oracle.L.orc_f32_to_bf16(float(v)) == int(oracle.f32_to_bf16_bits(np.array([v]))[0])


# ------------------------------------------------------------------------------- percentile analyzer (v1, C++)
def test_percentile_cases_of_the_reference_unit_tests(oracle):
    """ModelOptimizations/DlQuantization/test/TestPercentileEncodingAnalyzer.cpp:56-370: the assertions of its cases
    on data of the same distribution (the reference draws from std::normal_distribution; the bounds it asserts hold
    for any sample of that size)."""
    rng = np.random.default_rng(1)
    x = (rng.standard_normal(100000) * 2 + 2).astype(np.float32)
    pdf = oracle.new_pdf()
    pdf.update(x)
    e = pdf.compute_percentile_encoding(8, 99.9999)                      # Asymmetric, :56-109
    assert 2 - 12 < e.min < 2 - 4 and 2 + 4 < e.max < 2 + 12
    e = pdf.compute_percentile_encoding(8, 99.9999, sym=True)            # Symmetric, :111-159
    assert e.min > -np.abs(x).max() - e.delta and e.max < np.abs(x).max() and e.offset == -128 and e.bw == 8
    assert e.delta == pytest.approx((e.max - e.min) / 255, rel=1e-6)
    e = pdf.compute_percentile_encoding(8, 99.9999, sym=True, strict=True)   # StrictSymmetric, :161-210
    assert e.offset == -127 and e.min == -e.max and e.delta == pytest.approx((e.max - e.min) / 254, rel=1e-6)
    pos = np.abs(x)
    pdf = oracle.new_pdf()
    pdf.update(pos)
    e = pdf.compute_percentile_encoding(8, 99.9999, sym=True, unsigned_sym=True)   # SymmetricUnsigned, :212-260
    assert e.min == 0 and e.max == pytest.approx(pos.max(), abs=0.05) and e.offset == 0
    pdf = oracle.new_pdf()                                                # AllSameValuesAsymmetric, :311-346
    pdf.update(np.full(6000, 4, np.float32))
    e = pdf.compute_percentile_encoding(8, 99.9999)
    assert e.min <= 0 and e.max >= 3.99006
    pdf = oracle.new_pdf()
    pdf.update(np.full(6000, -5, np.float32))
    e = pdf.compute_percentile_encoding(8, 99.9999)
    assert e.min <= -4.99992 and e.max >= 0
    pdf = oracle.new_pdf()                                                # AllZeroesAsymmetric, :348-370
    pdf.update(np.zeros(6000, np.float32))
    e = pdf.compute_percentile_encoding(8, 99.9999)
    assert e.min == pytest.approx(-1.00392, abs=1e-4) and e.max == pytest.approx(0.996078, abs=1e-4)
    assert e.offset == -128 and e.bw == 8


def test_mse_cases_of_the_reference_unit_tests(oracle):
    """ModelOptimizations/DlQuantization/test/TestMseEncodingAnalyzer.cpp:56-317: the assertions of its cases on data
    of the same distributions (the reference draws from std::normal_distribution; the bounds it asserts hold for any
    sample of that size)."""
    rng = np.random.default_rng(1)
    x = (rng.standard_normal(100000) * 2 + 2).astype(np.float32)
    pdf = oracle.new_pdf()
    pdf.update(x)
    e = pdf.compute_mse_encoding(8)                                       # Asymmetric, :56-114
    assert 2 - 12 < e.min < 2 - 4 and 2 + 4 < e.max < 2 + 12
    # the reference also asserts min and max strictly inside the sample's extremes, which holds for its own draw; on
    # any draw they lie within one bucket of them
    bucket = pdf.x_left()[1] - pdf.x_left()[0]
    assert e.min > x.min() - bucket and e.max < x.max() + bucket
    x = (rng.standard_normal(6000) * 2 + 2).astype(np.float32)
    pdf = oracle.new_pdf()
    pdf.update(x)
    e = pdf.compute_mse_encoding(8, sym=True)                             # Symmetric, :116-163
    assert e.min > -np.abs(x).max() and e.max < np.abs(x).max() and e.offset == -128 and e.bw == 8
    assert e.delta == pytest.approx((e.max - e.min) / 255, rel=1e-6)
    assert e.offset == pytest.approx(e.min / e.delta, rel=1e-6)
    x = (rng.standard_normal(6000) - 2).astype(np.float32)
    pdf = oracle.new_pdf()
    pdf.update(x)
    e = pdf.compute_mse_encoding(8, sym=True, strict=True)                # StrictSymmetric, :165-211
    assert e.min > -np.abs(x).max() and e.max < np.abs(x).max()
    assert e.offset == -127 and e.min == -e.max and e.delta == pytest.approx((e.max - e.min) / 254, rel=1e-6)
    pos = np.maximum(x, 0)
    pdf = oracle.new_pdf()
    pdf.update(pos)
    e = pdf.compute_mse_encoding(8, sym=True, unsigned_sym=True)          # SymmetricUnsigned, :213-260
    assert e.min == 0 and e.max < np.abs(x).max() and e.bw == 8
    assert e.delta == pytest.approx((e.max - e.min) / 255, rel=1e-6) and e.offset == 0
    pdf = oracle.new_pdf()                                                # AllSameValuesAsymmetric, :262-295
    pdf.update(np.full(100, 4, np.float32))
    e = pdf.compute_mse_encoding(8)
    assert e.min <= 0 and e.max >= 3.9
    pdf = oracle.new_pdf()
    pdf.update(np.full(100, -5, np.float32))
    e = pdf.compute_mse_encoding(8)
    assert e.min <= -4.99992 and e.max >= 0
    pdf = oracle.new_pdf()                                                # AllZeroesAsymmetric, :297-317
    pdf.update(np.zeros(6000, np.float32))
    e = pdf.compute_mse_encoding(8)
    assert e.min == pytest.approx(-1.00392, abs=1e-4) and e.max == pytest.approx(0.996078, abs=1e-4)
    assert e.offset == -128 and e.bw == 8


def test_mse_search_against_brute_force(oracle):
    """The pair the search returns has the least cost among all pairs, by a cost written here from the definition
    (numpy, float64): quantize-dequantize of the bucket centres on the grid of (min, max), squared error weighted by
    the PDF.  A wrong clamp, a missed candidate or a dropped weight moves the winner."""
    rng = np.random.default_rng(3)
    x = np.concatenate([rng.standard_normal(50000), 8 * rng.standard_normal(200)]).astype(np.float32)
    pdf = oracle.new_pdf()
    pdf.update(x)
    best_min, best_max, mins, maxs, centers = pdf.mse_minimize(4)
    x_left, p = pdf.x_left(), pdf.pdf()
    index = np.clip(np.floor((centers.astype(np.float64) - x_left[0]) / (x_left[1] - x_left[0])), 0, 511).astype(int)
    weight = p[index]
    c = centers.astype(np.float64)

    def cost(lo, hi):
        delta = (hi - lo) / 15
        offset = np.round(lo / delta)
        if lo < 0 < hi:
            offset = -min(15.0, max(0.0, np.round(-lo / delta)))
        q = np.floor(np.clip(c, lo, hi) / delta - offset + 0.5)
        return float(np.sum(weight * (c - delta * (q + offset)) ** 2))
    costs = np.array([[cost(float(lo), float(hi)) if (lo, hi) != (0, 0) else np.inf for hi in maxs] for lo in mins])
    i, j = np.unravel_index(np.argmin(costs), costs.shape)
    assert costs[i, j] == pytest.approx(cost(float(best_min), float(best_max)), rel=1e-4)
    assert best_min < 0 < best_max and best_max < x.max() and best_min > x.min()      # outliers are clipped
    assert len(mins) + len(maxs) >= 100 and mins[-1] == 0 and maxs[-1] == 0


def test_entropy_cases_of_the_reference_unit_tests(oracle):
    """ModelOptimizations/DlQuantization/test/TestEntropyEncodingAnalyzer.cpp:56-314: the assertions of its cases on
    data of the same distributions."""
    rng = np.random.default_rng(1)
    x = (rng.standard_normal(100000) * 2 + 2).astype(np.float32)
    top = np.abs(x).max()
    prof = oracle.new_profile()
    prof.update(x)
    e = prof.compute_encoding(8)                                          # Asymmetric, :56-109
    assert 2 - 12 < e.min < 2 - 4 and 2 + 4 < e.max < 2 + 12
    e = prof.compute_encoding(8, sym=True)                                # Symmetric, :111-158
    assert e.min > -top and e.max < top and e.offset == -128 and e.bw == 8
    assert e.delta == pytest.approx((e.max - e.min) / 255, rel=1e-6)
    assert e.offset == pytest.approx(e.min / e.delta, rel=1e-6)
    e = prof.compute_encoding(8, sym=True, strict=True)                   # StrictSymmetric, :160-208
    assert e.min > -top and e.max < top and e.offset == -127 and e.min == -e.max
    assert e.delta == pytest.approx((e.max - e.min) / 254, rel=1e-6)
    pos = np.maximum(x, 0)
    prof = oracle.new_profile()
    prof.update(pos)
    e = prof.compute_encoding(8, sym=True, unsigned_sym=True)             # SymmetricUnsigned, :210-257
    assert e.min == 0 and e.max <= top and e.offset == 0 and e.bw == 8
    assert e.delta == pytest.approx((e.max - e.min) / 255, rel=1e-6)
    prof = oracle.new_profile()                                           # AllSameValuesAsymmetric, :259-292
    prof.update(np.full(100, 4, np.float32))
    e = prof.compute_encoding(8)
    assert e.min <= 0 and e.max >= 3.9
    prof = oracle.new_profile()
    prof.update(np.full(100, -5, np.float32))
    e = prof.compute_encoding(8)
    assert e.min <= -4.99992 and e.max >= 0
    prof = oracle.new_profile()                                           # AllZeroesAsymmetric, :294-314
    prof.update(np.zeros(6000, np.float32))
    e = prof.compute_encoding(8)
    assert e.min == pytest.approx(-1.00392, abs=1e-4) and e.max == pytest.approx(0.996078, abs=1e-4)
    assert e.offset == -128 and e.bw == 8


def test_entropy_histogram_invariants(oracle):
    """What the arithmetic fixes about the rescaling histogram: it spans exactly the range seen, every sample is
    counted once (redistribution moves whole counts: the total is the number of samples, exactly), a batch inside
    the range leaves the range alone, and the bins agree with numpy's histogram away from bin edges."""
    rng = np.random.default_rng(4)
    prof = oracle.new_profile()
    total, lo, hi = 0, np.inf, -np.inf
    for scale, shift in ((1.0, 0.0), (0.2, 0.1), (3.0, -1.0), (1.0, 9.0)):
        x = (rng.standard_normal(20000) * scale + shift).astype(np.float32)
        prof.update(x)
        total += x.size
        lo, hi = min(lo, float(x.min())), max(hi, float(x.max()))
        assert prof.range() == (lo, hi)
        hist = prof.histogram()
        assert hist.sum() == total and np.all(hist == np.round(hist)) and hist.min() >= 0
    prof = oracle.new_profile()
    x = rng.standard_normal(100000).astype(np.float32)
    prof.update(x)
    want, _ = np.histogram(x.astype(np.float64), bins=512, range=(float(x.min()), float(x.max())))
    # float32 bin arithmetic against float64: a sample within rounding of an edge may land next door
    assert np.abs(prof.histogram() - want).sum() <= 20 and prof.histogram().sum() == want.sum()


def test_entropy_search_against_a_direct_kl(oracle):
    """The divergence of the first window (the whole histogram, nothing saturated) against the KL divergence written
    here from its definition in numpy: P = the histogram, Q = 255 merged levels spread back over their non-empty
    bins, both smoothed by moving 1e-4 per empty bin from the non-empty ones, KL(P || Q) of the normalised two."""
    rng = np.random.default_rng(8)
    x = np.concatenate([rng.standard_normal(200000), [14.0, -11.0]]).astype(np.float32)
    prof = oracle.new_profile()
    prof.update(x)
    lo, hi, divergences = prof.optimize_kl(8)
    hist = prof.histogram()
    edges = np.ceil(np.arange(256) * (512 / 255)).astype(int)
    edges[-1] = 512
    q = np.zeros(512)
    for a, b in zip(edges[:-1], edges[1:]):
        nz = hist[a:b] != 0
        if nz.any():
            q[a:b][nz] = hist[a:b].sum() / nz.sum()

    def smooth(h):
        zeros = h == 0
        eps = 1e-4 * zeros.sum() / (~zeros).sum()
        return np.where(zeros, 1e-4, h - eps)
    p, q = smooth(hist.copy()), smooth(q)
    p, q = p / p.sum(), q / q.sum()
    assert divergences[0] == pytest.approx(float(np.sum(p * np.log(p / q))), rel=1e-5)
    assert len(divergences) == 129                                        # 512, 510, ... 256 bins
    # the winner is the window of least divergence, and it cuts the two far outliers off
    assert -11 < lo < 0 < hi < 14
    best = int(np.argmin(divergences))
    width = (float(x.max()) - float(x.min())) / 512
    assert hi - lo == pytest.approx((512 - 2 * best) * width, rel=1e-5)
