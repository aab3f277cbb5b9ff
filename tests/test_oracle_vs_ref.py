"""A/B of the C restatement (oracle/miq_oracle.c) against the reference's own DlQuantization CPU classes compiled in
place (oracle/_ref, built by `make -C oracle ref`).  Skipped where that library is absent (e.g. on the GPU box)."""
import numpy as np
import pytest


def _bits(a):
    return np.asarray(a, np.float32).view(np.uint32)


def _inputs(rng, n, scale=1.0):
    x = (rng.standard_normal(n) * scale).astype(np.float32)
    x[:8] = [np.nan, np.inf, -np.inf, 0.0, -0.0, 1e-42, -1e-42, 3.4e38]
    return x


@pytest.mark.parametrize("bw", [4, 8, 16])
@pytest.mark.parametrize("mnmx", [(-0.46, 0.72), (0.5, 1.0), (0.5, 0.5), (-0.5, -0.1), (-3.0, 3.0), (-1e-7, 2e-7),
                                  (-2.3, 0.0), (0.0, 6.0)])
def test_per_tensor_qdq_and_codes(oracle, ref, bw, mnmx):
    rng = np.random.default_rng(bw * 100 + int(abs(mnmx[0]) * 10))
    x = _inputs(rng, 200000, 1.5)
    e = oracle.fill_encoding_info(bw, *mnmx)
    assert e.astuple() == ref.fill_encoding_info(bw, *mnmx)
    # exact rounding ties: x = delta * (k + 0.5 + offset)
    k = np.arange(0, min(2 ** bw - 1, 4000))
    x[100:100 + k.size] = (np.float32(e.delta) * (k + 0.5 + e.offset)).astype(np.float32)
    assert np.array_equal(_bits(oracle.qdq_per_tensor(x, *mnmx, bw)), _bits(ref.qdq_per_tensor(x, *mnmx, bw)))
    for shift in (False, True):
        assert np.array_equal(_bits(oracle.quantize_per_tensor(x, *mnmx, bw, shift)),
                              _bits(ref.quantize_per_tensor(x, *mnmx, bw, shift)))


def test_per_channel_kernel_loop(oracle, ref):
    rng = np.random.default_rng(11)
    c, npc = 37, 513
    for outer in (1, 3):
        x = _inputs(rng, outer * c * npc, 0.05)
        enc_min = -np.abs(rng.standard_normal(c)) * 0.1
        enc_max = np.abs(rng.standard_normal(c)) * 0.1
        for bw in (4, 8):
            params = oracle.per_channel_params(enc_min, enc_max, bw)
            a = oracle.qdq_per_channel(x, c, npc, params)
            b = ref.qdq_per_channel(x, c, npc, params)
            assert np.array_equal(_bits(a), _bits(b))


def test_per_channel_params_match_torch_cpu_ops(oracle):
    """The torch extension derives per-channel delta/offset with float32 ATen ops; restate with torch CPU ops."""
    import torch
    rng = np.random.default_rng(12)
    for sym in (False, True):
        enc_max = np.abs(rng.standard_normal(4096)) * 0.3
        enc_min = -enc_max if sym else -np.abs(rng.standard_normal(4096)) * 0.3
        enc_min[5], enc_max[5] = 0.2, 0.7          # gated to 0
        enc_min[6], enc_max[6] = 0.0, 0.0          # degenerate range
        for bw in (4, 8):
            mn = torch.tensor(enc_min, dtype=torch.float64).to(torch.float32)
            mx = torch.tensor(enc_max, dtype=torch.float64).to(torch.float32)
            steps = 2.0 ** bw - 1
            if enc_min[0] == -enc_max[0]:
                steps -= 1
            zero = torch.zeros(1)
            mn = torch.minimum(mn, zero)
            mx = torch.maximum(mx, zero)
            mx = torch.maximum(mx, mn + 1e-5)
            delta = (mx - mn) / steps
            offset = torch.round(mn / delta)
            got = oracle.per_channel_params(enc_min, enc_max, bw)
            for g, t in zip(got, (mn, mx, delta, offset)):
                assert np.array_equal(_bits(g), _bits(t.numpy()))


def test_broadcast_qdq(oracle, ref):
    rng = np.random.default_rng(13)
    shape = (3, 8, 5, 4)
    x = _inputs(rng, int(np.prod(shape)), 1.0)
    strides = [8 * 5 * 4, 5 * 4, 4, 1]
    for enc_shape in ((1, 8, 1, 1), (3, 1, 1, 4), (1, 1, 1, 1), (1, 8, 5, 1)):
        n_enc = int(np.prod(enc_shape))
        est, acc = [], 1
        for d in reversed(enc_shape):
            est.append(acc if d > 1 else 0)
            acc *= d
        est = est[::-1]
        enc_min = -np.abs(rng.standard_normal(n_enc))
        enc_max = np.abs(rng.standard_normal(n_enc))
        params = oracle.per_channel_params(enc_min, enc_max, 8)
        a = oracle.qdq_broadcast(x, strides, est, params)
        b = ref.qdq_broadcast(x, strides, est, params)
        assert np.array_equal(_bits(a), _bits(b))


def test_get_computed_encodings(oracle, ref):
    rng = np.random.default_rng(14)
    cases = [(-1.0, 1.0), (0.0, 5.0), (-5.0, 0.0), (-np.inf, np.inf), (0.0, 0.01), (-3e38, 3e38), (1e-9, 2e-9)]
    cases += [tuple(sorted(rng.normal(0, 10, 2))) for _ in range(200)]
    for mn, mx in cases:
        for bw in (4, 8, 16):
            for sym, strict, uns in ((0, 0, 0), (1, 0, 0), (1, 1, 0), (1, 0, 1)):
                a = oracle.get_computed_encodings(bw, mn, mx, sym, strict, uns).astuple()
                b = ref.get_computed_encodings(bw, mn, mx, sym, strict, uns)
                assert a == b, (mn, mx, bw, sym, strict, uns)


def test_tf_analyzer(oracle, ref):
    rng = np.random.default_rng(15)
    tf = ref.new_tf()
    acc_min, acc_max = np.finfo(np.float64).max, -np.finfo(np.float64).max
    for _ in range(3):
        x = _inputs(rng, 50000, 2.0)
        x[1:3] = 0            # keep +-inf out so the accumulated range stays finite and data dependent
        x[7] = 0
        tf.update(x)
        mn, mx = oracle.minmax(x)
        acc_min, acc_max = min(acc_min, float(mn)), max(acc_max, float(mx))
    for bw in (4, 8):
        for sym, strict, uns in ((0, 0, 0), (1, 0, 0), (1, 1, 0), (1, 0, 1)):
            a = oracle.tf_compute_encoding(acc_min, acc_max, bw, sym, strict, uns).astuple()
            assert a == tf.compute_encoding(bw, sym, strict, uns)


def _relu_pareto(rng, n):
    x = np.abs(rng.standard_normal(n)).astype(np.float32)
    tail = rng.random(n) < 0.005
    x[tail] = (1.0 / np.sqrt(1.0 - rng.random(int(tail.sum())))).astype(np.float32)
    return x


@pytest.mark.parametrize("kind", ["n22", "relu_pareto", "gauss_outliers", "tiny", "zeros_then_data", "scale_1e-30",
                                  "scale_1e-22", "scale_1e-12", "scale_1e12", "scale_1e22", "scale_1e30"])
def test_tf_enhanced_pdf_candidates_costs(oracle, ref, n22, kind):
    rng = np.random.default_rng(16)
    if kind == "n22":
        batches = [n22]
    elif kind.startswith("scale_"):
        # extreme magnitudes: at the small end a candidate range is more than 2^31 PDF buckets wide and the reference's
        # (int) cast leaves the int range (its x86-64 build yields INT_MIN there, which the restatement spells out)
        scale = float(kind[6:])
        batches = [(rng.standard_normal(30000) * scale).astype(np.float32) for _ in range(2)]
        batches[1][::97] *= np.float32(1e6)
        batches[1][5:9] = [3e38, -3e38, np.inf, np.nan]
    elif kind == "relu_pareto":
        batches = [_relu_pareto(rng, 50000) for _ in range(4)]
    elif kind == "gauss_outliers":
        batches = [_inputs(rng, 30000, 3.0) for _ in range(3)]
        batches[0][1:3] = [40.0, -35.0]
        batches[0][7] = 0
    elif kind == "tiny":
        batches = [np.array([0.25], np.float32), np.array([0.25, 0.3, -0.1], np.float32)]
    else:
        batches = [np.zeros(100, np.float32), _relu_pareto(rng, 10000)]
    pdf, r = oracle.new_pdf(), ref.new_tfe()
    for b in batches:
        pdf.update(b)
        r.update(b)
    n, xl, p, it = r.pdf()
    assert n == 512 and it == pdf.iterations
    assert np.array_equal(xl, pdf.x_left())
    assert np.array_equal(p, pdf.pdf())
    assert pdf.find_range() == r.find_range()
    for bw in (4, 8):
        for sym, strict, uns in ((0, 0, 0), (1, 0, 0), (1, 1, 0), (1, 0, 1)):
            d, o = pdf.candidates(bw, sym, strict, uns)
            rd, ro, rc = r.candidates(bw, sym, strict, uns)
            assert np.array_equal(_bits(d), _bits(rd)) and np.array_equal(o, ro)
            enc, costs, best = pdf.compute_encoding(bw, sym, strict, uns)
            # costs: identical accumulation order and operations => bit-identical doubles
            assert np.array_equal(costs[:len(rc)].view(np.uint64), rc.view(np.uint64))
            assert enc.astuple() == r.compute_encoding(bw, sym, strict, uns)


def test_tf_enhanced_empty_states(oracle, ref):
    r = ref.new_tfe()
    assert oracle.new_pdf().compute_encoding(8)[0].astuple() == r.compute_encoding(8)
    pdf = oracle.new_pdf()
    z = np.zeros(64, np.float32)
    pdf.update(z)
    r.update(z)
    for bw in (4, 8, 16):
        assert pdf.compute_encoding(bw)[0].astuple() == r.compute_encoding(bw)


@pytest.mark.parametrize("percentile", [100.0, 99.9999, 99.9, 99.0, 90.0, 50.0])
def test_percentile_analyzer(oracle, ref, percentile):
    """PercentileEncodingAnalyzer<float>: same PDF accumulation as TF-Enhanced, different computeEncoding."""
    rng = np.random.default_rng(int(percentile * 100))
    for kind in ("normal", "relu", "negative", "outliers", "constant", "zeros-then-data"):
        pdf, an = oracle.new_pdf(), ref.new_percentile(percentile)
        batches = []
        for b in range(3):
            x = (rng.standard_normal(20000) * (1 + b) + 0.5).astype(np.float32)
            if kind == "relu":
                x = np.maximum(x, 0)
            elif kind == "negative":
                x = -np.abs(x) - 0.25
            elif kind == "outliers":
                x[:5] = 300.0
            elif kind == "constant":
                x[:] = 4.0
            elif kind == "zeros-then-data" and b == 0:
                x[:] = 0.0
            batches.append(x)
        for x in batches:
            pdf.update(x)
            an.update(x)
        for bw in (4, 8, 16):
            for sym, strict, uns in ((False, False, False), (True, False, False), (True, True, False),
                                     (True, False, True)):
                got = pdf.compute_percentile_encoding(bw, percentile, sym, strict, uns)
                want = an.compute_encoding(bw, sym, strict, uns)
                assert got.astuple() == want, (kind, bw, sym, strict, uns)


def test_percentile_analyzer_without_usable_statistics(oracle, ref):
    pdf, an = oracle.new_pdf(), ref.new_percentile(99.0)
    assert pdf.compute_percentile_encoding(8, 99.0).astuple() == an.compute_encoding(8)     # nothing seen: zeros
    z = np.zeros(100, np.float32)
    pdf.update(z)
    an.update(z)
    for bw, sym, strict in ((8, False, False), (8, True, True), (4, False, False)):
        assert pdf.compute_percentile_encoding(bw, 99.0, sym, strict).astuple() == an.compute_encoding(bw, sym, strict)


def _mse_batches(rng, kind):
    batches = []
    for b in range(3):
        x = (rng.standard_normal(20000) * (1 + b) + 0.5).astype(np.float32)
        if kind == "relu":
            x = np.maximum(x, 0)
        elif kind == "negative":
            x = -np.abs(x) - 0.25
        elif kind == "outliers":
            x[:5] = 300.0
        elif kind == "constant":
            x[:] = 4.0
        elif kind == "zeros-then-data" and b == 0:
            x[:] = 0.0
        elif kind == "far-from-zero":
            x = x * 0.01 + 50.0
        batches.append(x)
    return batches


@pytest.mark.parametrize("kind", ["normal", "relu", "negative", "outliers", "constant", "zeros-then-data",
                                  "far-from-zero"])
def test_mse_analyzer(oracle, ref, kind):
    """MseEncodingAnalyzer<float>: the PDF of TF-Enhanced, every pair of bucket edges either side of zero as a
    candidate range, squared error of the bucket centres as cost.  The winning pair and every field of the encoding."""
    rng = np.random.default_rng(len(kind))
    pdf, an = oracle.new_pdf(), ref.new_mse()
    for x in _mse_batches(rng, kind):
        pdf.update(x)
        an.update(x)
    for bw in (4, 8, 16):
        for sym, strict, uns in ((False, False, False), (True, False, False), (True, True, False), (True, False, True)):
            best = pdf.mse_minimize(bw, sym, strict, uns)
            assert (best[0], best[1]) == an.minimize(bw, sym, strict, uns), (kind, bw, sym, strict, uns)
            got = pdf.compute_mse_encoding(bw, sym, strict, uns)
            assert got.astuple() == an.compute_encoding(bw, sym, strict, uns), (kind, bw, sym, strict, uns)


def test_mse_cost_of_single_candidates(oracle, ref):
    """The cost function alone, on centres and weights that are not a PDF's: ranges that clip, that do not, one-sided
    ranges, all four symmetry modes."""
    rng = np.random.default_rng(5)
    an = ref.new_mse()
    centers = np.sort(rng.standard_normal(300).astype(np.float32) * 3)
    weights = rng.random(300).astype(np.float32)
    weights /= weights.sum()
    for bw in (2, 4, 8, 16, 24):
        for lo, hi in ((-1.0, 1.0), (-9.5, 0.25), (0.0, 2.0), (-3.0, 0.0), (-20.0, 20.0), (-1e-3, 1e-3)):
            for sym, strict, uns in ((False, False, False), (True, False, False), (True, True, False),
                                     (True, False, True)):
                got = np.float32(oracle.L.orc_mse_cost(bw, centers, weights, centers.size, lo, hi, int(sym),
                                                       int(strict), int(uns)))
                want = an.cost(bw, centers, weights, lo, hi, sym, strict, uns)
                assert got.tobytes() == want.tobytes(), (bw, lo, hi, sym, strict, uns)


def test_mse_analyzer_without_usable_statistics(oracle, ref):
    pdf, an = oracle.new_pdf(), ref.new_mse()
    assert pdf.compute_mse_encoding(8).astuple() == an.compute_encoding(8)                   # nothing seen: zeros
    z = np.zeros(100, np.float32)
    pdf.update(z)
    an.update(z)
    for bw, sym, strict in ((8, False, False), (8, True, True), (4, False, False)):
        assert pdf.compute_mse_encoding(bw, sym, strict).astuple() == an.compute_encoding(bw, sym, strict)


_ENTROPY_KINDS = ["normal", "relu", "negative", "outliers", "constant", "zeros-then-data", "far-from-zero",
                  "growing-range", "one-batch"]


def _entropy_batches(rng, kind):
    if kind == "growing-range":
        # every batch widens the range, to the left, to the right, on both sides: the histogram is redistributed
        return [(rng.standard_normal(5000) * s + m).astype(np.float32)
                for s, m in ((0.5, 0.0), (1.0, 2.0), (1.0, -3.0), (4.0, 0.0), (0.1, 0.0))]
    if kind == "one-batch":
        return [rng.standard_normal(50000).astype(np.float32)]
    return _mse_batches(rng, kind)


@pytest.mark.parametrize("kind", _ENTROPY_KINDS)
def test_entropy_analyzer(oracle, ref, kind):
    """EntropyEncodingAnalyzer<float>: the histogram after every batch (range, every bin, batch count), the range the
    KL window search returns, every field of the encoding."""
    rng = np.random.default_rng(len(kind) + 100)
    prof, an = oracle.new_profile(), ref.new_entropy()
    for x in _entropy_batches(rng, kind):
        prof.update(x)
        an.update(x)
        n, hist, rng_ref, it = an.histogram()
        assert prof.initialized == (n == 512) and prof.iterations == it
        if n:
            assert prof.range() == rng_ref
            assert np.array_equal(prof.histogram(), hist)
    for bw in (8, 4, 16):
        for sym, strict, uns in ((False, False, False), (True, False, False), (True, True, False), (True, False, True)):
            lo, hi, _ = prof.optimize_kl(bw, sym, strict, uns)
            assert (lo, hi) == an.optimize(bw, sym, strict, uns), (kind, bw, sym, strict, uns)
            got = prof.compute_encoding(bw, sym, strict, uns)
            assert got.astuple() == an.compute_encoding(bw, sym, strict, uns), (kind, bw, sym, strict, uns)


def test_entropy_analyzer_without_usable_statistics(oracle, ref):
    prof, an = oracle.new_profile(), ref.new_entropy()
    assert prof.compute_encoding(8).astuple() == an.compute_encoding(8)                      # nothing seen: zeros
    z = np.zeros(100, np.float32)
    prof.update(z)
    an.update(z)
    assert prof.iterations == an.histogram()[3] == 0                                          # the batch is not counted
    for bw, sym, strict in ((8, False, False), (8, True, True), (4, False, False)):
        assert prof.compute_encoding(bw, sym, strict).astuple() == an.compute_encoding(bw, sym, strict)
