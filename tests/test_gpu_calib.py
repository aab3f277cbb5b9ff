"""GPU parity of the calibration kernels (min/max, 512-bucket PDF, TF-Enhanced search) against the CPU oracle,
through the C ABI.  Bin counts, PDF, candidate lists, costs and the chosen encoding must be identical."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

TF, TFE = 0, 1


@pytest.fixture(scope="module")
def ops():
    from aimet_amd import ops as o
    return o


def _gpu(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def _relu_pareto(seed, n):
    """|N(0,1)| with a 0.5 % Pareto(alpha=2, x_m=1) tail: the post-ReLU activation model of the calibration config."""
    rng = np.random.default_rng(seed)
    x = np.abs(rng.standard_normal(n)).astype(np.float32)
    tail = rng.random(n) < 0.005
    x[tail] = (1.0 / np.sqrt(1.0 - rng.random(int(tail.sum())))).astype(np.float32)
    return x


def _check_tfe(ops, oracle, batches, modes=((8, 0, 0, 0), (8, 1, 0, 0), (8, 1, 1, 0), (8, 1, 0, 1), (4, 0, 0, 0))):
    an = ops.Analyzer(TFE)
    pdf = oracle.new_pdf()
    for b in batches:
        an.update_stats(_gpu(b))
        hist = pdf.update(b)
        if pdf.initialized:
            assert np.array_equal(an.last_batch_counts(), hist)
    xl, p = an.get_stats_histogram()
    if pdf.initialized:
        assert np.array_equal(xl, pdf.x_left())
        assert np.array_equal(p, pdf.pdf())
    else:
        assert xl.size == 0
    for bw, sym, strict, uns in modes:
        enc, valid = an.compute_encoding(bw, sym, strict, uns)
        oenc, ocosts, obest = pdf.compute_encoding(bw, sym, strict, uns)
        assert valid
        assert (enc.min, enc.max, enc.delta, enc.offset, enc.bw) == oenc.astuple(), (bw, sym, strict, uns)
        if pdf.initialized:
            d, o, c, best = an.last_search()
            od, oo = pdf.candidates(bw, sym, strict, uns)
            assert np.array_equal(d.view(np.uint32), od.view(np.uint32)) and np.array_equal(o, oo)
            assert np.array_equal(c.view(np.uint64), ocosts[:len(od)].view(np.uint64))   # costs bit-identical
            assert best == obest
    return an


def test_minmax(ops, oracle):
    for n in (1, 5, 1023, 100003, 1 << 22):
        rng = np.random.default_rng(n)
        x = (rng.standard_normal(n) * 3).astype(np.float32)
        if n > 10:
            x[3] = np.nan
        got = ops.minmax(_gpu(x)).cpu().numpy()
        mn, mx = oracle.minmax(x)
        assert got[0] == mn and got[1] == mx
    x = np.full(7, np.nan, np.float32)
    got = ops.minmax(_gpu(x)).cpu().numpy()
    assert got[0] == np.inf and got[1] == -np.inf


def test_minmax_per_channel(ops):
    g = torch.Generator().manual_seed(3)
    for shape, axis in (((64, 300), 0), ((3, 16, 50), 1), ((11008, 4096), 0), ((5, 7, 3, 3), 1)):
        x = torch.randn(shape, generator=g)
        c = shape[axis]
        npc = int(np.prod(shape[axis + 1:]))
        got = ops.minmax_per_channel(x.cuda(), c, npc).cpu()
        dims = [d for d in range(len(shape)) if d != axis]
        assert torch.equal(got[0], x.amin(dim=dims)) and torch.equal(got[1], x.amax(dim=dims))


def test_tf_analyzer(ops, oracle):
    an = ops.Analyzer(TF)
    e, valid = an.compute_encoding(8)
    assert not valid
    rng = np.random.default_rng(4)
    acc_min, acc_max = np.inf, -np.inf
    for i in range(3):
        x = (rng.standard_normal(50001) * (i + 1)).astype(np.float32)
        an.update_stats(_gpu(x))
        acc_min, acc_max = min(acc_min, float(x.min())), max(acc_max, float(x.max()))
    for bw in (4, 8):
        for sym, strict, uns in ((0, 0, 0), (1, 0, 0), (1, 1, 0), (1, 0, 1)):
            e, valid = an.compute_encoding(bw, sym, strict, uns)
            o = oracle.tf_compute_encoding(acc_min, acc_max, bw, sym, strict, uns)
            assert valid and (e.min, e.max, e.delta, e.offset, e.bw) == o.astuple()
    an.reset()
    assert not an.compute_encoding(8)[1]


def test_tfe_known_answer_n22(ops, oracle, vectors, n22):
    v = vectors["tf_enhanced_n22"]
    an = _check_tfe(ops, oracle, [n22])
    enc, _ = an.compute_encoding(8)
    assert enc.min == pytest.approx(v["exp_min"], abs=v["atol"]) and enc.max == pytest.approx(v["exp_max"], abs=v["atol"])
    y = ops.qdq_per_tensor(torch.full((16,), 5.0, device="cuda"), enc.min, enc.max, 8)
    assert float(y[0]) == pytest.approx(v["qdq_of_5"], abs=1e-3)


def test_tfe_multi_batch_relu_pareto(ops, oracle):
    _check_tfe(ops, oracle, [_relu_pareto(1003 + b, 200000 + 3 * b) for b in range(5)])


def test_tfe_outliers_nan_dropped(ops, oracle):
    rng = np.random.default_rng(6)
    b0 = (rng.standard_normal(100000)).astype(np.float32)
    b1 = b0.copy()
    b1[:10] = 1e6
    b1[10:15] = np.nan
    b1[15:20] = -np.inf
    an = _check_tfe(ops, oracle, [b0, b1], modes=((8, 0, 0, 0),))
    assert an.last_batch_counts().sum() == b1.size - 20


def test_tfe_all_zero_batches_then_data(ops, oracle, vectors):
    v = vectors["tf_enhanced_all_zeros"]
    an = ops.Analyzer(TFE)
    e, valid = an.compute_encoding(8)
    assert not valid                                   # nothing seen yet
    an.update_stats(torch.zeros(1000, device="cuda"))
    e, valid = an.compute_encoding(8)
    assert valid and e.offset == v["offset"]
    assert e.min == pytest.approx(v["exp_min"], abs=v["atol"]) and e.max == pytest.approx(v["exp_max"], abs=v["atol"])
    assert an.get_stats_histogram()[0].size == 0
    _check_tfe(ops, oracle, [np.zeros(64, np.float32), _relu_pareto(7, 30000), np.zeros(64, np.float32)])


def test_tfe_constant_and_tiny(ops, oracle):
    _check_tfe(ops, oracle, [np.full(100, 4.0, np.float32)], modes=((8, 0, 0, 0),))
    _check_tfe(ops, oracle, [np.full(100, -5.0, np.float32)], modes=((8, 0, 0, 0),))
    _check_tfe(ops, oracle, [np.array([0.25], np.float32), np.array([0.25, 0.3, -0.1], np.float32)])


@pytest.mark.parametrize("scale", [1e-30, 1e-22, 1e-12, 1.0, 1e12, 1e22, 1e30])
def test_tfe_bucket_index_at_extreme_scales(ops, oracle, scale):
    """The bucket index is round(x / bucket - offset) with an IEEE division.  The kernel divides through a reciprocal
    plus residual corrections where that is exact (bucket width in [2^-64, 2^64], |x| <= 2^60) and with a true
    division elsewhere; both sides of each limit, and a second batch with values far outside the first one's range."""
    rng = np.random.default_rng(77)
    b0 = (rng.standard_normal(150001) * scale).astype(np.float32)
    b1 = (rng.standard_normal(150001) * scale).astype(np.float32)
    b1[::97] *= np.float32(1e6)                       # outside the PDF range: dropped
    b1[5:9] = [3e38, -3e38, np.inf, np.nan]
    _check_tfe(ops, oracle, [b0, b1], modes=((8, 0, 0, 0), (8, 1, 0, 0)))


def test_tfe_reset_and_unaligned(ops, oracle):
    an = ops.Analyzer(TFE)
    x = _relu_pareto(8, 50001)
    an.update_stats(_gpu(x))
    an.reset()
    y = (np.random.default_rng(9).standard_normal(40003)).astype(np.float32)
    base = _gpu(np.concatenate([np.zeros(1, np.float32), y]))
    an.update_stats(base[1:])                          # 4-byte aligned only
    pdf = oracle.new_pdf()
    hist = pdf.update(y)
    assert np.array_equal(an.last_batch_counts(), hist)
    enc, _ = an.compute_encoding(8)
    assert (enc.min, enc.max, enc.delta, enc.offset, enc.bw) == pdf.compute_encoding(8)[0].astuple()


def _cfg3_batch(b, n):
    g = torch.Generator(device="cuda")
    g.manual_seed(1003 + b)
    x = torch.randn(n, device="cuda", generator=g).abs_()
    u = torch.rand(n, device="cuda", generator=g)
    t = torch.rand(n, device="cuda", generator=g)
    return torch.where(u < 0.005, (1 - t).rsqrt(), x)


def _same_search(an, pdf, modes=((8, 0, 0, 0), (8, 1, 0, 0), (4, 0, 0, 0))):
    for bw, sym, strict, uns in modes:
        enc, valid = an.compute_encoding(bw, sym, strict, uns)
        oenc, ocosts, obest = pdf.compute_encoding(bw, sym, strict, uns)
        assert valid and (enc.min, enc.max, enc.delta, enc.offset, enc.bw) == oenc.astuple(), (bw, sym, strict, uns)
        d, o, c, best = an.last_search()
        od, oo = pdf.candidates(bw, sym, strict, uns)
        assert np.array_equal(d.view(np.uint32), od.view(np.uint32)) and np.array_equal(o, oo)
        assert np.array_equal(c.view(np.uint64), ocosts[:len(od)].view(np.uint64))
        assert best == obest


def test_cfg3_full_size_bit_exact(ops, oracle):
    """The calibration configuration at its size: 16 batches of [32,256,28,28].  One analyzer is fed back to back with
    nothing read in between (the path a calibration loop takes: counts folded by the following launch, bucket
    parameters learnt asynchronously), a second one is read after every batch.  Per-batch counts, the final PDF
    (as bits), every candidate cost and the chosen encodings equal the oracle's."""
    n = 32 * 256 * 28 * 28
    stream_an, step_an = ops.Analyzer(TFE), ops.Analyzer(TFE)
    pdf = oracle.new_pdf()
    for b in range(16):
        x = _cfg3_batch(b, n)
        stream_an.update_stats(x)
        step_an.update_stats(x)
        hist = pdf.update(x.cpu().numpy())
        got = step_an.last_batch_counts()
        assert np.array_equal(got, hist), b
        assert int(got.sum()) <= n
    for an in (stream_an, step_an):
        xl, p = an.get_stats_histogram()
        assert np.array_equal(xl.view(np.uint64), pdf.x_left().view(np.uint64))
        assert np.array_equal(p.view(np.uint64), pdf.pdf().view(np.uint64))
        assert np.array_equal(an.last_batch_counts(), hist)
        _same_search(an, pdf)


def test_tfe_updates_across_streams(ops, oracle):
    """Batches queued on alternating torch streams: the analyzer orders each stream after the previous one, so the
    result is that of the same batches queued on one stream."""
    batches = [_relu_pareto(70 + b, 400000 + 13 * b) for b in range(8)]
    dev = [_gpu(b) for b in batches]
    torch.cuda.synchronize()
    an = ops.Analyzer(TFE)
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    for k, b in enumerate(dev):
        with torch.cuda.stream(streams[k % 2]):
            an.update_stats(b)
    pdf = oracle.new_pdf()
    for b in batches:
        pdf.update(b)
    xl, p = an.get_stats_histogram()          # on the default stream: ordered after both
    torch.cuda.synchronize()
    assert np.array_equal(xl.view(np.uint64), pdf.x_left().view(np.uint64))
    assert np.array_equal(p.view(np.uint64), pdf.pdf().view(np.uint64))
    _same_search(an, pdf, modes=((8, 0, 0, 0),))


@pytest.mark.parametrize("mode", [TF, TFE, 2])
def test_encodings_queued_ahead(ops, oracle, mode):
    """Several analyzers whose searches are queued before the first result is read: every answer is the one an
    analyzer gives that was asked directly.  A request is dropped by any call in between (another batch, other
    arguments) and the answer is then that of the new state."""
    def enc_tuple(e):
        return (e.min, e.max, e.delta, e.offset, e.bw)

    data = [[_gpu(_relu_pareto(900 + 10 * k + b, 120000 + 7 * k)) for b in range(3)] for k in range(6)]
    queued, direct = [ops.Analyzer(mode) for _ in data], [ops.Analyzer(mode) for _ in data]
    for group in (queued, direct):
        for an, batches in zip(group, data):
            if mode == 2:
                an.set_percentile(99.9)
            for b in batches:
                an.update_stats(b)
    for an in queued:
        an.queue_encoding(8, True, False, False)
    want = [enc_tuple(an.compute_encoding(8, True, False, False)[0]) for an in direct]
    got = [enc_tuple(an.compute_encoding(8, True, False, False)[0]) for an in queued]
    assert got == want
    # other arguments than the queued ones
    queued[0].queue_encoding(8, True, False, False)
    assert enc_tuple(queued[0].compute_encoding(4, False, False, False)[0]) == \
        enc_tuple(direct[0].compute_encoding(4, False, False, False)[0])
    # another batch after the request
    extra = _gpu(_relu_pareto(77, 50000) * 3)
    queued[1].queue_encoding(8, False, False, False)
    queued[1].update_stats(extra)
    direct[1].update_stats(extra)
    assert enc_tuple(queued[1].compute_encoding(8, False, False, False)[0]) == \
        enc_tuple(direct[1].compute_encoding(8, False, False, False)[0])
    # a histogram read between request and answer uses the same staging memory
    if mode != TF:
        queued[2].queue_encoding(8, False, False, False)
        queued[2].get_stats_histogram()
        assert enc_tuple(queued[2].compute_encoding(8, False, False, False)[0]) == \
            enc_tuple(direct[2].compute_encoding(8, False, False, False)[0])
    # nothing to queue without statistics
    fresh = ops.Analyzer(mode)
    fresh.queue_encoding(8, False, False, False)
    assert fresh.compute_encoding(8, False, False, False)[1] is False


def test_tfe_back_to_back_without_reads(ops, oracle):
    """update_stats calls queued with no read-back between them: a leading all-zero batch (no range yet), ragged batch
    sizes, a reset in the middle; only the final state is read and compared with the oracle fed the same batches."""
    rng = np.random.default_rng(31)
    first = [np.zeros(4096, np.float32)] + [_relu_pareto(40 + b, 300000 + 17 * b) for b in range(9)]
    second = [(rng.standard_normal(250001 + 5 * b) * (1 + 0.1 * b)).astype(np.float32) for b in range(12)]
    an = ops.Analyzer(TFE)
    dev = [[_gpu(b) for b in first], [_gpu(b) for b in second]]
    torch.cuda.synchronize()
    for b in dev[0]:
        an.update_stats(b)
    an.reset()
    for b in dev[1]:
        an.update_stats(b)
    pdf = oracle.new_pdf()
    for b in second:
        hist = pdf.update(b)
    xl, p = an.get_stats_histogram()
    assert np.array_equal(xl.view(np.uint64), pdf.x_left().view(np.uint64))
    assert np.array_equal(p.view(np.uint64), pdf.pdf().view(np.uint64))
    assert np.array_equal(an.last_batch_counts(), hist)
    _same_search(an, pdf)
    # the same without the reset, zero batch first
    an2, pdf2 = ops.Analyzer(TFE), oracle.new_pdf()
    for b in dev[0]:
        an2.update_stats(b)
    for b in first:
        pdf2.update(b)
    xl, p = an2.get_stats_histogram()
    assert np.array_equal(xl.view(np.uint64), pdf2.x_left().view(np.uint64))
    assert np.array_equal(p.view(np.uint64), pdf2.pdf().view(np.uint64))
    _same_search(an2, pdf2, modes=((8, 0, 0, 0),))


@pytest.mark.parametrize("outer,c,npc", [(1, 1, 100003), (1, 1, 3), (1, 1, 1 << 22), (1, 300, 4096), (1, 7, 70001),
                                         (6, 32, 784), (3, 5, 40000), (4, 1000, 9), (2, 3, 1 << 18)])
def test_minmax_with_and_without_workspace(ops, outer, c, npc):
    """Both reductions (stored partials folded by a second kernel; atomics on ordered keys) give the exact values."""
    import ctypes
    from aimet_amd._lib import check, lib
    torch.manual_seed(outer * 1000 + c + npc)
    x = torch.randn(outer, c, npc)
    x.view(-1)[::97] = float("nan")                                  # NaN is ignored
    x.view(-1)[5 % x.numel()] = -0.0
    xg = x.cuda()
    want_min = torch.nan_to_num(x, nan=float("inf")).amin(dim=(0, 2))
    want_max = torch.nan_to_num(x, nan=float("-inf")).amax(dim=(0, 2))
    got = ops.minmax_per_channel(xg, c, npc).cpu()
    assert torch.equal(got[0], want_min) and torch.equal(got[1], want_max)
    out = torch.empty(2, c, device="cuda")
    check(lib.miq_minmax_per_channel_f32(xg.data_ptr(), c, xg.numel(), npc, out.data_ptr(), None,
                                         ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)))
    assert torch.equal(out.cpu(), got)
    if c == 1:
        flat = ops.minmax(xg.reshape(-1)[1:])                        # misaligned base: scalar loads
        rest = x.reshape(-1)[1:]
        assert flat[0].item() == torch.nan_to_num(rest, nan=float("inf")).min().item()
        assert flat[1].item() == torch.nan_to_num(rest, nan=float("-inf")).max().item()


# ------------------------------------------------------------------------------------------ percentile analyzer
PERCENTILE = 2


@pytest.mark.parametrize("percentile", [100.0, 99.9999, 99.9, 99.0, 90.0, 50.0])
def test_percentile_analyzer_matches_the_oracle(ops, oracle, percentile):
    """PercentileEncodingAnalyzer<float>: the PDF is the TF-Enhanced one; every field of the encoding is identical."""
    rng = np.random.default_rng(int(percentile * 10))
    cases = {
        "normal": [(rng.standard_normal(30000) * (1 + b) + 0.5).astype(np.float32) for b in range(3)],
        "relu-pareto": [_relu_pareto(20 + b, 50000) for b in range(2)],
        "negative": [(-np.abs(rng.standard_normal(10000)) - 0.25).astype(np.float32)],
        "constant": [np.full(6000, 4, np.float32)],
        "zeros": [np.zeros(6000, np.float32)],
        "zeros-then-data": [np.zeros(100, np.float32), rng.standard_normal(9999).astype(np.float32)],
    }
    for kind, batches in cases.items():
        an, pdf = ops.Analyzer(PERCENTILE), oracle.new_pdf()
        an.set_percentile(percentile)
        for b in batches:
            an.update_stats(_gpu(b))
            pdf.update(b)
        for bw, sym, strict, uns in ((8, 0, 0, 0), (8, 1, 0, 0), (8, 1, 1, 0), (8, 1, 0, 1), (4, 0, 0, 0),
                                     (16, 0, 0, 0)):
            e, valid = an.compute_encoding(bw, sym, strict, uns)
            want = pdf.compute_percentile_encoding(bw, percentile, sym, strict, uns)
            assert valid and (e.min, e.max, e.delta, e.offset, e.bw) == want.astuple(), (kind, bw, sym, strict, uns)


def test_percentile_analyzer_edge_behaviour(ops):
    from aimet_amd._lib import MiqError
    an = ops.Analyzer(PERCENTILE)
    e, valid = an.compute_encoding(8)
    assert not valid and (e.min, e.max, e.delta, e.offset) == (0, 0, 0, 0)        # nothing seen
    with pytest.raises(MiqError):
        an.set_percentile(101.0)
    x = torch.randn(5000, device="cuda")
    an.update_stats(x)
    xl, p = an.get_stats_histogram()                                              # the PDF is inspectable
    assert len(xl) == 512 and abs(p.sum() - 1.0) < 1e-9
    e100, _ = an.compute_encoding(8)
    an.set_percentile(95.0)
    e95, _ = an.compute_encoding(8)
    assert e95.max < e100.max and e95.min > e100.min
    an.reset()
    assert not an.compute_encoding(8)[1]


# ------------------------------------------------------------------------------------------------ MSE analyzer
MSE = 3


@pytest.mark.parametrize("kind", ["normal", "relu-pareto", "negative", "constant", "zeros", "zeros-then-data",
                                  "far-from-zero", "outliers"])
def test_mse_analyzer_matches_the_oracle(ops, oracle, kind):
    """MseEncodingAnalyzer<float>: the PDF is the TF-Enhanced one; the search over pairs of bucket edges runs on the
    device, one lane per candidate, each accumulating its cost bucket by bucket in the reference's order and types:
    every field of the encoding is identical, and so is the winning candidate."""
    rng = np.random.default_rng(len(kind))
    batches = {
        "normal": lambda: [(rng.standard_normal(30000) * (1 + b) + 0.5).astype(np.float32) for b in range(3)],
        "relu-pareto": lambda: [_relu_pareto(20 + b, 50000) for b in range(2)],
        "negative": lambda: [(-np.abs(rng.standard_normal(10000)) - 0.25).astype(np.float32)],
        "constant": lambda: [np.full(6000, 4, np.float32)],
        "zeros": lambda: [np.zeros(6000, np.float32)],
        "zeros-then-data": lambda: [np.zeros(100, np.float32), rng.standard_normal(9999).astype(np.float32)],
        "far-from-zero": lambda: [(rng.standard_normal(20000) * 0.01 + 50).astype(np.float32)],
        "outliers": lambda: [np.concatenate([rng.standard_normal(50000), [300.0, -120.0]]).astype(np.float32)],
    }[kind]()
    an, pdf = ops.Analyzer(MSE), oracle.new_pdf()
    for b in batches:
        an.update_stats(_gpu(b))
        pdf.update(b)
    for bw, sym, strict, uns in ((8, 0, 0, 0), (8, 1, 0, 0), (8, 1, 1, 0), (8, 1, 0, 1), (4, 0, 0, 0), (4, 1, 0, 0),
                                 (16, 0, 0, 0), (2, 0, 0, 0)):
        e, valid = an.compute_encoding(bw, sym, strict, uns)
        want = pdf.compute_mse_encoding(bw, sym, strict, uns)
        assert valid and (e.min, e.max, e.delta, e.offset, e.bw) == want.astuple(), (kind, bw, sym, strict, uns)


def test_mse_analyzer_edge_behaviour(ops):
    an = ops.Analyzer(MSE)
    e, valid = an.compute_encoding(8)
    assert not valid and (e.min, e.max, e.delta, e.offset) == (0, 0, 0, 0)        # nothing seen
    torch.manual_seed(0)
    x = torch.cat([torch.randn(100000, device="cuda"), torch.tensor([40.0, -35.0], device="cuda")])
    an.update_stats(x)
    xl, p = an.get_stats_histogram()                                              # the PDF is inspectable
    assert len(xl) == 512 and abs(p.sum() - 1.0) < 1e-9
    e4, _ = an.compute_encoding(4)
    e8, _ = an.compute_encoding(8)
    assert e4.max < 40 and e4.min > -35                                           # the outliers are clipped
    assert e4.max - e4.min < e8.max - e8.min                                      # a coarse grid clips more
    tf = ops.Analyzer(0)
    tf.update_stats(x)
    grid = lambda e: torch.clamp(torch.round(x / e.delta) * e.delta, e.min, e.max)
    assert (grid(e4) - x).square().mean() < (grid(tf.compute_encoding(4)[0]) - x).square().mean()
    from aimet_amd._lib import MiqError
    with pytest.raises(MiqError):
        an.last_search()                                                          # the TF-Enhanced analyzer's hook
    an.reset()
    assert not an.compute_encoding(8)[1]


def test_mse_scheme_through_the_tensor_quantizer_object(oracle):
    """libpymo's QuantizationMode.QUANTIZATION_MSE through the AimetTensorQuantizer object
    (TrainingExtensions/torch/src/AimetTensorQuantizer.cpp:74-126 over DLQ/src/QuantizerFactory.cpp:85-88)."""
    from aimet_amd.common import libpymo
    from aimet_amd.common.AimetTensorQuantizer import AimetTensorQuantizer
    rng = np.random.default_rng(9)
    x = (rng.standard_normal(40000) * 2 - 1).astype(np.float32)
    q = AimetTensorQuantizer(libpymo.QuantizationMode.QUANTIZATION_MSE)
    q.updateStats(_gpu(x), True)
    encoding, valid = q.getEncoding(8, False, False, False)
    pdf = oracle.new_pdf()
    pdf.update(x)
    want = pdf.compute_mse_encoding(8)
    assert valid and (encoding.min, encoding.max, encoding.delta, encoding.offset, encoding.bw) == want.astuple()


# -------------------------------------------------------------------------------------------- entropy analyzer
ENTROPY = 4


def _entropy_cases(rng):
    return {
        "normal": [(rng.standard_normal(30000) * (1 + b) + 0.5).astype(np.float32) for b in range(3)],
        "relu-pareto": [_relu_pareto(20 + b, 50000) for b in range(2)],
        "negative": [(-np.abs(rng.standard_normal(10000)) - 0.25).astype(np.float32)],
        "constant": [np.full(6000, 4, np.float32)],
        "zeros": [np.zeros(6000, np.float32)],
        "zeros-then-data": [np.zeros(100, np.float32), rng.standard_normal(9999).astype(np.float32)],
        "far-from-zero": [(rng.standard_normal(20000) * 0.01 + 50).astype(np.float32)],
        # every batch widens the range -- to the right, to the left, on both sides -- then one falls inside it
        "growing-range": [(rng.standard_normal(5003) * s + m).astype(np.float32)
                          for s, m in ((0.5, 0.0), (1.0, 2.0), (1.0, -3.0), (4.0, 0.0), (0.1, 0.0))],
        "large": [rng.standard_normal(3_000_001).astype(np.float32)],
    }


@pytest.mark.parametrize("kind", ["normal", "relu-pareto", "negative", "constant", "zeros", "zeros-then-data",
                                  "far-from-zero", "growing-range", "large"])
def test_entropy_analyzer_matches_the_oracle(ops, oracle, kind):
    """EntropyEncodingAnalyzer<float>: after every batch the histogram -- its range, each of the 512 counts, the
    number of batches counted -- is the reference's, and so is every field of the encoding for each symmetry mode
    (the KL window search runs for 8 bits; other bitwidths keep the histogram's range)."""
    batches = _entropy_cases(np.random.default_rng(len(kind) + 7))[kind]
    an, prof = ops.Analyzer(ENTROPY), oracle.new_profile()
    for b in batches:
        an.update_stats(_gpu(b))
        prof.update(b)
        counts, span, seen, batches_counted = an.entropy_histogram()
        assert seen == prof.initialized and batches_counted == prof.iterations
        if seen:
            assert span == prof.range()
            assert np.array_equal(counts, prof.histogram())
    for bw, sym, strict, uns in ((8, 0, 0, 0), (8, 1, 0, 0), (8, 1, 1, 0), (8, 1, 0, 1), (4, 0, 0, 0), (16, 1, 0, 0)):
        e, valid = an.compute_encoding(bw, sym, strict, uns)
        want = prof.compute_encoding(bw, sym, strict, uns)
        assert valid and (e.min, e.max, e.delta, e.offset, e.bw) == want.astuple(), (kind, bw, sym, strict, uns)


def test_entropy_analyzer_on_views_and_unaligned_tensors(ops, oracle):
    rng = np.random.default_rng(2)
    x = rng.standard_normal(40003).astype(np.float32)
    an, prof = ops.Analyzer(ENTROPY), oracle.new_profile()
    an.update_stats(_gpu(x)[1:])                                                  # not 16-byte aligned
    prof.update(x[1:])
    an.update_stats(_gpu(x)[:7])                                                  # fewer samples than one vector pass
    prof.update(x[:7])
    counts, span, _, _ = an.entropy_histogram()
    assert span == prof.range() and np.array_equal(counts, prof.histogram())


def test_entropy_analyzer_edge_behaviour(ops):
    from aimet_amd._lib import MiqError
    an = ops.Analyzer(ENTROPY)
    e, valid = an.compute_encoding(8)
    assert not valid and (e.min, e.max, e.delta, e.offset) == (0, 0, 0, 0)        # nothing seen
    torch.manual_seed(0)
    x = torch.cat([torch.randn(200000, device="cuda"), torch.tensor([14.0, -11.0], device="cuda")])
    an.update_stats(x)
    counts, span, seen, batches_counted = an.entropy_histogram()
    assert seen and batches_counted == 1 and counts.sum() == x.numel() and span == (-11.0, 14.0)
    e8, _ = an.compute_encoding(8)
    assert -11 < e8.min < 0 < e8.max < 14                                         # the two outliers are cut off
    e4, _ = an.compute_encoding(4)
    assert e4.min <= -11 and e4.max >= 14 - e4.delta                              # no search below or above 8 bits
    with pytest.raises(MiqError):
        an.get_stats_histogram()                                                  # counts, not a PDF
    with pytest.raises(MiqError):
        ops.Analyzer(1).entropy_histogram()
    an.reset()
    assert not an.compute_encoding(8)[1]
    an.update_stats(torch.zeros(100, device="cuda"))
    e, valid = an.compute_encoding(8)
    assert valid and e.offset == -128 and abs(e.min + 1.00392) < 1e-4             # only zeros: the range of [-1, 1]


def test_entropy_scheme_through_the_tensor_quantizer_object(oracle):
    """libpymo's QuantizationMode.QUANTIZATION_ENTROPY through the AimetTensorQuantizer object
    (TrainingExtensions/torch/src/AimetTensorQuantizer.cpp:74-126 over DLQ/src/QuantizerFactory.cpp:89-92)."""
    from aimet_amd.common import libpymo
    from aimet_amd.common.AimetTensorQuantizer import AimetTensorQuantizer
    rng = np.random.default_rng(9)
    x = (rng.standard_normal(40000) * 2 - 1).astype(np.float32)
    q = AimetTensorQuantizer(libpymo.QuantizationMode.QUANTIZATION_ENTROPY)
    q.updateStats(_gpu(x), True)
    encoding, valid = q.getEncoding(8, False, False, False)
    prof = oracle.new_profile()
    prof.update(x)
    want = prof.compute_encoding(8)
    assert valid and (encoding.min, encoding.max, encoding.delta, encoding.offset, encoding.bw) == want.astuple()


def test_encoding_analyzer_for_python(oracle):
    """libpymo.EncodingAnalyzerForPython (PyModelOptimizations.cpp:216-219) with each mode of the factory, fed with a
    numpy array as the reference's callers feed it: every field of the encoding against the oracle."""
    from aimet_amd.common import libpymo
    Mode = libpymo.QuantizationMode
    rng = np.random.default_rng(12)
    x = (rng.standard_normal(30000) * 1.5 + 0.25).astype(np.float32)
    pdf, prof = oracle.new_pdf(), oracle.new_profile()
    pdf.update(x)
    prof.update(x)
    expected = {Mode.QUANTIZATION_TF: oracle.tf_compute_encoding(float(x.min()), float(x.max()), 8),
                Mode.QUANTIZATION_TF_ENHANCED: pdf.compute_encoding(8)[0],
                Mode.QUANTIZATION_PERCENTILE: pdf.compute_percentile_encoding(8, 100.0),
                Mode.QUANTIZATION_MSE: pdf.compute_mse_encoding(8),
                Mode.QUANTIZATION_ENTROPY: prof.compute_encoding(8)}
    for mode, want in expected.items():
        analyzer = libpymo.EncodingAnalyzerForPython(mode)
        encoding, valid = analyzer.computeEncoding(8, False, False, False)
        assert not valid and encoding.delta == 0
        analyzer.updateStats(x, False)
        encoding, valid = analyzer.computeEncoding(8, False, False, False)
        assert valid and encoding.bw == 8 and encoding.min <= 0 <= encoding.max
        assert (encoding.min, encoding.max, encoding.delta, encoding.offset, encoding.bw) == want.astuple(), mode
    # a mode without an analyzer of its own gets the TF analyzer
    fallback = libpymo.EncodingAnalyzerForPython(Mode.QUANTIZATION_RANGE_LEARNING)
    fallback.updateStats(torch.from_numpy(x), True)
    tf = libpymo.EncodingAnalyzerForPython(Mode.QUANTIZATION_TF)
    tf.updateStats(_gpu(x), True)
    a, b = fallback.computeEncoding(8, False, False, False)[0], tf.computeEncoding(8, False, False, False)[0]
    assert (a.min, a.max, a.delta, a.offset) == (b.min, b.max, b.delta, b.offset)
    assert a.min <= float(x.min()) and a.max >= float(x.max()) - a.delta


def test_analyzer_dying_during_a_stream_capture(ops):
    """Destroying an analyzer frees pinned memory, which the runtime refuses during a stream capture (the capture is
    invalidated); the garbage collector may run the destructor right there.  A handle that dies while the current
    stream is capturing is parked and destroyed later."""
    import gc
    x = torch.randn(4096, device="cuda")
    doomed = [ops.Analyzer(mode) for mode in (0, 1, 2, 3, 4)]
    for analyzer in doomed:
        analyzer.update_stats(x)
        analyzer.compute_encoding(8)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        y = x * 2
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        y = x * 2
        del doomed, analyzer
        gc.collect()
        assert len(ops._parked_handles) == 5
    graph.replay()
    torch.cuda.synchronize()
    assert torch.equal(y, x * 2)
    survivor = ops.Analyzer(1)                                                    # outside a capture: parked handles go
    assert not ops._parked_handles
    survivor.update_stats(x)
    assert survivor.compute_encoding(8)[1]


def test_percentile_scheme_through_the_v1_quantizers():
    """test_tensor_quantizer / quantsim flow of the reference with quant_scheme = post_training_percentile."""
    from aimet_amd.common import libpymo
    from aimet_amd.common.defs import QuantScheme
    from aimet_amd.v1.quantsim import QuantizationSimModel
    from aimet_amd.v1.tensor_quantizer import StaticGridPerTensorQuantizer
    torch.manual_seed(0)
    x = torch.randn(40000, device="cuda")
    x[:4] = 500.0
    q = StaticGridPerTensorQuantizer(8, libpymo.RoundingMode.ROUND_NEAREST, QuantScheme.post_training_percentile,
                                     use_symmetric_encodings=False, enabled_by_default=True)
    q.set_percentile_value(99.9)
    q.update_encoding_stats(x)
    q.compute_encoding()
    assert q.encoding.max < 10 and q.encoding.min > -10                   # the outliers are cut off
    q.reset_encoding_stats()
    q.set_percentile_value(100)
    q.update_encoding_stats(x)
    q.compute_encoding()
    assert q.encoding.max > 490

    model = torch.nn.Sequential(torch.nn.Conv2d(3, 8, 3), torch.nn.ReLU(), torch.nn.Conv2d(8, 4, 3)).cuda()
    data = torch.randn(8, 3, 12, 12, device="cuda")
    data[0, 0, 0, 0] = 1000.0
    sim = QuantizationSimModel(model, data[:1], quant_scheme=QuantScheme.post_training_percentile)
    with pytest.raises(ValueError):
        sim.set_percentile_value(80)
    sim.set_percentile_value(99)
    sim.compute_encodings(lambda m, a: m(a), data)
    wrappers = dict(sim.quant_wrappers())
    first = wrappers['0']
    out_enc = wrappers['1'].output_quantizers[0].encoding                  # Conv + ReLU: quantized after the ReLU
    full = model[1](model[0](data))
    assert out_enc.max < full.max().item() * 0.5                           # activations: clipped at 99 %
    w_enc = first.param_quantizers['weight'].encoding
    w_abs = model[0].weight.abs().max().item()
    assert max(abs(w_enc.min), w_enc.max) >= w_abs * 0.99                  # parameters: always 100 %
    assert torch.isfinite(sim.model(data)).all()
