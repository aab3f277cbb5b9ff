"""GPU parity of the v2 histogram observer and SQNR search against the CPU restatement of the reference
(oracle/sqnr_oracle.py: torch CPU ops incl. torch.histc), through the C ABI.

Bar: histogram counts, ranges and the chosen (min, max) identical; candidate scores within 1e-5 relative (they are
summed in double on the GPU and in float32 by torch.sum on the CPU).
"""
import math

import numpy as np
import pytest
import torch

from oracle import sqnr_oracle as sq

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ea():
    from aimet_amd.v2.quantization import encoding_analyzer
    return encoding_analyzer


def _batches(seed):
    g = torch.Generator().manual_seed(seed)
    a = torch.randn(30000, generator=g)
    b = torch.randn(50000, generator=g) * 3 + 1            # range grows on both sides
    c = torch.randn(20000, generator=g) * 0.2               # inside the range
    d = torch.randn(1000, generator=g).abs() * 20           # grows on the right only
    e = a.clone()
    e[:4] = torch.tensor([float('inf'), -float('inf'), float('nan'), 1e30])
    return [a, b, c, d, e]


def _same_hist(dev, ref: sq.Histogram):
    assert torch.equal(dev.histogram.cpu(), ref.histogram)
    assert dev.min.item() == ref.min.item() and dev.max.item() == ref.max.item()
    assert torch.equal(dev.bin_edges.cpu(), ref.bin_edges)


@pytest.mark.parametrize("num_bins", [2048, 512, 100])
def test_histograms_match_torch_histc_across_merges(ea, num_bins):
    obs = ea._HistogramObserver((1,), num_bins)
    ref = sq.SqnrAnalyzer(1, num_bins)
    for x in _batches(1):
        new = obs.collect_and_merge_stats(x.cuda())
        ref_new = ref.update_stats(x)
        _same_hist(new[0], ref_new[0])
        _same_hist(obs.get_stats()[0], ref.stats[0])


def test_edge_inputs(ea):
    for x in (torch.full((1000,), 3.25), torch.zeros(77), torch.tensor([1.0]), torch.tensor([-2.0, 5.0]),
              torch.arange(-100, 101) / 100):
        obs = ea._HistogramObserver((1,), 2048)
        ref = sq.SqnrAnalyzer(1, 2048)
        for rep in range(2):                      # the second round merges an identical batch (equal min and max)
            new = obs.collect_and_merge_stats(x.cuda())
            ref_new = ref.update_stats(x)
            _same_hist(new[0], ref_new[0])
            _same_hist(obs.get_stats()[0], ref.stats[0])
    obs = ea._HistogramObserver((1,), 16)
    stats = obs.collect_and_merge_stats(torch.tensor([float('nan'), float('inf')]).cuda())
    with pytest.raises(ValueError):
        stats[0]
    with pytest.raises(RuntimeError):
        obs.collect_stats(torch.randn(10))        # CPU tensor


def test_large_batch_counts(ea):
    g = torch.Generator().manual_seed(5)
    x = torch.randn(32 * 256 * 28 * 28 // 4, generator=g).abs()
    obs = ea._HistogramObserver((1,), 2048)
    new = obs.collect_and_merge_stats(x.cuda())
    _same_hist(new[0], sq.collect_histogram(x, 2048))


def test_very_large_and_concentrated_inputs(ea):
    """Everything in one bin is the worst case for the per-workgroup counters and the replica merge: a constant tensor of
    more than 130 M elements, first as the batch histogram, then merged a second time; and concentrated data next to
    a few other values."""
    n = 2048 * 63488 + 4099
    x = torch.full((n,), 0.75, device="cuda")
    obs = ea._HistogramObserver((1,), 2048)
    for rep in (1, 2):
        obs.collect_and_merge_stats(x)
        hist = obs.get_stats()[0].histogram
        want = float(np.float32(rep * n))             # the histogram is float32, as torch.histc's is
        assert hist.max().item() == want and (hist > 0).sum().item() == 1
    del x
    y = torch.zeros(40_000_000, device="cuda")
    y[::1000] = 1.0
    y[1::1000] = 1.0 / 2048          # the bin next to the zeros'
    obs = ea._HistogramObserver((1,), 2048)
    new = obs.collect_and_merge_stats(y)
    hist = new[0].histogram
    assert hist[0].item() == 40_000_000 - 80_000 and hist[1].item() == 40_000 and hist[-1].item() == 40_000
    assert hist.sum().item() == 40_000_000


def test_updates_inside_and_outside_the_running_range(ea):
    """An update of running statistics bins the batch over the statistics' range while it looks for the batch's own
    range, and redoes the binning only when the range grew.  Long runs of batches that stay inside, batches that grow
    the range on one side or both, a batch that repeats the extremes exactly, non-finite values in either kind of
    batch, sizes that are not a multiple of the vector width: the running histogram equals torch.histc + merge_stats
    of the restatement after every update, and the counters the library keeps in its workspace are back at zero."""
    g = torch.Generator().manual_seed(21)
    obs = ea._HistogramObserver((1,), 2048)
    ref = sq.SqnrAnalyzer(1, 2048)
    first = torch.randn(70001, generator=g) * 2
    plan = [first]
    plan += [torch.randn(50000 + 7 * k, generator=g) * 0.5 for k in range(6)]            # inside
    plan += [torch.cat([torch.randn(1000, generator=g), first.max().view(1), first.min().view(1)])]   # touches both ends
    plan += [torch.randn(30000, generator=g) * 4]                                          # grows on both sides
    plan += [torch.randn(30000, generator=g) for _ in range(3)]                            # inside the new range
    plan += [torch.rand(999, generator=g) * 40]                                            # grows on the right
    inside_bad = torch.randn(20000, generator=g)
    inside_bad[:3] = torch.tensor([float('nan'), float('inf'), -float('inf')])
    plan += [inside_bad]                                                                   # inside, non-finite values
    grow_bad = torch.randn(20000, generator=g) * 30
    grow_bad[5:8] = torch.tensor([float('nan'), float('inf'), -float('inf')])
    plan += [grow_bad, torch.randn(4096 * 64, generator=g)]
    for x in plan:
        obs.merge_stats(None, x.cuda())
        ref.update_stats(x)
        _same_hist(obs.get_stats()[0], ref.stats[0])
        assert int(obs._workspace[:2 * 2048].abs().sum()) == 0                    # pylint: disable=protected-access


def test_per_channel_updates_where_some_ranges_grow(ea):
    """Per-channel statistics, one update in which some channels stay inside their range and others grow: each
    histogram takes its own path."""
    torch.manual_seed(22)
    shape = (5, 1, 1)
    obs = ea._HistogramObserver(shape, 512)
    ref = sq.SqnrAnalyzer(5, 512)
    base = torch.randn(5, 40, 1000)
    scales = [torch.tensor(v).view(5, 1, 1) for v in ([1.0] * 5, [0.5, 2.0, 0.5, 3.0, 0.9], [0.1] * 5,
                                                       [4.0, 0.2, 0.2, 0.2, 5.0], [1.0] * 5)]
    for k, sc in enumerate(scales):
        x = torch.randn(5, 40, 1000) * sc if k else base
        obs.merge_stats(None, x.cuda())
        ref.update_stats(x)
        st = obs.get_stats()
        for i in range(5):
            _same_hist(st[i], ref.stats[i])
    # rows long enough for the wide workgroups, a length that is and one that is not a multiple of the vector width
    for length in (262144, 200003):
        obs = ea._HistogramObserver((3, 1), 2048)
        ref = sq.SqnrAnalyzer(3, 2048)
        for sc in ([1.0, 1.0, 1.0], [0.5, 2.0, 0.7], [0.3, 0.3, 3.0], [1.0, 1.0, 1.0]):
            x = torch.randn(3, length) * torch.tensor(sc).view(3, 1)
            obs.merge_stats(None, x.cuda())
            ref.update_stats(x)
            st = obs.get_stats()
            for i in range(3):
                _same_hist(st[i], ref.stats[i])


@pytest.mark.parametrize("symmetric", [False, True])
@pytest.mark.parametrize("num_steps,gamma", [(255.0, 3.0), (255.0, 1.0), (15.0, 3.0), (65535.0, 3.0)])
def test_search_matches_restatement(ea, symmetric, num_steps, gamma):
    an = ea.SqnrEncodingAnalyzer((1,), gamma=gamma)
    ref = sq.SqnrAnalyzer(1, 2048, gamma=gamma)
    g = torch.Generator().manual_seed(7)
    for scale, shift in ((1.0, 0.3), (2.0, -0.5)):
        x = torch.randn(40000, generator=g) * scale + shift
        x[:3] = torch.tensor([25.0, -14.0, 18.0])          # outliers: clipping is worth it
        an.update_stats(x.cuda())
        ref.update_stats(x)
    rmin, rmax, rnoise = ref.compute_encodings(num_steps, symmetric)
    st = an.observer.get_stats()
    from aimet_amd import ops
    gmin, gmax, gnoise, best = ops.v2_sqnr_search(st.hist, st.minmax, num_steps, symmetric, gamma, 17, 101, 21,
                                                  want_details=True)
    assert gnoise.shape == rnoise.shape
    assert torch.allclose(gnoise.cpu().float(), rnoise, rtol=1e-5, atol=0)
    ref_best = int(torch.argmin(rnoise[0]))
    if int(best[0]) != ref_best:
        # a near-tie resolved differently by the two summation orders: the scores must be indistinguishable
        assert abs(rnoise[0, int(best[0])] - rnoise[0, ref_best]) <= 2e-6 * rnoise[0, ref_best]
    else:
        assert torch.equal(gmin.cpu(), rmin) and torch.equal(gmax.cpu(), rmax)
    qmin, qmax = an.compute_encodings(num_steps, symmetric)
    assert torch.equal(qmin, gmin.view(1)) and torch.equal(qmax, gmax.view(1))


def test_per_channel(ea):
    torch.manual_seed(10)
    x = torch.randn(6, 3, 5, 100) * torch.linspace(0.5, 3, 6).view(6, 1, 1, 1)
    shape = (6, 1, 1, 1)
    an = ea.SqnrEncodingAnalyzer(shape)
    ref = sq.SqnrAnalyzer(6, 2048)
    for t in (x, x / 2, x * 1.5):
        an.update_stats(t.cuda())
        ref.update_stats(t)
    st = an.observer.get_stats()
    for i in range(6):
        _same_hist(st[i], ref.stats[i])
        assert st[i].min.item() == (x[i] * 1.5).min().item() and st[i].max.item() == (x[i] * 1.5).max().item()
    qmin, qmax = an.compute_encodings(255.0, False)
    rmin, rmax, _ = ref.compute_encodings(255.0, False)
    assert qmin.shape == shape and qmax.shape == shape
    assert torch.equal(qmin.cpu().view(-1), rmin) and torch.equal(qmax.cpu().view(-1), rmax)
    with pytest.raises(RuntimeError):
        ea.SqnrEncodingAnalyzer((1, 4, 1, 1)).update_stats(x.cuda())     # shape does not broadcast to the input


@pytest.mark.parametrize("num_bins", [4096, 2048, 64])
def test_short_rows_at_several_bin_counts(ea, num_bins):
    """Six short rows per update at the largest bin count the library takes (the general kernels), the default one
    and a small one (one launch per update)."""
    torch.manual_seed(24)
    obs = ea._HistogramObserver((6, 1), num_bins)
    ref = sq.SqnrAnalyzer(6, num_bins)
    for sc in (1.0, 0.4, 2.5, 1.0):
        x = torch.randn(6, 1500) * sc
        obs.merge_stats(None, x.cuda())
        ref.update_stats(x)
        st = obs.get_stats()
        for i in range(6):
            _same_hist(st[i], ref.stats[i])


@pytest.mark.parametrize("length", [1500, 6144, 7004, 7001])
def test_many_rows_one_workgroup_each(ea, length):
    """More than a thousand histograms per update: each row goes to one workgroup that does the whole update (rows that
    fit its registers, rows it reads twice, a length that is not a multiple of the vector width), first batch, batches
    inside the range and batches that grow some rows' ranges, rows with non-finite values."""
    torch.manual_seed(23)
    rows = 1100
    obs = ea._HistogramObserver((rows, 1), 2048)
    grow = torch.ones(rows, 1)
    grow[::7] = 3.0
    sample = sorted(set(list(range(0, rows, 97)) + [3, 7, rows - 1]))   # the restatement follows these rows only
    ref = sq.SqnrAnalyzer(len(sample), 2048)
    for k, sc in enumerate((1.0, 0.5, grow, 0.8)):
        x = torch.randn(rows, length) * sc
        if k == 1:
            x[3, :3] = torch.tensor([float('nan'), float('inf'), -float('inf')])
        obs.merge_stats(None, x.cuda())
        ref.update_stats(x[sample])
        st = obs.get_stats()
        for at, i in enumerate(sample):
            _same_hist(st[i], ref.stats[at])


@pytest.mark.parametrize("symmetric", [False, True])
def test_many_sparse_channels(ea, symmetric):
    """96 channels of 300 samples: most of the 2048 bins of a channel are empty, and a search over this many histograms
    walks only the bins that hold something.  Scores and choices against the restatement, which walks all bins."""
    torch.manual_seed(11)
    channels = 96
    x = torch.randn(channels, 300) * torch.logspace(-2, 2, channels).view(-1, 1) + torch.linspace(-1, 1, channels).view(-1, 1)
    x[5] = 0.0                                             # one histogram with a single occupied bin
    an = ea.SqnrEncodingAnalyzer((channels, 1))
    ref = sq.SqnrAnalyzer(channels, 2048)
    an.update_stats(x.cuda())
    ref.update_stats(x)
    rmin, rmax, rnoise = ref.compute_encodings(255.0, symmetric)
    st = an.observer.get_stats()
    from aimet_amd import ops
    gmin, gmax, gnoise, best = ops.v2_sqnr_search(st.hist, st.minmax, 255.0, symmetric, 3.0, 17, 101, 21,
                                                  want_details=True)
    assert (st.hist == 0).float().mean().item() > 0.8
    assert torch.allclose(gnoise.cpu().float(), rnoise, rtol=1e-5, atol=0)
    ref_best = torch.argmin(rnoise, dim=1)
    agree = best.cpu().long() == ref_best
    assert agree.float().mean().item() > 0.9
    assert torch.equal(gmin.cpu()[agree], rmin[agree]) and torch.equal(gmax.cpu()[agree], rmax[agree])
    for c in torch.nonzero(~agree).flatten().tolist():
        # a near-tie resolved differently by the two summation orders: the scores must be indistinguishable
        assert abs(rnoise[c, int(best[c])] - rnoise[c, int(ref_best[c])]) <= 2e-6 * rnoise[c, int(ref_best[c])]


def test_reference_cases_through_the_analyzer(ea):
    # test_encoding_analyzer.py:659-674: equally spaced input, gamma = 1 -> the observed range exactly
    x = torch.arange(-100, 101) / 100
    an = ea.SqnrEncodingAnalyzer(shape=(1,), gamma=1)
    observed_delta = torch.tensor(2 / 255.0)
    observed_offset = torch.round(-1 / observed_delta)
    observed_min = observed_offset * observed_delta
    observed_max = observed_min + 255 * observed_delta
    an.update_stats(x.cuda())
    qmin, qmax = an.compute_encodings(num_steps=math.pow(2, 8) - 1, is_symmetric=False)
    assert torch.equal(qmin.cpu(), observed_min.view((1,))) and torch.equal(qmax.cpu(), observed_max.view((1,)))
    # :676-709: one severe outlier is clipped at 3/4 of its value
    expected_delta = torch.Tensor([0.1])
    outlier_val = (255 * expected_delta) / 0.75
    n = round(12 * 255 * outlier_val.item() / expected_delta.item() - 12 * (255 ** 2))
    an = ea.SqnrEncodingAnalyzer((1,), gamma=1.0)
    torch.manual_seed(0)
    an.update_stats((torch.rand((1, n)) * 255 * expected_delta).cuda())
    an.update_stats(torch.Tensor([outlier_val]).view(1, 1).cuda())
    qmin, qmax = an.compute_encodings(math.pow(2, 8) - 1, is_symmetric=False)
    assert torch.allclose(qmin.cpu(), torch.Tensor([0])) and torch.allclose(qmax.cpu(), expected_delta * 255)
    # no statistics / bad arguments
    from aimet_amd.v2.utils import StatisticsNotFoundError
    fresh = ea.SqnrEncodingAnalyzer((1,))
    with pytest.raises(StatisticsNotFoundError):
        fresh.compute_encodings(255, False)
    with pytest.raises(ValueError):
        an.compute_encodings(0, False)
    with pytest.raises(ValueError):
        ea.SqnrEncodingAnalyzer((1,), num_bins=0)
    # dynamic encodings from the batch's own statistics
    dmin, dmax = an.compute_dynamic_encodings(torch.randn(1000).cuda(), 255, False)
    assert dmin.shape == (1,) and dmin.item() < 0 < dmax.item()


def test_quantizer_with_sqnr_analyzer(ea):
    """QuantizeDequantize calibrated by the SQNR analyzer (the injection point of the reference's quantizer ctor)."""
    from aimet_amd.v2.quantization.affine import QuantizeDequantize
    torch.manual_seed(3)
    x = torch.randn(64, 128).cuda()
    x[0, 0] = 40.0
    q = QuantizeDequantize((), bitwidth=8, symmetric=False, encoding_analyzer=ea.SqnrEncodingAnalyzer(())).cuda()
    with q.compute_encodings():
        q(x)
    assert q.is_initialized()
    want_min, want_max = q.encoding_analyzer.compute_encodings(255, False)
    # the quantizer snaps the range to its grid (offset rounding): within one step of the analyzer's answer
    assert abs(q.get_min().item() - want_min.item()) <= q.get_scale().item()
    assert abs(q.get_max().item() - want_max.item()) <= q.get_scale().item()
    y = q(x)
    inside = (x >= q.get_min()) & (x <= q.get_max())
    assert (y - x)[inside].abs().max().item() <= 0.5 * q.get_scale().item() * 1.001


# ------------------------------------------------------------------------------------------ percentile calibration
def test_percentile_known_answers_on_gpu(ea):
    # test_encoding_analyzer.py:544-655 of the reference
    for bad in (-1, 49, 5, 101):
        with pytest.raises(ValueError):
            ea.PercentileEncodingAnalyzer((), percentile=bad, num_bins=3)
    x = torch.arange(start=0, end=1001, step=1, dtype=torch.float).cuda()
    an = ea.PercentileEncodingAnalyzer((), percentile=99, num_bins=500)
    an.update_stats(x)
    lo, hi = an.compute_encodings(num_steps=math.pow(2, 8) - 1, is_symmetric=False)
    assert lo.item() == 0 and hi.item() == 990.0 and lo.shape == ()
    lo, hi = an.compute_encodings(num_steps=math.pow(2, 8) - 2, is_symmetric=True)
    assert lo.item() == -990.0 and hi.item() == 990.0
    an = ea.PercentileEncodingAnalyzer((), percentile=100, num_bins=1)
    an.update_stats(torch.arange(start=-2, end=10, step=1, dtype=torch.float).cuda())
    lo, hi = an.compute_encodings(is_symmetric=True, num_steps=pow(2, 3) - 1)
    assert lo.item() == pytest.approx(-12.0) and hi.item() == pytest.approx(9.0)
    x = torch.arange(start=0, end=101, step=1, dtype=torch.float)
    x[-1], x[-2] = 1000, 800
    an = ea.PercentileEncodingAnalyzer(num_bins=2048, shape=(1,), percentile=90.)
    an.update_stats(x.cuda())
    lo, hi = an.compute_encodings(num_steps=255, is_symmetric=False)
    assert 89 < hi.item() < 91
    with pytest.raises(Exception):
        ea.PercentileEncodingAnalyzer((), percentile=99).compute_encodings(255, False)      # no statistics


@pytest.mark.parametrize("percentile", [100, 99.9, 99, 90, 50])
@pytest.mark.parametrize("symmetric", [False, True])
def test_percentile_matches_the_restatement(ea, percentile, symmetric):
    torch.manual_seed(12)
    x = torch.randn(5, 4000) * torch.linspace(0.5, 3, 5).view(5, 1) + 0.3
    x[2, :10] = 40.0                                            # outliers in one channel
    an = ea.PercentileEncodingAnalyzer((5, 1), num_bins=512, percentile=percentile)
    ref = sq.PercentileAnalyzer(5, 512, percentile)
    for t in (x, x * 0.7, x * 1.2 - 0.1):
        an.update_stats(t.cuda())
        ref.update_stats(t)
    lo, hi = an.compute_encodings(255, symmetric)
    rlo, rhi = ref.compute_encodings(255, symmetric)
    assert lo.shape == (5, 1)
    assert torch.allclose(lo.cpu().view(-1), rlo.view(-1), rtol=1e-6, atol=0)
    assert torch.allclose(hi.cpu().view(-1), rhi.view(-1), rtol=1e-6, atol=0)


def test_quantizer_module_with_percentile_analyzer(ea):
    from aimet_amd.v2.quantization import affine
    torch.manual_seed(13)
    x = torch.randn(64, 256).cuda()
    x[0, 0] = 100.0
    q = affine.QuantizeDequantize((), 8, False,
                                  encoding_analyzer=ea.PercentileEncodingAnalyzer((), percentile=99.9)).cuda()
    with q.compute_encodings():
        q(x)
    assert q.get_max().item() < 10                               # the outlier is clipped away
    err = (q(x) - x).abs().flatten()
    assert err.median().item() <= q.get_scale().item() / 2 and (err > q.get_scale().item()).float().mean() < 0.003
