"""The cases of the reference's own encoding-analyzer tests (TrainingExtensions/torch/test/python/v2/quantization/
test_encoding_analyzer.py:51-540) on the GPU analyzers: behaviour common to all analyzers, the min-max analyzer, the
histogram observer (range merges, infinities, multi-dimensional shapes)."""
import math

import pytest
import torch

import _hist_cases as hc

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ea():
    from aimet_amd.v2.quantization import encoding_analyzer
    return encoding_analyzer


def _all_analyzers(ea):
    return [ea.MinMaxEncodingAnalyzer(()), ea.PercentileEncodingAnalyzer((), num_bins=3, percentile=99),
            ea.SqnrEncodingAnalyzer((1,))]


# ------------------------------------------------------------------------------------------- every analyzer (:51-110)
def test_compute_encodings_with_invalid_num_steps(ea):
    for an in _all_analyzers(ea):
        an.update_stats(torch.randn(3, 4).cuda())
        with pytest.raises(ValueError):
            an.compute_encodings(num_steps=0, is_symmetric=False)


def test_reset_stats(ea):
    for an in _all_analyzers(ea):
        an.update_stats(torch.randn(3, 4).cuda())
        if isinstance(an, ea.MinMaxEncodingAnalyzer):
            assert an.observer.stats.min is not None and an.observer.stats.max is not None
        else:
            assert all(x.min is not None and x.max is not None for x in an.observer.stats)
        an.reset_stats()
        if isinstance(an, ea.MinMaxEncodingAnalyzer):
            assert an.observer.stats.min is None and an.observer.stats.max is None
        else:
            assert all(x.min is None and x.max is None for x in an.observer.stats)


def test_compute_encodings_with_no_stats(ea):
    for an in _all_analyzers(ea):
        with pytest.raises(RuntimeError):
            an.compute_encodings(num_steps=8, is_symmetric=False)


@pytest.mark.parametrize('dtype', [torch.float, torch.half])
@pytest.mark.parametrize('symmetric', [True, False])
def test_continuity(ea, symmetric, dtype):
    # a range scaled by (1 -+ eps) moves the encodings by at most eps, monotonically
    for an in _all_analyzers(ea):
        normal_range = torch.arange(-128, 128).to(dtype).cuda() / 256
        eps = torch.finfo(dtype).eps
        num_steps = math.pow(2, 8) - 2
        min_1, max_1 = an.compute_dynamic_encodings(normal_range * (1 - eps), num_steps=num_steps,
                                                    is_symmetric=symmetric)
        min_2, max_2 = an.compute_dynamic_encodings(normal_range, num_steps=num_steps, is_symmetric=symmetric)
        min_3, max_3 = an.compute_dynamic_encodings(normal_range * (1 + eps), num_steps=num_steps,
                                                    is_symmetric=symmetric)
        assert min_3 <= min_2 <= min_1 <= max_1 <= max_2 <= max_3
        for a, b in ((max_1, max_2), (min_1, min_2), (max_2, max_3), (min_2, min_3)):
            assert torch.allclose(a.float(), b.float(), atol=eps)


# --------------------------------------------------------------------------------------- min-max analyzer (:112-205)
def test_minmax_known_answers(ea):
    an = ea.MinMaxEncodingAnalyzer(())
    an.update_stats(torch.arange(start=0, end=26, step=0.5, dtype=torch.float).cuda())
    lo, hi = an.compute_encodings(num_steps=math.pow(2, 8) - 1, is_symmetric=False)
    assert torch.isclose(lo, torch.zeros((), device="cuda")) and torch.isclose(hi, torch.tensor(25.5, device="cuda"))
    lo, hi = an.compute_encodings(num_steps=math.pow(2, 8) - 2, is_symmetric=True)
    assert torch.isclose(lo, torch.tensor(-25.5, device="cuda")) and torch.isclose(hi, torch.tensor(25.5, device="cuda"))
    an = ea.MinMaxEncodingAnalyzer(())
    an.update_stats(torch.arange(start=-2, end=10, step=1, dtype=torch.float).cuda())
    lo, hi = an.compute_encodings(is_symmetric=True, num_steps=pow(2, 3) - 1)
    assert lo.item() == pytest.approx(-12.0) and hi.item() == pytest.approx(9.0)


@pytest.mark.parametrize("min_max_size", [[3, 4], [2, 3, 1], [4], [1]])
def test_minmax_update_stats_with_different_dimensions(ea, min_max_size):
    x = torch.randn(2, 3, 4)
    an = ea.MinMaxEncodingAnalyzer(min_max_size)
    an.update_stats(x.cuda())
    assert list(an.observer.stats.min.shape) == min_max_size and list(an.observer.stats.max.shape) == min_max_size
    padded = [1] * (3 - len(min_max_size)) + list(min_max_size)
    reduce_dims = [d for d in range(3) if padded[d] == 1]
    assert torch.equal(an.observer.stats.min.cpu(), x.amin(dim=reduce_dims, keepdim=True).reshape(min_max_size))
    assert torch.equal(an.observer.stats.max.cpu(), x.amax(dim=reduce_dims, keepdim=True).reshape(min_max_size))
    with pytest.raises(RuntimeError):
        ea.MinMaxEncodingAnalyzer([3, 4]).update_stats(torch.randn(2, 3, 5).cuda())


def test_minmax_degenerate_inputs(ea):
    an = ea.MinMaxEncodingAnalyzer(())
    an.update_stats(torch.full((), 3.0).cuda())
    num_steps = pow(2, 8) - 1
    lo, hi = an.compute_encodings(num_steps=num_steps, is_symmetric=False)
    assert lo.item() == 0.0 and hi.item() == pytest.approx(3.0)
    lo, hi = an.compute_encodings(num_steps=num_steps - 1, is_symmetric=True)
    assert lo.item() == pytest.approx(-3.0) and hi.item() == pytest.approx(3.0)
    an = ea.MinMaxEncodingAnalyzer(())
    an.update_stats(torch.zeros(()).cuda())
    eps = torch.finfo(torch.float32).eps
    lo, hi = an.compute_encodings(num_steps=num_steps, is_symmetric=False)
    assert lo.item() == 0 and hi.item() == pytest.approx(eps * num_steps, rel=1e-6)
    lo, hi = an.compute_encodings(num_steps=num_steps, is_symmetric=True)
    assert lo.item() == pytest.approx(-eps * math.ceil(num_steps / 2), rel=1e-6)
    assert hi.item() == pytest.approx(eps * math.floor(num_steps / 2), rel=1e-6)


@pytest.mark.parametrize('symmetric', [True, False])
def test_minmax_overflow(ea, symmetric):
    an = ea.MinMaxEncodingAnalyzer(())
    an.update_stats((torch.arange(10) * torch.finfo(torch.float).eps).cuda())
    num_steps = pow(2, 8) - 2
    lo, hi = an.compute_encodings(num_steps=num_steps, is_symmetric=symmetric)
    scale = (hi - lo) / 255
    assert scale != 0 and torch.allclose(scale, torch.tensor(torch.finfo(scale.dtype).eps, device="cuda"), rtol=0.01)
    an.update_stats((torch.arange(10) * torch.finfo(torch.float).max).cuda())
    lo, hi = an.compute_encodings(num_steps=num_steps, is_symmetric=symmetric)
    assert torch.all(torch.isfinite(lo)) and torch.all(torch.isfinite(hi))


# ------------------------------------------------------------------------------------- histogram observer (:207-540)
@pytest.mark.parametrize("name,num_bins,steps", hc.MERGE_CASES)
def test_histogram_merge_cases(ea, name, num_bins, steps):
    an = ea.PercentileEncodingAnalyzer((), num_bins=num_bins, percentile=99)
    for batch, mn, mx, hist, edges in steps:
        an.update_stats(torch.tensor(batch, dtype=torch.float32).cuda())
        assert len(an.observer.stats) == 1
        st = an.observer.stats[0]
        assert st.min.item() == pytest.approx(mn) and st.max.item() == pytest.approx(mx), name
        if hist is not None:
            assert st.histogram.tolist() == hist, name
            assert torch.allclose(st.bin_edges.cpu(), torch.tensor(edges, dtype=torch.float32)), name
        assert st.histogram.is_cuda and st.bin_edges.is_cuda


def test_histogram_infinite_inputs(ea):
    an = ea.PercentileEncodingAnalyzer((), num_bins=10, percentile=99)
    for batch, mn, mx, bins, edges in hc.INF_CASE:
        an.update_stats(torch.tensor(batch).cuda())
        st = an.observer.stats[0]
        assert st.min.item() == mn and st.max.item() == mx
        for b, count in bins.items():
            assert st.histogram[b].item() == count
        assert torch.allclose(st.bin_edges.cpu(), torch.tensor(edges))
    old = an.observer.stats[0].histogram.clone()
    an.update_stats(torch.tensor(hc.INF_THIRD_BATCH).cuda())
    st = an.observer.stats[0]
    assert st.histogram[0] == old[0] + 2 and st.histogram[-1] == old[-1] + 1
    # nothing finite at all: reported when the statistics are next read
    bad = ea.PercentileEncodingAnalyzer((), num_bins=10, percentile=99)
    bad.update_stats(torch.tensor([hc.INF, -hc.INF, -hc.INF, hc.INF, hc.INF]).cuda())
    with pytest.raises(ValueError):
        _ = bad.observer.stats[0]


def test_histogram_degenerate_inputs(ea):
    # :219-255: a single repeated value / only zeros -> a one-unit-wide histogram around it
    for value in (3.0, 0.0):
        an = ea.PercentileEncodingAnalyzer((), num_bins=3, percentile=99)
        an.update_stats(torch.full((), value).cuda())
        st = an.observer.stats[0]
        cum_sum = torch.cumsum(st.histogram, dim=0)
        edge = st.bin_edges[torch.searchsorted(cum_sum, torch.quantile(cum_sum, 99 / 100))]
        num_steps = pow(2, 8) - 1
        lo, hi = an.compute_encodings(num_steps=num_steps, is_symmetric=False)
        if value > 0:
            assert lo.item() == 0.0 and torch.allclose(hi, edge)
            lo, hi = an.compute_encodings(num_steps=num_steps - 1, is_symmetric=True)
            assert torch.allclose(lo, -edge) and torch.allclose(hi, edge)
        else:
            assert torch.allclose(lo, edge) and hi.item() == 0
            lo, hi = an.compute_encodings(num_steps=num_steps - 1, is_symmetric=True)
            assert torch.allclose(lo, edge) and torch.allclose(hi, -edge)
    for num_bins in (-1, 0):
        with pytest.raises(ValueError):
            ea.PercentileEncodingAnalyzer(num_bins=num_bins, shape=(), percentile=99)
        with pytest.raises(ValueError):
            ea.SqnrEncodingAnalyzer((), num_bins)


@pytest.mark.parametrize('symmetric', [True, False])
@pytest.mark.parametrize('shape', [(4,), (3, 1), (2, 1, 1), (3, 4), (2, 3, 1), (2, 1, 4), (2, 3, 4)])
def test_compute_encodings_multidimensional(ea, symmetric, shape):
    # :434-450
    x = torch.arange(24, dtype=torch.float).view(2, 3, 4).cuda()
    for an in (ea.PercentileEncodingAnalyzer(shape=shape, percentile=99), ea.SqnrEncodingAnalyzer(shape=shape)):
        an.update_stats(x)
        lo, hi = an.compute_encodings(num_steps=math.pow(2, 8) - 1, is_symmetric=symmetric)
        assert lo.shape == shape and hi.shape == shape and lo.is_cuda and hi.is_cuda


def test_collect_stats_multidimensional(ea):
    # :452-512: histogram i belongs to element i of the observer shape, in row-major order
    x = torch.arange(24, dtype=torch.float).view(2, 3, 4)
    for shape in ((4,), (3, 1), (2, 1, 1), (3, 4), (2, 3, 1), (2, 1, 4), (2, 3, 4)):
        observer = ea._HistogramObserver(shape, num_bins=5)      # pylint: disable=protected-access
        histograms = observer.collect_stats(x.cuda())
        padded = (1,) * (3 - len(shape)) + tuple(shape)
        reduce_dims = [d for d in range(3) if padded[d] == 1]
        want_min = (x.amin(dim=reduce_dims) if reduce_dims else x).reshape(-1)
        want_max = (x.amax(dim=reduce_dims) if reduce_dims else x).reshape(-1)
        assert len(histograms) == want_min.numel()
        for i in range(want_min.numel()):
            assert histograms[i].min.item() == want_min[i].item() and histograms[i].max.item() == want_max[i].item()
            assert histograms[i].histogram.sum().item() == 24 // want_min.numel()
