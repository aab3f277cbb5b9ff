"""Pins the restatement of the v2 SQNR encoding analyzer (oracle/sqnr_oracle.py) to the reference's own tests
(TrainingExtensions/torch/test/python/v2/quantization/test_encoding_analyzer.py:657-881) and to brute force."""
import math

import numpy as np
import pytest
import torch

from oracle import sqnr_oracle as sq


def test_uniform_grid_gives_observed_encodings_exactly():
    # test_encoding_analyzer.py:659-674
    x = torch.arange(-100, 101) / 100
    an = sq.SqnrAnalyzer(gamma=1)
    observed_delta = torch.tensor(2 / 255.0)
    observed_offset = torch.round(-1 / observed_delta)
    observed_min = observed_offset * observed_delta
    observed_max = observed_min + 255 * observed_delta
    an.update_stats(x)
    qmin, qmax, _ = an.compute_encodings(math.pow(2, 8) - 1, False)
    assert torch.equal(qmin, observed_min.view((1,)))
    assert torch.equal(qmax, observed_max.view((1,)))


def test_outlier_is_clipped_to_three_quarters():
    # test_encoding_analyzer.py:676-709: n = 260,100 uniform samples + one outlier -> min 0, max 25.5
    expected_delta = torch.Tensor([0.1])
    outlier_val = (255 * expected_delta) / 0.75
    n = round(12 * 255 * outlier_val.item() / expected_delta.item() - 12 * (255 ** 2))
    assert n == 260100                                # (the comment in the reference test says 210,100)
    torch.manual_seed(0)
    an = sq.SqnrAnalyzer(gamma=1.0)
    an.update_stats(torch.rand((1, n)) * 255 * expected_delta)
    an.update_stats(torch.Tensor([outlier_val]).view(1, 1))
    qmin, qmax, _ = an.compute_encodings(math.pow(2, 8) - 1, False)
    assert torch.allclose(qmin, torch.Tensor([0]))
    assert torch.allclose(qmax, expected_delta * 255)


def test_clamp_delta_offset_candidates():
    # test_encoding_analyzer.py:746-771
    num_steps = 255
    deltas = torch.Tensor([[1 / 4, 3 / 4, 5 / 4]])
    offsets = torch.Tensor([-255, -128, 0])[None, :]
    should_clamp = torch.Tensor([[False, False, False], [True, False, True], [True, True, True]]).to(torch.bool)
    dc, oc = sq.clamp_delta_offset_values(torch.Tensor([-128]), torch.Tensor([127]), num_steps, deltas, offsets)
    assert torch.all(torch.where(should_clamp, dc < deltas[:, :, None], dc == deltas[:, :, None]))
    mn = dc * oc
    assert torch.all(mn > -128.5) and torch.all(mn + dc * num_steps < 127.5)


def test_pick_test_candidates():
    # test_encoding_analyzer.py:773-834
    deltas, offsets = sq.pick_test_candidates_asymmetric(torch.Tensor([-128]), torch.Tensor([127]), 255,
                                                         num_deltas=5, num_offset_candidates=7)
    assert deltas.shape == (1, 5, 7) and offsets.shape == (1, 5, 7)
    for value in [1 / 4, 1 / 2, 3 / 4, 1]:
        assert value in deltas
    for value in [-255, -204, -153, -102, -51, 0, -128]:
        assert value in offsets
    mn = torch.round(offsets * deltas)
    assert torch.all(mn > -128.5) and torch.all(mn + deltas * 255 < 127.5)
    deltas, offsets = sq.pick_test_candidates_symmetric(torch.Tensor([-100]), torch.Tensor([127.5]), 255, num_deltas=5)
    assert deltas.shape == (1, 5, 1)
    for value in [1 / 4, 1 / 2, 3 / 4, 1]:
        assert value in deltas
    assert torch.all(offsets == -128) and offsets.numel() == 1


def test_estimated_noise_is_close_to_measured_noise():
    # test_encoding_analyzer.py:836-862
    torch.manual_seed(1)
    x = torch.randn(2, 1000)
    x[0][0] = 100
    x[0][1] = -50
    hists = [sq.collect_histogram(x[i], 2048) for i in range(2)]
    deltas = torch.Tensor([0.001, 0.1, 0.5, 1.0])[None, :, None].expand(2, 4, 6)
    offsets = torch.Tensor([-255, -204, -153, -102, -51, 0]).expand_as(deltas)
    d, o = deltas[:, :, :, None], offsets[:, :, :, None]
    qdq = x[:, None, None, :].div(d).sub(o).round().clamp(0, 255).add(o).mul(d)
    exp = torch.pow(x[:, None, None, :] - qdq, 2).sum(dim=-1)
    est = sq.estimate_clip_and_quant_noise(hists, deltas, offsets, 255, gamma=1.0)
    assert torch.allclose(exp, est, rtol=0.01)


def test_select_best_delta_offset():
    # test_encoding_analyzer.py:864-881
    torch.manual_seed(2)
    x = (torch.rand(2, 1000) - torch.Tensor([[0.5], [0.0]])) * torch.Tensor([[1.], [2.]])
    hists = [sq.collect_histogram(x[i], 2048) for i in range(2)]
    deltas = torch.Tensor([1 / 510.0, 1 / 255.0, 2 / 255.0])[None, :, None].expand(2, 3, 3)
    offsets = torch.Tensor([-200, -128, 0]).expand_as(deltas)
    bd, bo, _ = sq.select_best_candidates(deltas, offsets, hists, 255, 1.0)
    assert torch.equal(bd, torch.Tensor([1 / 255.0, 2 / 255.0]).view(2, 1))
    assert torch.equal(bo, torch.Tensor([-128, 0]).view(2, 1))


def test_histogram_against_brute_force_binning():
    """collect_histogram against a direct count of elements per bin in float64 (away from bin boundaries the two must
    agree; Σ counts must equal the number of finite-or-infinite, non-NaN elements)."""
    torch.manual_seed(3)
    x = torch.randn(50000) * 3
    x[:5] = torch.tensor([float('inf'), -float('inf'), float('nan'), 7.5, -7.5])
    h = sq.collect_histogram(x, 2048)
    assert h.histogram.sum().item() == 49999          # NaN dropped, +-inf folded into the end bins
    lo, hi = h.bin_edges[0].double(), h.bin_edges[-1].double()
    xf = x[x.isfinite()].double()
    pos = torch.clamp(((xf - lo) / (hi - lo) * 2048).floor().long(), 0, 2047)
    direct = torch.bincount(pos, minlength=2048).float()
    direct[0] += 1
    direct[-1] += 1
    # float32 bin arithmetic may move an element sitting on a boundary to the neighbouring bin
    assert (h.histogram - direct).abs().sum().item() <= 20


def test_merge_keeps_mass_and_range():
    torch.manual_seed(4)
    an = sq.SqnrAnalyzer()
    a, b = torch.randn(4000), torch.randn(6000) * 2.5 + 1
    an.update_stats(a)
    an.update_stats(b)
    st = an.stats[0]
    assert st.min == min(a.min(), b.min()) and st.max == max(a.max(), b.max())
    # re-binning rounds split bins, so the mass is preserved to within the number of source bins
    assert abs(st.histogram.sum().item() - 10000) <= 2048 * 0.5
    an.update_stats(a * 0.1)                       # inside the range: histogram simply accumulates
    assert an.stats[0].min == st.min and abs(an.stats[0].histogram.sum().item() - 14000) <= 1024


# ------------------------------------------------------------------------------------------ percentile calibration
def test_percentile_known_answers():
    # test_encoding_analyzer.py:562-595: 0..1000 in 500 bins, 99 % -> [0, 990]; symmetric with 254 steps -> +-990
    x = torch.arange(start=0, end=1001, step=1, dtype=torch.float)
    an = sq.PercentileAnalyzer(1, 500, 99)
    an.update_stats(x)
    lo, hi = an.compute_encodings(math.pow(2, 8) - 1, False)
    assert lo.item() == 0 and hi.item() == 990.0
    lo, hi = an.compute_encodings(math.pow(2, 8) - 2, True)
    assert lo.item() == -990.0 and hi.item() == 990.0


def test_percentile_100_is_the_observed_range_and_non_strict_symmetric_grid():
    # test_encoding_analyzer.py:596-622
    an = sq.PercentileAnalyzer(1, 1, 100)
    an.update_stats(torch.arange(start=-2, end=10, step=1, dtype=torch.float))
    lo, hi = an.compute_encodings(pow(2, 3) - 1, True)
    assert torch.isclose(lo, torch.tensor([-12.0])).all() and torch.isclose(hi, torch.tensor([9.0])).all()
    torch.manual_seed(0)
    x = torch.randn(10000) * 2 + 2
    an = sq.PercentileAnalyzer(1, 3, 100)
    an.update_stats(x)
    lo, hi = an.compute_encodings(254, True)
    assert torch.allclose(lo, -x.abs().max()) and torch.allclose(hi, x.abs().max())
    lo, hi = an.compute_encodings(255, False)
    assert torch.allclose(lo, x.min()) and torch.allclose(hi, x.max())


def test_percentile_50_and_outliers():
    # test_encoding_analyzer.py:624-655
    x = torch.arange(start=0, end=1001, step=1, dtype=torch.float)
    an = sq.PercentileAnalyzer(1, 3, 50)
    an.update_stats(x)
    st = an.stats[0]
    cum = torch.cumsum(st.histogram, dim=0)
    mid = st.bin_edges[torch.searchsorted(cum, torch.quantile(cum, 0.5))]
    lo, hi = an.compute_encodings(254, True)
    assert lo.item() == -mid.item() and hi.item() == mid.item()
    lo, hi = an.compute_encodings(255, False)
    assert lo.item() == 0 and hi.item() == mid.item()
    x = torch.arange(start=0, end=101, step=1, dtype=torch.float)
    x[-1], x[-2] = 1000, 800
    an = sq.PercentileAnalyzer(1, 2048, 90.0)
    an.update_stats(x)
    lo, hi = an.compute_encodings(255, False)
    assert 89 < hi.item() < 91


def test_adjust_min_max_widens_degenerate_ranges():
    eps = sq.MINIMUM_SCALE
    lo, hi = sq.adjust_min_max(torch.tensor([0.5, 0.0]), torch.tensor([2.0, 0.0]), 255, False)
    assert lo.tolist() == [0.0, 0.0] and hi[0] == 2.0 and hi[1].item() == pytest.approx(eps * 255)
    lo, hi = sq.adjust_min_max(torch.tensor([0.0]), torch.tensor([0.0]), 255, True)
    assert hi.item() == pytest.approx(127 * eps, rel=1e-6) and lo.item() == pytest.approx(-128 * eps, rel=1e-6)


# ------------------------------------------------------------- the reference's histogram-observer cases (golden)
def _run(an, batch):
    an.update_stats(torch.tensor(batch, dtype=torch.float32))
    return an.stats[0]


@pytest.mark.parametrize("name,num_bins,steps", __import__("_hist_cases").MERGE_CASES)
def test_histogram_merge_cases_of_the_reference(name, num_bins, steps):
    an = sq.SqnrAnalyzer(1, num_bins)
    for batch, mn, mx, hist, edges in steps:
        st = _run(an, batch)
        assert st.min.item() == pytest.approx(mn) and st.max.item() == pytest.approx(mx), name
        if hist is not None:
            assert st.histogram.tolist() == hist, name
            assert torch.allclose(st.bin_edges, torch.tensor(edges, dtype=torch.float32)), name


def test_infinite_inputs_are_clipped_to_the_finite_range():
    import _hist_cases as hc
    an = sq.SqnrAnalyzer(1, 10)
    for batch, mn, mx, bins, edges in hc.INF_CASE:
        st = _run(an, batch)
        assert st.min.item() == mn and st.max.item() == mx
        for b, count in bins.items():
            assert st.histogram[b].item() == count
        assert torch.allclose(st.bin_edges, torch.tensor(edges))
    old = an.stats[0].histogram.clone()
    st = _run(an, hc.INF_THIRD_BATCH)
    assert st.histogram[0] == old[0] + 2 and st.histogram[-1] == old[-1] + 1
    with pytest.raises(ValueError):
        sq.SqnrAnalyzer(1, 10).update_stats(torch.tensor([hc.INF, -hc.INF, -hc.INF, hc.INF, hc.INF]))
