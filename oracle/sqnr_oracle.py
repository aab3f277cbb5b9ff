"""CPU restatement of the reference's v2 histogram observer and SQNR encoding analyzer -- TEST INFRASTRUCTURE, never
imported by the product.

Plain torch ops on CPU tensors (torch.histc included: the arithmetic of this part of the reference lives in ATen, which
is installed here), following, statement for statement,
EA = TrainingExtensions/torch/src/python/aimet_torch/v2/quantization/encoding_analyzer.py:

  create_bin_edges / collect_histogram    EA:131-205  (_HistogramObserver.collect_stats, _handle_inputs, _create_bin_edges)
  merge_histogram                         EA:207-262  (_HistogramObserver.merge_stats, _get_bin_num)
  pick_test_candidates[_asymmetric|_symmetric], clamp_delta_offset_values     EA:594-660
  estimate_clip_and_quant_noise           EA:675-725
  select_best_candidates, compute_encodings_from_stats                        EA:566-592, 662-673
  adjust_min_max, percentile_encodings_from_stats                             EA:397-425, 486-519

Pinned by the reference's own tests (TrainingExtensions/torch/test/python/v2/quantization/test_encoding_analyzer.py:
657-881, restated in tests/test_oracle_sqnr.py): exact encodings of a uniform grid, the outlier construction, candidate
grids, clamping, estimated-vs-measured noise, best-candidate selection; the percentile part by :544-655 (sequential
data with known percentiles, 100 % = observed range, non-strict symmetric grid, outliers).
"""
import math
from typing import List, NamedTuple, Optional

import torch

MINIMUM_SCALE = torch.finfo(torch.float32).eps       # EA:322


class Histogram(NamedTuple):
    histogram: Optional[torch.Tensor] = None
    bin_edges: Optional[torch.Tensor] = None
    min: Optional[torch.Tensor] = None
    max: Optional[torch.Tensor] = None


def create_bin_edges(min_val, max_val, num_bins):
    if max_val == min_val:
        min_val = min_val - 0.5
        max_val = max_val + 0.5
    min_val, max_val = min_val.float(), max_val.float()
    step = (max_val - min_val) / num_bins
    return torch.arange(0, num_bins + 1) * step + min_val


def collect_histogram(hist_input: torch.Tensor, num_bins: int) -> Histogram:
    if not torch.any(hist_input.isfinite()):
        raise ValueError('Input tensor cannot contain only infinite or only NaN values')
    hist_min = hist_input[hist_input.isfinite()].min()
    hist_max = hist_input[hist_input.isfinite()].max()
    bin_edges = create_bin_edges(hist_min, hist_max, num_bins)
    histogram = torch.histc(hist_input.to(torch.float), bins=num_bins, min=bin_edges[0], max=bin_edges[-1])
    histogram[0] += torch.sum(hist_input < bin_edges[0])
    histogram[-1] += torch.sum(hist_input > bin_edges[-1])
    return Histogram(histogram, bin_edges, hist_min, hist_max)


def _get_bin_num(num_bins, bin_width, curr_min, data):
    bin_tensor = torch.full(data.shape, num_bins - 1)
    index_tensor = (data - curr_min) / bin_width
    return torch.minimum(index_tensor.to(torch.int32), bin_tensor)


def merge_histogram(curr_stats: Histogram, new_stats: Histogram, curr_input: torch.Tensor, num_bins: int) -> Histogram:
    """One histogram's share of _HistogramObserver.merge_stats; curr_input is the flattened batch."""
    if curr_stats.histogram is None:
        return new_stats
    updated_min = min(new_stats.min, curr_stats.min)
    updated_max = max(new_stats.max, curr_stats.max)
    if updated_min == curr_stats.min and updated_max == curr_stats.max:
        histogram_updates = curr_stats.histogram
    else:
        dest_bin_width = (updated_max - updated_min) / num_bins
        src_bin_width = (curr_stats.max - curr_stats.min) / num_bins
        histogram_updates = torch.zeros(num_bins)
        src_bin_start = curr_stats.min + (src_bin_width * torch.arange(0, num_bins))
        dest_bin_index = _get_bin_num(num_bins, dest_bin_width, updated_min, src_bin_start)
        dest_bin_end = updated_min + dest_bin_width * (dest_bin_index + 1)
        split_hist_value = torch.round(((dest_bin_end - src_bin_start) / src_bin_width) * curr_stats.histogram)
        dest_bin_updates = torch.minimum(split_hist_value, curr_stats.histogram)
        for i, dest_bin in enumerate(dest_bin_index):
            histogram_updates[dest_bin] += dest_bin_updates[i]
        other_bins = torch.nonzero(torch.where(dest_bin_updates < curr_stats.histogram, 1, 0))
        other_bin_index = _get_bin_num(num_bins, dest_bin_width, updated_min, src_bin_start + dest_bin_width)
        other_bin_updates = curr_stats.histogram - dest_bin_updates
        for bin_num in other_bins:
            histogram_updates[other_bin_index[bin_num]] += other_bin_updates[bin_num]
    expanded_histogram = torch.histc(curr_input.to(torch.float), bins=num_bins, min=updated_min, max=updated_max)
    expanded_histogram += histogram_updates
    expanded_histogram[0] += torch.sum(curr_input == -float('inf'))
    expanded_histogram[-1] += torch.sum(curr_input == float('inf'))
    expanded_bin_edges = create_bin_edges(updated_min, updated_max, num_bins)
    return Histogram(expanded_histogram, expanded_bin_edges, updated_min, updated_max)


def clamp_delta_offset_values(min_vals, max_vals, num_steps, test_deltas, test_offsets):
    test_min = test_deltas[:, :, None] * test_offsets[:, None, :]
    test_max = test_min + test_deltas[:, :, None] * num_steps
    test_min = torch.max(min_vals[:, None, None], test_min)
    test_max = torch.min(max_vals[:, None, None], test_max)
    test_deltas = (test_max - test_min) / num_steps
    min_delta = torch.Tensor([MINIMUM_SCALE]).to(dtype=test_deltas.dtype)
    test_deltas = torch.max(test_deltas, min_delta)
    test_offsets = torch.round(test_min / test_deltas)
    return test_deltas, test_offsets


def pick_test_candidates_asymmetric(min_vals, max_vals, num_steps, num_deltas=17, num_offset_candidates=21):
    kw = {"dtype": torch.float32}
    max_delta = (max_vals - min_vals).to(torch.float32) / num_steps
    observed_offset = torch.round(min_vals / max_delta)
    observed_min = max_delta * observed_offset
    observed_max = observed_min + max_delta * num_steps
    search_space = torch.arange(start=1, end=(1 + num_deltas), step=1, **kw)
    test_deltas = max_delta[:, None] * search_space[None, :] / (num_deltas - 1)
    num_offsets = min(num_steps + 2, num_offset_candidates)
    test_offset_step = num_steps / (num_offsets - 2)
    test_offsets = torch.round(torch.arange(start=-num_steps, end=test_offset_step, step=test_offset_step, **kw))
    test_offsets = test_offsets[None, :].expand(min_vals.shape[0], -1)
    test_offsets = torch.concat((test_offsets, observed_offset[:, None]), dim=1)
    return clamp_delta_offset_values(observed_min, observed_max, num_steps, test_deltas, test_offsets)


def pick_test_candidates_symmetric(min_vals, max_vals, num_steps, num_deltas=101):
    kw = {"dtype": torch.float32}
    max_delta = 2 * torch.max(max_vals, -min_vals).to(torch.float32) / num_steps
    test_offsets = torch.full((1,), (-num_steps) // 2, **kw)
    search_space = torch.arange(start=1, end=(1 + num_deltas), step=1, **kw)
    test_deltas = max_delta[:, None] * search_space[None, :] / (num_deltas - 1)
    min_delta = torch.Tensor([MINIMUM_SCALE]).to(**kw)
    test_deltas = torch.max(test_deltas, min_delta)
    return test_deltas[:, :, None], test_offsets[:, None, None]


def pick_test_candidates(stats: List[Histogram], num_steps, symmetric, **kw):
    min_vals = torch.stack([stat.min for stat in stats])
    max_vals = torch.stack([stat.max for stat in stats])
    min_vals = torch.min(min_vals, torch.zeros_like(min_vals))
    max_vals = torch.max(max_vals, torch.zeros_like(max_vals))
    max_vals = torch.max(max_vals, min_vals + MINIMUM_SCALE * num_steps)
    if symmetric:
        return pick_test_candidates_symmetric(min_vals, max_vals, num_steps,
                                              **{k: v for k, v in kw.items() if k == "num_deltas"})
    return pick_test_candidates_asymmetric(min_vals, max_vals, num_steps, **kw)


def estimate_clip_and_quant_noise(stats: List[Histogram], test_deltas, test_offsets, num_steps, gamma=1.0):
    kw = {"dtype": test_deltas.dtype}
    hists = torch.stack([stat.histogram for stat in stats])
    bin_edges = torch.stack([stat.bin_edges for stat in stats])
    hist_delta = bin_edges[:, 1] - bin_edges[:, 0]
    hist_offsets = hist_delta[:, None] * torch.arange(0, bin_edges.shape[1] - 1, **kw)[None, :]
    hist_midpoints = (bin_edges[:, 0] + hist_delta / 2)[:, None] + hist_offsets
    test_offsets_bcast = test_offsets[:, :, :, None]
    test_deltas_bcast = test_deltas[:, :, :, None]
    hist_midpoints_qdq = hist_midpoints[:, None, None, :].div(test_deltas_bcast).sub(test_offsets_bcast).round()
    if gamma != 1.0:
        clipped = torch.logical_or(hist_midpoints_qdq < 0, hist_midpoints_qdq > num_steps)
    hist_midpoints_qdq = hist_midpoints_qdq.clamp_(0, num_steps).add_(test_offsets_bcast).mul_(test_deltas_bcast)
    square_error = hist_midpoints_qdq.sub_(hist_midpoints[:, None, None, :]).pow_(2).mul_(hists[:, None, None, :])
    if gamma != 1.0:
        square_error = torch.where(clipped, square_error * gamma, square_error)
    return torch.sum(square_error, dim=-1)


def select_best_candidates(test_deltas, test_offsets, stats, num_steps, gamma):
    noise = estimate_clip_and_quant_noise(stats, test_deltas, test_offsets, num_steps, gamma)
    _, min_idx = torch.min(noise.flatten(start_dim=1), dim=1)
    best_delta = torch.gather(test_deltas.flatten(start_dim=1), dim=1, index=min_idx[:, None])
    if test_offsets.numel() == 1:
        best_offset = test_offsets
    else:
        best_offset = torch.gather(test_offsets.flatten(start_dim=1), dim=1, index=min_idx[:, None])
    return best_delta, best_offset, noise


def compute_encodings_from_stats(stats: List[Histogram], num_steps, is_symmetric, gamma=3.0, shape=None, **kw):
    """Returns (min, max, noise) with noise of shape (num_histograms, num_candidates)."""
    if stats[0].histogram is None:
        raise RuntimeError('No statistics present to compute encodings.')
    if num_steps <= 0:
        raise ValueError('The number of quantization bins cannot be less than or equal to 0.')
    test_deltas, test_offsets = pick_test_candidates(stats, num_steps, is_symmetric, **kw)
    best_delta, best_offset, noise = select_best_candidates(test_deltas, test_offsets, stats, num_steps, gamma)
    min_enc = best_offset * best_delta
    max_enc = min_enc + num_steps * best_delta
    min_enc = min_enc.to(stats[0].min.dtype)
    max_enc = max_enc.to(stats[0].max.dtype)
    shape = shape if shape is not None else (len(stats),)
    return min_enc.view(shape), max_enc.view(shape), noise.flatten(start_dim=1)


class SqnrAnalyzer:
    """Per-tensor or per-row (shape (C, 1) on [C, N] inputs) analyzer assembled from the functions above."""

    def __init__(self, num_histograms=1, num_bins=2048, gamma=3.0):
        self.num_histograms, self.num_bins, self.gamma = num_histograms, num_bins, gamma
        self.stats = [Histogram() for _ in range(num_histograms)]

    def update_stats(self, x: torch.Tensor):
        rows = x.reshape(self.num_histograms, -1)
        new = [collect_histogram(rows[i], self.num_bins) for i in range(self.num_histograms)]
        self.stats = [merge_histogram(self.stats[i], new[i], rows[i], self.num_bins)
                      for i in range(self.num_histograms)]
        return new

    def compute_encodings(self, num_steps, is_symmetric):
        return compute_encodings_from_stats(self.stats, num_steps, is_symmetric, self.gamma)


# ------------------------------------------------------------------------------------------ percentile calibration
def adjust_min_max(curr_min, curr_max, num_steps, is_symmetric):
    """EA:397-425: the range is widened to contain zero, kept finite and at least MINIMUM_SCALE * num_steps wide; a
    symmetric grid takes the larger of the two half ranges."""
    curr_min = torch.minimum(curr_min, torch.zeros_like(curr_min)).clone()
    curr_max = torch.maximum(curr_max, torch.zeros_like(curr_max)).clone()
    curr_min = curr_min.clamp(min=torch.finfo(curr_max.dtype).min, max=0)
    curr_max = curr_max.clamp(min=0, max=torch.finfo(curr_max.dtype).max)
    too_close = (curr_max - curr_min) / num_steps < MINIMUM_SCALE
    if is_symmetric:
        curr_min = torch.where(too_close, curr_min - MINIMUM_SCALE * math.ceil(num_steps / 2), curr_min)
        curr_max = torch.where(too_close, curr_max + MINIMUM_SCALE * math.floor(num_steps / 2), curr_max)
        num_pos_steps, num_neg_steps = math.floor(num_steps / 2), math.ceil(num_steps / 2)
        delta = torch.maximum(curr_max / num_pos_steps, -curr_min / num_neg_steps)
        curr_min, curr_max = -num_neg_steps * delta, num_pos_steps * delta
    else:
        curr_max = torch.where(too_close, curr_max + MINIMUM_SCALE * num_steps, curr_max)
    return curr_min, curr_max


def percentile_encodings_from_stats(stats: List[Histogram], percentile: float, num_steps, is_symmetric):
    """EA:486-519 (PercentileEncodingAnalyzer.compute_encodings_from_stats): per histogram, the bin edges at which the
    cumulative count reaches (100 - p) % and p % of the total, then adjust_min_max."""
    mins, maxs = [], []
    for h in stats:
        cum_sum = torch.cumsum(h.histogram, dim=0)
        max_index = torch.searchsorted(cum_sum, cum_sum[-1] * percentile / 100)
        min_index = torch.searchsorted(cum_sum, cum_sum[-1] * (1 - percentile / 100))
        if percentile == 100:
            min_index, max_index = 0, -1
        lo, hi = adjust_min_max(h.bin_edges[min_index], h.bin_edges[max_index], num_steps, is_symmetric)
        mins.append(lo)
        maxs.append(hi)
    return torch.stack(mins), torch.stack(maxs)


class PercentileAnalyzer(SqnrAnalyzer):
    def __init__(self, num_histograms=1, num_bins=2048, percentile=100.0):
        super().__init__(num_histograms, num_bins)
        self.percentile = percentile

    def compute_encodings(self, num_steps, is_symmetric):
        return percentile_encodings_from_stats(self.stats, self.percentile, num_steps, is_symmetric)
