"""Data of the reference's histogram-observer tests (TrainingExtensions/torch/test/python/v2/quantization/
test_encoding_analyzer.py:286-540): sequences of batches with the running min, max, histogram and bin edges expected
after each batch.  Used against the CPU restatement and against the GPU observer."""
INF = float("inf")

# name, num_bins, [(batch, min, max, histogram or None, bin_edges or None), ...]
MERGE_CASES = [
    ("resize_histogram", 3, [                                                          # :286-313
        ([2.0, 3.5, 4.2, 5.0], 2, 5, [1, 1, 2], [2.0, 3.0, 4.0, 5.0]),
        ([5.3, 6.4, 7.0, 8.0], 2, 8, [2, 3, 3], [2.0, 4.0, 6.0, 8.0]),
        ([-4.2, 0, 2.3, 4.5], -4.2, 8, [1, 4, 7], [-4.2, -0.133333, 3.933333, 8.0]),
    ]),
    ("ambiguous_bins", 3, [                                                            # :315-336
        ([-4.2, 2.4, 7.0, 8.0], -4.2, 8, [1, 1, 2], [-4.2, -0.133333, 3.933333, 8.0]),
        ([-6.7, -2.5, 7.2, 10.3], -6.7, 10.3, [3, 1, 4], [-6.7, -1.03333, 4.63333, 10.3]),
    ]),
    ("bin_splitting", 3, [                                                             # :338-356
        ([1, 7, 5.3, 6, 5.7, 6.8, 6.2, 2.8, 3.9], 1, 7, [2, 1, 6], [1, 3, 5, 7]),
        ([0, 9, 7.8, 2.5, 4.6, 6.2, 8.8], 0, 9, [4, 5, 7], [0, 3, 6, 9]),
    ]),
    ("one_bin", 1, [                                                                   # :358-364
        ([1, 7, 5.3, 6, 5.7, 6.8, 6.2, 2.8, 3.9], 1, 7, None, None),
    ]),
    ("without_resizing", 3, [                                                          # :404-432
        ([2.0, 3.5, 4.2, 5.0], 2, 5, [1, 1, 2], [2, 3, 4, 5]),
        ([2.0, 3.3, 4.8, 5], 2, 5, [2, 2, 4], [2, 3, 4, 5]),
        ([3.1, 3.3, 3.7, 3.9], 2, 5, [2, 6, 4], [2, 3, 4, 5]),
    ]),
    ("during_merging", 10, [                                                           # :514-540
        ([float(v) for v in range(-50, 51)], -50, 50, None, None),
        ([float(v) * 1.5 for v in range(-50, 51)], -75, 75, [10, 15, 25, 25, 25, 25, 25, 26, 15, 11],
         [-75, -60, -45, -30, -15, 0, 15, 30, 45, 60, 75]),
    ]),
]

# infinities are clipped to the finite range of their batch (:366-395); (batch, min, max, {bin: count})
INF_CASE = [
    ([1, 7, 5.3, 6, INF, INF], 1, 7, {9: 3},
     [1.0, 1.6, 2.2, 2.8, 3.4, 4.0, 4.6, 5.2, 5.8, 6.4, 7.0]),
    ([0, 17, -5, 3, -INF, INF, -INF], -5, 17, {9: 2, 0: 3},
     [-5.0, -2.8, -0.6, 1.6, 3.8, 6.0, 8.2, 10.4, 12.6, 14.8, 17.0]),
]
INF_THIRD_BATCH = [10, -INF, INF, -INF]          # adds 2 to the first bin and 1 to the last
