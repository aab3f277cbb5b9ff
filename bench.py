#!/usr/bin/env python3
"""Benchmark of the quantization-simulation hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--full]

A "step" is one quantize-dequantize forward + straight-through backward pass over one weight tensor of the
per-output-channel symmetric int8 configuration ([11008, 4096] fp32, Laplace(0, 0.02) with 0.1 % outliers x20).
Inputs are resident in HBM before the timed region; three distinct buffer sets are rotated so that the 256 MB
last-level cache cannot serve the traffic.  One JSON line is printed:

  value            whole-job algorithmic GB/s of fwd+bwd (20 B/element: fwd reads x, writes y; bwd reads x and g,
                   writes gx) over the K timed steps
  roofline         the dominant kernel (backward, 12 B/element): mean duration of K back-to-back launches bracketed
                   by a HIP event pair on the launching stream, against the 8 TB/s HBM peak
  cpu_baseline     the single-threaded C restatement of the reference's CPU loops (oracle/), timed on this host on a
                   bounded sample of the same workload
  extra            the other cells of the measurement matrix (per-tensor activation QDQ, the weight shapes x dtypes x
                   bit-widths, TF-Enhanced calibration elements/s) measured the same way, fewer repetitions
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0

# HBM bytes per launch at the main shape, from hardware counters (two rocprofv3 --pmc runs, FETCH_SIZE and WRITE_SIZE,
# each scaled by what the same counter reads for a plain elementwise kernel of known traffic: x2.000 and x1.000).
# The counter runs are separate from this program; these are their results for [11008,4096] fp32.
MEASURED_TRAFFIC_BYTES = {"ste_bwd_per_channel_f32": 542.47e6, "qdq_fwd_per_channel_f32": 363.65e6,
                          "qdq_mask_fwd_per_channel_f32": 372.08e6, "ste_mask_bwd_f32": 372.07e6}


def _laplace_weights(torch, shape, seed, device):
    g = torch.Generator(device=device).manual_seed(seed)
    u = torch.rand(shape, device=device, generator=g) - 0.5
    w = -0.02 * torch.sign(u) * torch.log1p(-2 * u.abs())
    out = torch.rand(shape, device=device, generator=g) < 0.001
    return torch.where(out, w * 20, w).contiguous()


def _sym_channel_params(torch, ops, w, c, npc, bw):
    """Per-output-channel symmetric TF (min/max) encodings -> the v1 per-channel kernel parameters."""
    mm = ops.minmax_per_channel(w.float(), c, npc).cpu().double()
    emin, emax = torch.empty(c), torch.empty(c)
    for i in range(c):
        lo, hi = min(0.0, float(mm[0, i])), max(0.0, float(mm[1, i]))
        hi = max(hi, lo + 0.01)
        e = ops.get_computed_encodings(bw, lo, hi, True, False, False)
        emin[i], emax[i] = e.min, e.max
    steps = 2 ** bw - 1 - (1 if float(emin[0]) == -float(emax[0]) else 0)
    return ops.per_channel_params(emin.to(w.device), emax.to(w.device), steps), emin.to(w.device), emax.to(w.device)


def _time_fwd_bwd(torch, fwd, bwd, sets, steps, warmup):
    """Runs warmup + steps fwd+bwd passes, rotating buffer sets; returns (wall ms/step, mean fwd ms, mean bwd ms).

    The step time is wall-clock over exactly `steps` passes between two synchronisations (one HIP event pair around
    the same region cross-checks it).  The per-kernel durations come from two more regions of `steps` back-to-back
    launches of that kernel alone, each bracketed by a HIP event pair on the launching stream: events between every
    pair of launches would put a ~5 us bubble after each kernel and distort both numbers.
    """
    for i in range(warmup):
        s = sets[i % len(sets)]
        fwd(s)
        bwd(s)
    e = [torch.cuda.Event(enable_timing=True) for _ in range(6)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    e[0].record()
    for i in range(steps):
        s = sets[i % len(sets)]
        fwd(s)
        bwd(s)
    e[1].record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    assert e[0].elapsed_time(e[1]) / steps <= wall_ms * 1.001
    e[2].record()
    for i in range(steps):
        fwd(sets[i % len(sets)])
    e[3].record()
    e[4].record()
    for i in range(steps):
        bwd(sets[i % len(sets)])
    e[5].record()
    torch.cuda.synchronize()
    return wall_ms, e[2].elapsed_time(e[3]) / steps, e[4].elapsed_time(e[5]) / steps


def _graph_replay_ms(torch, fn, sets, launches):
    """Mean duration of `launches` back-to-back launches of fn (rotating the buffer sets) replayed from a HIP graph:
    the kernels as the GPU runs them when the host is not what paces them.  For tensors of a few MB the Python and
    launch cost of a call (6 to 8 us) exceeds the kernel's duration, and the eager figures measure the host."""
    try:
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for i in range(3):
                fn(sets[i % len(sets)])
        torch.cuda.current_stream().wait_stream(side)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            for i in range(launches):
                fn(sets[i % len(sets)])
        graph.replay()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        graph.replay()
        e1.record()
        torch.cuda.synchronize()
        ms = e0.elapsed_time(e1) / launches
        del graph
        return ms
    except RuntimeError:
        return None


def _saved_mask_figures(wall, f, b, n, esz):
    """Bytes the saved-mask step moves: forward reads x, writes y and n / 8 bytes of mask; backward reads the
    gradient and the mask, writes the input gradient.  GB/s on those bytes; and what the same time would be worth on
    the 5-accesses-per-element formulation the other figures use."""
    fwd_bytes, bwd_bytes = 2 * esz * n + n / 8, 2 * esz * n + n / 8
    return {"ms_per_step": wall, "fwd_ms": f, "bwd_ms": b, "bytes_moved_per_step": fwd_bytes + bwd_bytes,
            "fwd_GBps_moved": fwd_bytes / f / 1e6, "bwd_GBps_moved": bwd_bytes / b / 1e6,
            "fwd_bwd_GBps_moved": (fwd_bytes + bwd_bytes) / wall / 1e6,
            "frac_hbm_moved": (fwd_bytes + bwd_bytes) / wall / 1e6 / HBM_PEAK_GBPS,
            "fwd_bwd_GBps_on_recompute_formulation": 5 * esz * n / wall / 1e6}


def bench_per_channel(torch, ops, shape, dtype, bw, steps, warmup, seed, nsets=3):
    dev = torch.device("cuda", 0)
    c, npc = shape[0], 1
    for d in shape[1:]:
        npc *= d
    n = c * npc
    esz = 4 if dtype == torch.float32 else 2
    # enough distinct sets that one rotation moves well over 256 MB
    while nsets * n * esz * 5 < 1.5e9 and nsets < 64:
        nsets += 1
    sets = []
    w0 = _laplace_weights(torch, shape, seed, dev)
    (mn, mx, delta, offset), emin, emax = _sym_channel_params(torch, ops, w0, c, npc, bw)
    for k in range(nsets):
        w = (w0 if k == 0 else _laplace_weights(torch, shape, seed + 97 * k, dev)).to(dtype)
        g = torch.randn(shape, device=dev, generator=torch.Generator(device=dev).manual_seed(seed + 100 + k)).to(dtype)
        sets.append((w, g, torch.empty_like(w), torch.empty_like(w)))

    def fwd(s):
        ops.qdq_per_channel(s[0], c, npc, mn, mx, delta, offset, out=s[2])

    def bwd(s):
        ops.ste_bwd_per_channel(s[0], s[1], c, npc, emin, emax, out=s[3])

    if n < 8e6:
        steps = max(steps, 100)                 # microsecond kernels: more launches per region
    wall, f, b = _time_fwd_bwd(torch, fwd, bwd, sets, steps, warmup)
    out = {"shape": list(shape), "dtype": "fp32" if esz == 4 else "bf16", "bw": bw, "elements": n,
           "ms_per_step": wall, "fwd_ms": f, "bwd_ms": b,
           "fwd_GBps": 2 * esz * n / f / 1e6, "bwd_GBps": 3 * esz * n / b / 1e6,
           "fwd_bwd_GBps": 5 * esz * n / wall / 1e6, "buffer_sets": nsets}
    # the same step with the straight-through mask saved by the forward, one bit per element, and read by the
    # backward instead of x
    masks = [ops._new_mask(s[0]) for s in sets]                      # pylint: disable=protected-access

    def fwd_m(s):
        ops.qdq_mask_per_channel(s[0], c, npc, mn, mx, delta, offset, emin, emax, out=s[2], mask=s[4])

    def bwd_m(s):
        ops.ste_bwd_mask(s[4], s[1], out=s[3])

    msets = [s + (m,) for s, m in zip(sets, masks)]
    out["saved_mask"] = _saved_mask_figures(*_time_fwd_bwd(torch, fwd_m, bwd_m, msets, steps, warmup), n, esz)
    if n < 2e7:
        # host-paced above; the same launches replayed from a HIP graph
        gf = _graph_replay_ms(torch, fwd, sets, min(64, 4 * nsets))
        gb = _graph_replay_ms(torch, bwd, sets, min(64, 4 * nsets))
        if gf and gb:
            out["graph_replay"] = {"fwd_ms": gf, "bwd_ms": gb, "fwd_GBps": 2 * esz * n / gf / 1e6,
                                   "bwd_GBps": 3 * esz * n / gb / 1e6,
                                   "fwd_bwd_GBps": 5 * esz * n / (gf + gb) / 1e6,
                                   "frac_hbm": 5 * esz * n / (gf + gb) / 1e6 / HBM_PEAK_GBPS}
    return out


def bench_fp8(torch, ops, steps, warmup):
    """8-bit float simulation (fake cast to the E4M3-shaped grid scaled to maxval) of the main weight shape, per
    output channel, and of the activation shape, per tensor: forward only (its gradient is a pass-through)."""
    dev = torch.device("cuda", 0)
    out = {}
    for name, shape, per_channel in (("per_channel_11008x4096", (11008, 4096), True),
                                     ("per_tensor_32x64x56x56", (32, 64, 56, 56), False)):
        n = 1
        for d in shape:
            n *= d
        nsets = max(3, int(1.2e9 // (8 * n)))
        sets = []
        for k in range(nsets):
            x = torch.randn(shape, device=dev, generator=torch.Generator(device=dev).manual_seed(1201 + k))
            sets.append((x, torch.empty_like(x)))
        maxval = sets[0][0].abs().amax(dim=1) if per_channel else sets[0][0].abs().max()
        grid = ops.fp8_grid(maxval)                 # as the tensor quantizer holds it between calls
        ev = [torch.cuda.Event(enable_timing=True) for _ in range(2)]
        for i in range(warmup):
            ops.fp8_fake_cast(sets[i % nsets][0], None, out=sets[i % nsets][1], grid=grid)
        torch.cuda.synchronize()
        ev[0].record()
        for i in range(steps):
            ops.fp8_fake_cast(sets[i % nsets][0], None, out=sets[i % nsets][1], grid=grid)
        ev[1].record()
        torch.cuda.synchronize()
        ms = ev[0].elapsed_time(ev[1]) / steps
        out[name] = {"elements": n, "ms_per_call": ms, "GBps": 8 * n / ms / 1e6,
                     "frac_hbm": 8 * n / ms / 1e6 / HBM_PEAK_GBPS, "buffer_sets": nsets}
    return out


def bench_per_tensor(torch, ops, steps, warmup):
    dev = torch.device("cuda", 0)
    shape = (32, 64, 56, 56)
    n = 32 * 64 * 56 * 56
    nsets = 16                                  # 16 x 4 x 25.7 MB = 1.6 GB rotated
    sets = []
    for k in range(nsets):
        x = torch.randn(shape, device=dev, generator=torch.Generator(device=dev).manual_seed(1001 + k))
        g = torch.randn(shape, device=dev, generator=torch.Generator(device=dev).manual_seed(1101 + k))
        sets.append((x, g, torch.empty_like(x), torch.empty_like(x)))
    mm = ops.minmax(sets[0][0]).cpu()
    lo, hi = min(0.0, float(mm[0])), max(0.0, float(mm[1]))
    e = ops.get_computed_encodings(8, lo, max(hi, lo + 0.01), False, False, False)

    def fwd(s):
        ops.qdq_per_tensor(s[0], e.min, e.max, 8, out=s[2])

    def bwd(s):
        ops.ste_bwd_per_tensor(s[0], s[1], e.min, e.max, out=s[3])

    wall, f, b = _time_fwd_bwd(torch, fwd, bwd, sets, max(steps, 100), warmup)
    out = {"shape": list(shape), "dtype": "fp32", "bw": 8, "elements": n, "ms_per_step": wall, "fwd_ms": f,
           "bwd_ms": b, "fwd_GBps": 8 * n / f / 1e6, "bwd_GBps": 12 * n / b / 1e6,
           "fwd_bwd_GBps": 20 * n / wall / 1e6, "frac_hbm": 20 * n / wall / 1e6 / HBM_PEAK_GBPS, "buffer_sets": nsets}
    gf, gb = _graph_replay_ms(torch, fwd, sets, 64), _graph_replay_ms(torch, bwd, sets, 64)
    if gf and gb:
        out["graph_replay"] = {"fwd_ms": gf, "bwd_ms": gb, "fwd_bwd_GBps": 20 * n / (gf + gb) / 1e6,
                               "frac_hbm": 20 * n / (gf + gb) / 1e6 / HBM_PEAK_GBPS}
    # the same step with the straight-through mask saved by the forward (one bit per element)
    msets = [s + (ops._new_mask(s[0]),) for s in sets]              # pylint: disable=protected-access

    def fwd_m(s):
        ops.qdq_mask_per_tensor(s[0], e.min, e.max, 8, out=s[2], mask=s[4])

    def bwd_m(s):
        ops.ste_bwd_mask(s[4], s[1], out=s[3])

    out["saved_mask"] = _saved_mask_figures(*_time_fwd_bwd(torch, fwd_m, bwd_m, msets, max(steps, 100), warmup), n, 4)
    gf, gb = _graph_replay_ms(torch, fwd_m, msets, 64), _graph_replay_ms(torch, bwd_m, msets, 64)
    if gf and gb:
        out["saved_mask"]["graph_replay"] = {"fwd_ms": gf, "bwd_ms": gb, "ms_per_step": gf + gb}
    # the same region with one buffer set: 103 MB of operands, served by the 256 MB last-level cache
    one = sets[:1]
    wall1, f1, b1 = _time_fwd_bwd(torch, fwd, bwd, one, max(steps, 100), warmup)
    out["same_buffer_cache_resident"] = {"ms_per_step": wall1, "fwd_ms": f1, "bwd_ms": b1,
                                         "fwd_bwd_GBps": 20 * n / wall1 / 1e6}
    return out


def bench_calibration(torch, ops, reps):
    """TF-Enhanced calibration: 16 batches of [32,256,28,28] post-ReLU-like fp32, then the 8-bit asymmetric search."""
    dev = torch.device("cuda", 0)
    n = 32 * 256 * 28 * 28
    batches = []
    for b in range(16):
        g = torch.Generator(device=dev).manual_seed(1003 + b)
        x = torch.randn(n, device=dev, generator=g).abs_()
        u = torch.rand(n, device=dev, generator=g)
        t = torch.rand(n, device=dev, generator=g)
        batches.append(torch.where(u < 0.005, (1 - t).rsqrt(), x).contiguous())
    an = ops.Analyzer(1, dev)
    acc_ms, search_ms, total_ms = [], [], []
    for r in range(reps + 1):
        an.reset()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t0 = time.perf_counter()
        e0.record()
        for x in batches:
            an.update_stats(x)
        e1.record()
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        enc, valid = an.compute_encoding(8)
        t2 = time.perf_counter()
        if r == 0:
            continue                              # first repetition warms up
        acc_ms.append(e0.elapsed_time(e1))
        search_ms.append((t2 - t1) * 1e3)
        total_ms.append((t2 - t0) * 1e3)
    acc = sum(acc_ms) / len(acc_ms)
    tot = sum(total_ms) / len(total_ms)
    elems = 16 * n
    # the same accumulation when the calibration batches are larger (one update call = one launch: the launch's fixed
    # cost is what keeps the 25.7 MB batches of the configuration below the kernel's streaming rate).  Two rows per
    # size: distinct buffers rotated so that every read comes from HBM, and one buffer read over and over, which at
    # 25.7 and 103 MB is served by the 256 MB last-level cache and is labelled so.
    by_size = {}
    for mult in (1, 4, 8):
        nrot = max(2, 16 // mult)
        bigs = [torch.cat(batches[k * mult:(k + 1) * mult]) if mult > 1 else batches[k] for k in range(nrot)]
        for label, pick in (("rotated_hbm", lambda i: bigs[i % nrot]), ("same_buffer_cache_resident", lambda i: bigs[0])):
            an.reset()
            an.update_stats(pick(0))
            an.update_stats(pick(1))
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            reps = 16
            e0.record()
            for i in range(reps):
                an.update_stats(pick(i))
            e1.record()
            torch.cuda.synchronize()
            ms = e0.elapsed_time(e1) / reps
            by_size.setdefault(f"{mult}x[32,256,28,28]", {})[label] = {
                "update_us": ms * 1e3, "GBps": 4 * n * mult / ms / 1e6,
                "frac_hbm": 4 * n * mult / ms / 1e6 / HBM_PEAK_GBPS}
        del bigs
    # the other searches on the same PDF: percentile (host arithmetic on the buckets read back) and least squared error
    # over pairs of bucket edges (three launches, one lane per pair); wall time of compute_encoding, statistics in place
    other_searches = {}
    for name, mode in (("percentile_99.9", 2), ("mse", 3)):
        other = ops.Analyzer(mode, dev)
        if mode == 2:
            other.set_percentile(99.9)
        for x in batches[:4]:
            other.update_stats(x)
        for bw in (8, 4):
            other.compute_encoding(bw)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(10):
                e, _ = other.compute_encoding(bw)
            other_searches[f"{name}_bw{bw}"] = {"compute_encoding_us": (time.perf_counter() - t0) / 10 * 1e6,
                                                "encoding": [e.min, e.max, e.delta, e.offset]}
        del other
    # the entropy analyzer keeps a histogram of another kind (it follows the range of the data): two streaming passes
    # and one small launch per batch, the KL window search on the host
    ent = ops.Analyzer(4, dev)
    for x in batches[:2]:
        ent.update_stats(x)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for x in batches:
        ent.update_stats(x)
    e1.record()
    torch.cuda.synchronize()
    ent_update_ms = e0.elapsed_time(e1) / len(batches)
    ent.compute_encoding(8)
    t0 = time.perf_counter()
    for _ in range(10):
        e, _ = ent.compute_encoding(8)
    entropy = {"update_us": ent_update_ms * 1e3, "update_GBps_of_one_read": 4 * n / ent_update_ms / 1e6,
               "compute_encoding_us": (time.perf_counter() - t0) / 10 * 1e6,
               "encoding": [e.min, e.max, e.delta, e.offset]}
    del ent
    return {"elements": elems, "accumulate_ms": acc, "search_ms_wall": sum(search_ms) / len(search_ms),
            "update_by_batch_size": by_size, "other_searches_on_the_same_pdf": other_searches,
            "entropy_analyzer": entropy,
            "total_ms_wall": tot, "elements_per_s": elems / (tot / 1e3),
            "accumulate_GBps": 17 * 4 * n / acc / 1e6, "accumulate_frac_hbm": 17 * 4 * n / acc / 1e6 / HBM_PEAK_GBPS,
            "encoding": [enc.min, enc.max, enc.delta, enc.offset]}


def bench_seq_mse(torch, ops):
    """Sequential MSE's search on one Linear [4096, 4096] layer (4 bits, 20 candidates, 4 batches of [512, 4096]
    inputs) over the v1 wrappers (per channel) and the v2 quantized modules (per channel, and blocks of 128 input
    channels), beside the GEMMs alone; and the loss kernel on the blockwise search's [32, 512, 4096] products."""
    from aimet_amd.common.defs import QuantScheme
    from aimet_amd.v1.qc_quantize_op import StaticGridQuantWrapper
    from aimet_amd.v1.seq_mse import SeqMseParams, optimize_module
    from aimet_amd.v2 import seq_mse as v2
    from aimet_amd.v2.nn import QuantizationMixin
    from aimet_amd.v2.quantization.affine import QuantizeDequantize
    dev = torch.device("cuda", 0)
    torch.manual_seed(1006)
    layer = torch.nn.Linear(4096, 4096).to(dev)
    x = torch.randn(4, 512, 4096, device=dev)
    params = SeqMseParams(num_batches=4)

    def v1_search():
        wrapper = StaticGridQuantWrapper(layer, 4, 16, 'nearest', QuantScheme.post_training_tf)
        wrapper.enable_per_channel_quantization()
        quantizer = wrapper.param_quantizers['weight']
        quantizer.update_encoding_stats(layer.weight.data)
        quantizer.compute_encoding()
        return lambda: optimize_module(wrapper, x, x, params)

    def v2_search(shape, block_size):
        qmodule = QuantizationMixin.from_module(layer)
        qmodule.param_quantizers['weight'] = quantizer = QuantizeDequantize(shape, 4, True,
                                                                            block_size=block_size).to(dev)
        with quantizer.compute_encodings():
            quantizer(qmodule.weight.data)
        return lambda: v2.optimize_module(qmodule, x, x, params)

    def wall_ms(make):
        make()()                                  # warm-up on a quantizer of its own: a search freezes its quantizer
        search = make()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        search()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) * 1e3

    out = {"layer": [4096, 4096], "inputs": [4, 512, 4096], "candidates": 20, "bitwidth": 4,
           "v1_per_channel_ms": wall_ms(v1_search),
           "v2_per_channel_ms": wall_ms(lambda: v2_search([4096, 1], None)),
           "v2_blocks_of_128_ms": wall_ms(lambda: v2_search([4096, 32], [-1, -1]))}
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(84):
        torch.nn.functional.linear(x[0], layer.weight)
    torch.cuda.synchronize()
    out["the_84_gemms_alone_ms"] = (time.perf_counter() - t0) * 1e3
    a, b = torch.randn(32, 512, 4096, device=dev), torch.randn(32, 512, 4096, device=dev)
    for kind, name in ((ops.COLUMN_ERROR_SQUARED, "squared"), (ops.COLUMN_ERROR_SQUARED_AND_SIGNAL, "squared_and_signal")):
        ops.column_error(a, b, kind)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(10):
            ops.column_error(a, b, kind)
        e1.record()
        torch.cuda.synchronize()
        ms = e0.elapsed_time(e1) / 10
        out[f"column_error_{name}_32x512x4096"] = {"ms": ms, "GBps": 2 * a.numel() * 4 / ms / 1e6,
                                                   "frac_hbm": 2 * a.numel() * 4 / ms / 1e6 / HBM_PEAK_GBPS}
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(10):
        (a - b).square_().sum(1)
    torch.cuda.synchronize()
    out["the_same_loss_by_tensor_operations_ms"] = (time.perf_counter() - t0) * 1e3 / 10
    return out


def _adaround_layer(torch, seed=1005, out_features=4096, in_features=4096, rows=2048):
    """cfg5 objects: Linear [4096,4096] fp32, W ~ N(0, 0.02); X [2048,4096] ~ N(0,1); Y = X W^T; 4-bit per-channel."""
    from aimet_amd.common.defs import QuantScheme
    from aimet_amd.v1.adaround.adaround_wrapper import AdaroundWrapper
    from aimet_amd.v1.qc_quantize_op import StaticGridQuantWrapper
    dev = torch.device("cuda", 0)
    g = torch.Generator(device=dev).manual_seed(seed)
    lin = torch.nn.Linear(in_features, out_features, bias=False).to(dev)
    lin.weight.data = torch.randn(out_features, in_features, device=dev, generator=g) * 0.02
    x = torch.randn(rows, in_features, device=dev, generator=g)
    y = torch.nn.functional.linear(x, lin.weight.data)
    qw = StaticGridQuantWrapper(lin, 4, 8, round_mode='nearest', quant_scheme=QuantScheme.post_training_tf,
                                is_symmetric=True)
    qw.enable_per_channel_quantization()
    q = qw.param_quantizers['weight']
    q.update_encoding_stats(lin.weight.data)
    q.compute_encoding()
    return AdaroundWrapper(qw), x, y


def bench_launch_floors(torch, ops, launches=200):
    """What launches of the benchmark's tensor sizes cost on this GPU whatever the kernel computes: back-to-back launches
    of the simplest kernels of the same traffic (torch's elementwise add with a scalar for 1-read-1-write, with a tensor
    for 2-read-1-write), rotated over several buffer sets, one event pair around the region.  The fractions
    of HBM peak that the per-tensor cell and the calibration loop are held against come from here."""
    dev = torch.device("cuda", 0)
    out = {}
    for name, n in (("32x64x56x56", 32 * 64 * 56 * 56), ("11008x4096", 11008 * 4096)):
        sets = 16 if n < (1 << 24) else 3
        a = [torch.randn(n, device=dev) for _ in range(sets)]
        b = [torch.randn(n, device=dev) for _ in range(sets)]
        c = [torch.empty(n, device=dev) for _ in range(sets)]
        kinds = {
            "one_read_one_write": (8, lambda i: torch.add(a[i % sets], 1.0, out=c[i % sets])),
            "two_reads_one_write": (12, lambda i: torch.add(a[i % sets], b[i % sets], out=c[i % sets])),
        }
        row = {}
        for kind, (bytes_per_elem, fn) in kinds.items():
            for i in range(5):
                fn(i)
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            torch.cuda.synchronize()
            e0.record()
            for i in range(launches):
                fn(i)
            e1.record()
            torch.cuda.synchronize()
            us = e0.elapsed_time(e1) / launches * 1e3
            row[kind] = {"us_per_launch": us, "GBps": bytes_per_elem * n / us / 1e3,
                         "frac_hbm": bytes_per_elem * n / us / 1e3 / HBM_PEAK_GBPS}
        row["fwd_plus_bwd_floor_us"] = row["one_read_one_write"]["us_per_launch"] + row["two_reads_one_write"]["us_per_launch"]
        row["fwd_plus_bwd_floor_frac_hbm"] = 20 * n / row["fwd_plus_bwd_floor_us"] / 1e3 / HBM_PEAK_GBPS
        out[name] = row
        del a, b, c
    return out


def bench_adaround(torch, ops, iterations, timed_kernel_iters=50):
    """AdaRound inner loop of one Linear [4096,4096] layer (cfg5): whole loop wall-clock through AdaroundOptimizer, then
    the three kernels of one iteration timed with events."""
    from aimet_amd.v1.adaround.adaround_loss import AdaroundHyperParameters
    from aimet_amd.v1.adaround.adaround_optimizer import AdaroundOptimizer
    wrapper, x, y = _adaround_layer(torch)
    timed_kernel_iters = min(timed_kernel_iters, iterations)
    n = wrapper.weight.numel()
    o, k = wrapper.weight.shape
    params = AdaroundHyperParameters(iterations, 0.01, (20, 2), 0.2)
    torch.manual_seed(1005)
    batches = [torch.randperm(x.size(0))[:32] for _ in range(iterations)]
    res = {"layer": [o, k], "rows_cached": x.size(0), "batch": 32, "bitwidth": 4, "iterations": iterations}
    for name, fused in (("fused_mfma", True), ("elementwise_plus_torch_gemm", False)):
        AdaroundOptimizer.use_fused_linear = fused
        alpha0 = wrapper.alpha.data.clone()
        AdaroundOptimizer.optimize_rounding_on_cached_acts(wrapper, None, x, y, params, batches=batches[:20])  # warm-up
        wrapper.alpha.data.copy_(alpha0)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        AdaroundOptimizer.optimize_rounding_on_cached_acts(wrapper, None, x, y, params, batches=batches)
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        res[name] = {"ms_per_iteration": dt * 1e3 / iterations, "iterations_per_s": iterations / dt}
        if not fused:
            wrapper.alpha.data.copy_(alpha0)
    AdaroundOptimizer.use_fused_linear = True

    # per-kernel times of the fused iteration (floor(W / delta) as the optimizer stores it: int8 for this 4-bit grid;
    # the algorithmic bytes below stay those of the float32 formulation, 8 and 28 B/element).  Each kernel is timed over
    # a region of back-to-back launches of that kernel alone between one event pair (events between single launches
    # would put a bubble after every kernel); the forward region is the pair of launches the forward entry point makes
    # (split-K GEMM + loss/gradient kernel).
    w = ops.adaround_floor_i8(wrapper.weight.detach(), wrapper.num_channel, wrapper.n_per_channel, wrapper.delta,
                              wrapper.offset, wrapper.clip_min, wrapper.clip_max)
    floor_storage = "int8"
    if w is None:
        w = ops.adaround_floor(wrapper.weight.detach(), wrapper.num_channel, wrapper.n_per_channel, wrapper.delta)
        floor_storage = "float32"
    alpha = wrapper.alpha.data
    m, v = torch.zeros_like(alpha), torch.zeros_like(alpha)
    ws = ops.adaround_linear_workspace(o, k, w.device)
    gout = torch.empty(32, o, device=w.device)
    idx = torch.stack(batches[:timed_kernel_iters]).to(torch.int32).to(w.device)

    def fwd(i):
        ops.adaround_linear_fwd(w, alpha, x, idx[i], y, None, wrapper.num_channel, wrapper.delta, wrapper.offset,
                                wrapper.clip_min, wrapper.clip_max, 0, ws, gout)

    def bwd(i):
        ops.adaround_linear_bwd_adam(w, gout, x, idx[i], alpha, m, v, wrapper.num_channel, wrapper.delta,
                                     wrapper.offset, wrapper.clip_min, wrapper.clip_max, 0.01, 10.0, 1e-3, 0.9, 0.999,
                                     1e-8, i + 1)

    def region(fn):
        for i in range(3):
            fn(i)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        e0.record()
        for i in range(timed_kernel_iters):
            fn(i)
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / timed_kernel_iters

    f, b = region(fwd), region(bwd)
    # bytes the kernels move per weight element: floor(W / delta) (1 byte as int8, 4 as float32) + alpha in the
    # forward; floor + alpha, m, v read and alpha, m, v written in the backward (hardware counters agree within 3 %).
    # The figures "on the float32 formulation" price the same time at 8 and 28 B/element, what a kernel that kept
    # floor(W / delta) as float32 would move; they are not what the memory system saw.
    fb = w.element_size()
    res["fused_kernels"] = {
        "timing": "mean over back-to-back launches of one kernel between one event pair",
        "fwd_ms": f, "bwd_ms": b, "floor_storage": floor_storage,
        "fwd_bytes_moved": (fb + 4) * n, "fwd_GBps": (fb + 4) * n / f / 1e6,
        "fwd_frac_hbm": (fb + 4) * n / f / 1e6 / HBM_PEAK_GBPS,
        "fwd_GBps_on_float32_formulation": 8 * n / f / 1e6,
        "fwd_mfma_TFLOPs": 2.0 * 32 * n / f / 1e9,
        "bwd_bytes_moved": (fb + 24) * n, "bwd_GBps": (fb + 24) * n / b / 1e6,
        "bwd_frac_hbm": (fb + 24) * n / b / 1e6 / HBM_PEAK_GBPS,
        "bwd_GBps_on_float32_formulation": 28 * n / b / 1e6,
        "bwd_mfma_TFLOPs": 2.0 * 32 * n / b / 1e9}

    # the same layer with 64, 128 and 256 rows per iteration (2, 4, 8 blocks of 32 through the same kernels: the
    # weight-shaped traffic stays, the MFMA work and the activation reads grow with the rows), each against the general
    # path (soft-rounding kernel, torch GEMMs, fused backward kernel) on the same batches
    per_rows = []
    for rows_it in (32, 64, 128, 256):
        gout_r = torch.empty(rows_it, o, device=w.device)
        ws_r = ops.adaround_linear_workspace(o, k, w.device, rows_it)
        torch.manual_seed(1005 + rows_it)
        idx_r = torch.stack([torch.randperm(x.size(0))[:rows_it] for _ in range(timed_kernel_iters)])
        idx_dev = idx_r.to(torch.int32).to(w.device)

        def fwd_r(i):
            ops.adaround_linear_fwd(w, alpha, x, idx_dev[i], y, None, wrapper.num_channel, wrapper.delta, wrapper.offset,
                                    wrapper.clip_min, wrapper.clip_max, 0, ws_r, gout_r)

        def bwd_r(i):
            ops.adaround_linear_bwd_adam(w, gout_r, x, idx_dev[i], alpha, m, v, wrapper.num_channel, wrapper.delta,
                                         wrapper.offset, wrapper.clip_min, wrapper.clip_max, 0.01, 10.0, 1e-3, 0.9,
                                         0.999, 1e-8, i + 1)

        f_r, b_r = region(fwd_r), region(bwd_r)
        loops = {}
        n_it = min(200, iterations)
        for name, fused in (("fused", True), ("general", False)):
            AdaroundOptimizer.use_fused_linear = fused
            AdaroundOptimizer.fused_rows_limit = 256      # (the optimizer's own choice stops at 128 rows)
            alpha0 = wrapper.alpha.data.clone()
            bl = [idx_r[i % timed_kernel_iters] for i in range(n_it)]
            AdaroundOptimizer.optimize_rounding_on_cached_acts(wrapper, None, x, y, params, batches=bl[:10])
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            AdaroundOptimizer.optimize_rounding_on_cached_acts(wrapper, None, x, y, params, batches=bl)
            torch.cuda.synchronize()
            loops[name] = (time.perf_counter() - t0) * 1e3 / n_it
            wrapper.alpha.data.copy_(alpha0)
        AdaroundOptimizer.use_fused_linear = True
        AdaroundOptimizer.fused_rows_limit = 128
        per_rows.append({"rows": rows_it, "fwd_ms": f_r, "bwd_ms": b_r,
                         "fwd_GBps_moved": (fb + 4) * n / f_r / 1e6, "bwd_GBps_moved": (fb + 24) * n / b_r / 1e6,
                         "fwd_mfma_TFLOPs": 2.0 * rows_it * n / f_r / 1e9, "bwd_mfma_TFLOPs": 2.0 * rows_it * n / b_r / 1e9,
                         "loop_ms_per_iteration_fused": loops["fused"],
                         "loop_ms_per_iteration_general": loops["general"]})
    res["rows_per_iteration"] = per_rows

    # convolution layers take the general path (soft-rounding kernel, torch's convolution and its weight gradient, fused
    # backward / Adam kernel): the iteration with the loss gradient written out against autograd's recording of it
    from aimet_amd.common.defs import QuantScheme
    from aimet_amd.v1.adaround.adaround_wrapper import AdaroundWrapper
    from aimet_amd.v1.qc_quantize_op import StaticGridQuantWrapper
    conv_rows = []
    for cin, cout, ksize, hw in ((256, 256, 3, 14), (512, 512, 3, 7), (1024, 256, 1, 14), (64, 64, 3, 56)):
        torch.manual_seed(1005)
        conv = torch.nn.Conv2d(cin, cout, ksize, padding=ksize // 2, bias=False).to(w.device)
        xc = torch.randn(256, cin, hw, hw, device=w.device)
        with torch.no_grad():
            yc = conv(xc)
        qw = StaticGridQuantWrapper(conv, 4, 8, round_mode='nearest', quant_scheme=QuantScheme.post_training_tf,
                                    is_symmetric=True)
        qw.enable_per_channel_quantization()
        qw.param_quantizers['weight'].update_encoding_stats(conv.weight.data)
        qw.param_quantizers['weight'].compute_encoding()
        layer = AdaroundWrapper(qw)
        row = {"conv": [cout, cin, ksize, ksize], "input": [32, cin, hw, hw]}
        n_it = min(200, iterations)
        hp = AdaroundHyperParameters(n_it, 0.01, (20, 2), 0.2)
        for name, explicit, one_pass in (("ms_per_iteration", True, True),
                                         ("ms_per_iteration_loss_gradient_by_tensor_operations", True, False),
                                         ("ms_per_iteration_through_autograd", False, False)):
            AdaroundOptimizer.use_explicit_gradient = explicit
            AdaroundOptimizer.use_fused_recon_gradient = one_pass
            alpha0 = layer.alpha.data.clone()
            AdaroundOptimizer.optimize_rounding_on_cached_acts(layer, torch.relu, xc, yc,
                                                               AdaroundHyperParameters(10, 0.01, (20, 2), 0.2))
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            AdaroundOptimizer.optimize_rounding_on_cached_acts(layer, torch.relu, xc, yc, hp)
            torch.cuda.synchronize()
            row[name] = (time.perf_counter() - t0) * 1e3 / n_it
            layer.alpha.data.copy_(alpha0)
        AdaroundOptimizer.use_explicit_gradient = True
        AdaroundOptimizer.use_fused_recon_gradient = True
        conv_rows.append(row)
    res["convolution_layers_general_path"] = conv_rows

    # the GEMM-bound variant: every iteration uses all 2048 cached rows.  The fused kernels are built for the
    # reference's batch of 32 (the weight-shaped traffic dominates there); a batch of 2048 goes through the general
    # path: soft-rounding kernel, torch's GEMMs (hipBLASLt) for the layer and its weight gradient, fused
    # backward/regulariser/Adam kernel.  The two GEMMs are also timed alone.
    rows = x.size(0)
    full = [torch.arange(rows) for _ in range(12)]
    alpha0 = wrapper.alpha.data.clone()
    full_params = AdaroundHyperParameters(max(iterations, len(full)), 0.01, (20, 2), 0.2)
    AdaroundOptimizer.optimize_rounding_on_cached_acts(wrapper, None, x, y, full_params, batches=full[:2])
    wrapper.alpha.data.copy_(alpha0)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    AdaroundOptimizer.optimize_rounding_on_cached_acts(wrapper, None, x, y, full_params, batches=full[2:])
    torch.cuda.synchronize()
    it_ms = (time.perf_counter() - t0) * 1e3 / 10
    wrapper.alpha.data.copy_(alpha0)
    wq = torch.randn(o, k, device=x.device) * 0.02
    go = torch.randn(rows, o, device=x.device)

    def gemms(i):
        torch.nn.functional.linear(x, wq)
        torch.mm(go.t(), x)

    g_ms = region(gemms)
    flops = 2 * 2.0 * rows * o * k
    res["batch_2048_gemm_bound"] = {
        "path": "soft-round kernel + torch GEMMs (hipBLASLt) + fused backward/Adam kernel; the MFMA-fused kernels "
                "take up to 256 rows",
        "ms_per_iteration": it_ms, "gflop_per_iteration": flops / 1e9,
        "iteration_TFLOPs": flops / it_ms / 1e9,
        "gemms_alone_ms": g_ms, "gemms_alone_TFLOPs": flops / g_ms / 1e9,
        "gemms_alone_frac_fp32_mfma_peak": flops / g_ms / 1e9 / 157.3}
    return res


def torch_ops_adaround_baseline(torch, iterations=20):
    """The same iteration written with stock torch ops + autograd + torch.optim.Adam on the GPU (what the reference's
    Python does when run on PyTorch-ROCm): a comparison figure, not part of the product."""
    wrapper, x, y = _adaround_layer(torch)
    w = wrapper.weight.detach()
    d, o = wrapper.delta.view(-1, 1), wrapper.offset.view(-1, 1)
    alpha = torch.nn.Parameter(wrapper.alpha.data.clone())
    opt = torch.optim.Adam([alpha])
    torch.manual_seed(1005)

    def step(it):
        idx = torch.randperm(x.size(0))[:32].to(x.device)
        opt.zero_grad()
        h = torch.clamp(torch.sigmoid(alpha) * 1.2 - 0.1, 0, 1)
        wq = (torch.clamp(torch.floor(w / d) + h - o, wrapper.clip_min, wrapper.clip_max) + o) * d
        out = torch.nn.functional.linear(x[idx], wq)
        recon = (torch.norm(out - y[idx], p="fro", dim=1) ** 2).mean()
        h2 = torch.clamp(torch.sigmoid(alpha) * 1.2 - 0.1, 0, 1)
        rnd = 0.01 * torch.add(1, -(torch.add(2 * h2, -1).abs()).pow(10.0)).sum()
        (recon + rnd).backward()
        opt.step()

    for it in range(3):
        step(it)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for it in range(iterations):
        step(it)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    return {"ms_per_iteration": dt * 1e3 / iterations, "iterations": iterations,
            "what": "torch elementwise ops + autograd + torch.optim.Adam on the same GPU"}


def _resnet50_shaped(torch):
    """ResNet-50 layer shapes from Conv2d / ReLU / MaxPool / Add / Linear modules (batch norms folded away)."""
    from torch import nn
    from aimet_amd.v1.nn.modules.custom import Add

    class Bottleneck(nn.Module):
        def __init__(self, cin, mid, cout, stride):
            super().__init__()
            self.conv1, self.relu1 = nn.Conv2d(cin, mid, 1), nn.ReLU()
            self.conv2, self.relu2 = nn.Conv2d(mid, mid, 3, stride=stride, padding=1), nn.ReLU()
            self.conv3 = nn.Conv2d(mid, cout, 1)
            self.down = nn.Conv2d(cin, cout, 1, stride=stride) if (stride != 1 or cin != cout) else None
            self.add, self.relu3 = Add(), nn.ReLU()

        def forward(self, x):
            y = self.conv3(self.relu2(self.conv2(self.relu1(self.conv1(x)))))
            return self.relu3(self.add(y, x if self.down is None else self.down(x)))

    class Net(nn.Module):
        def __init__(self):
            super().__init__()
            self.conv1, self.relu = nn.Conv2d(3, 64, 7, stride=2, padding=3), nn.ReLU()
            self.maxpool = nn.MaxPool2d(3, stride=2, padding=1)
            blocks, cin = [], 64
            for mid, count, stride in ((64, 3, 1), (128, 4, 2), (256, 6, 2), (512, 3, 2)):
                for i in range(count):
                    blocks.append(Bottleneck(cin, mid, mid * 4, stride if i == 0 else 1))
                    cin = mid * 4
            self.layers = nn.Sequential(*blocks)
            self.avgpool, self.flatten, self.fc = nn.AdaptiveAvgPool2d(1), nn.Flatten(), nn.Linear(2048, 1000)

        def forward(self, x):
            x = self.layers(self.maxpool(self.relu(self.conv1(x))))
            return self.fc(self.flatten(self.avgpool(x)))

    torch.manual_seed(1004)
    return Net().eval()


def quantsim_resnet50_shaped(torch, batch=64, quant_scheme='tf', v2=False):
    """The simulation-model workload: the ResNet-50-shaped net on the GPU, a QuantizationSimModel around it with int8
    per-channel symmetric weight quantizers and int8 per-tensor activation quantizers (Conv+ReLU and Add+ReLU
    supergroups, model input quantized), calibrated on 16 of the `batch` seeded N(0,1) images.
    Returns (model, sim, images).  quant_scheme: a scheme's short name or a QuantScheme; v2: the v2 simulation model."""
    import tempfile
    if v2:
        from aimet_amd.v2.quantsim import QuantizationSimModel
    else:
        from aimet_amd.v1.quantsim import QuantizationSimModel
    dev = torch.device("cuda", 0)
    model = _resnet50_shaped(torch).to(dev)
    g = torch.Generator(device=dev).manual_seed(1004)
    x = torch.randn(batch, 3, 224, 224, device=dev, generator=g)
    cfg = {"defaults": {"ops": {"is_output_quantized": "True"},
                        "params": {"is_quantized": "True", "is_symmetric": "True"},
                        "strict_symmetric": "False", "per_channel_quantization": "True"},
           "params": {"bias": {"is_quantized": "False"}},
           "op_type": {"Flatten": {"is_output_quantized": "False"}},
           "supergroups": [{"op_list": ["Conv", "Relu"]}, {"op_list": ["Add", "Relu"]}],
           "model_input": {"is_input_quantized": "True"}, "model_output": {}}
    with tempfile.NamedTemporaryFile("w", suffix=".json", delete=False) as f:
        json.dump(cfg, f)
    sim = QuantizationSimModel(model, dummy_input=x[:2], quant_scheme=quant_scheme, default_output_bw=8,
                               default_param_bw=8, config_file=f.name)
    os.unlink(f.name)
    with torch.no_grad():
        sim.compute_encodings(lambda m, a: m(a), x[:16])
    return model, sim, x


def bench_quantsim(torch, steps=10, batch=64):
    """cfg4: QuantizationSimModel forward on a random-init ResNet-50-shaped net, batch 64, int8 per-channel weight
    quantizers and int8 per-tensor activation quantizers; QDQ overhead against the plain fp32 forward."""
    model, sim, x = quantsim_resnet50_shaped(torch, batch)

    def timed(fn):
        with torch.no_grad():
            for _ in range(5):                      # (the first passes after a change of batch size are slow)
                fn()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(steps):
                fn()
            torch.cuda.synchronize()
        return (time.perf_counter() - t0) * 1e3 / steps

    from aimet_amd.v1.qc_quantize_op import StaticGridQuantWrapper

    def requantizing(fn):
        # the reference's behaviour: every parameter quantized again in every forward
        StaticGridQuantWrapper.cache_quantized_params = False
        try:
            return timed(fn)
        finally:
            StaticGridQuantWrapper.cache_quantized_params = True

    # the three variants in turn, several rounds, median of the rounds: one variant timed after another in a single
    # block differs by +-0.3 ms from run to run, more than what separates them
    rounds = [(timed(lambda: model(x)), timed(lambda: sim.model(x)), requantizing(lambda: sim.model(x)))
              for _ in range(5)]
    fp32_ms, sim_ms, sim_requant_ms = (sorted(r[k] for r in rounds)[len(rounds) // 2] for k in range(3))
    requant_b1_ms = requantizing(lambda: sim.model(x[:1]))
    # every weight tensor of the model in one launch against one launch per tensor (events around back-to-back
    # repetitions; outputs preallocated on both sides)
    from aimet_amd import ops
    entries = []
    for _, w in sim.quant_wrappers():
        q = w.param_quantizers.get("weight")
        if q is None or not q.enabled or not isinstance(q.encoding, list):
            continue
        data = w._module_to_wrap.weight.data                          # pylint: disable=protected-access
        entries.append((data, data.shape[0], data[0].numel(), *q.device_params(data.device)[:4]))
    multi = ops.QdqMulti(entries)
    outs = multi.outputs

    def one_by_one():
        for e, o in zip(entries, outs):
            ops.qdq_per_channel(e[0], e[1], e[2], *e[3:7], out=o)

    def events(fn, reps=20):
        fn()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        e0.record()
        for _ in range(reps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / reps

    multi_ms, single_ms = events(multi), events(one_by_one)
    weights = {"tensors": len(entries), "elements": multi.elements,
               "note": "102 MB of weights: rewritten back to back they stay in the 256 MB last-level cache",
               "one_launch_ms": multi_ms, "one_launch_GBps": 8 * multi.elements / multi_ms / 1e6,
               "one_launch_frac_hbm": 8 * multi.elements / multi_ms / 1e6 / HBM_PEAK_GBPS,
               "launch_per_tensor_ms": single_ms, "launch_per_tensor_GBps": 8 * multi.elements / single_ms / 1e6}
    # Latency at batch 1: launch- and Python-bound when run eagerly, so the simulated forward is also captured in a HIP
    # graph (nothing on the path waits for the device) and replayed.
    x1 = x[:1].clone()
    lat = {"fp32_eager_ms": timed(lambda: model(x1)), "sim_eager_ms": timed(lambda: sim.model(x1)),
           "sim_eager_requantizing_params_ms": requant_b1_ms}
    with torch.no_grad():
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(3):
                sim.model(x1)
        torch.cuda.current_stream().wait_stream(side)
        graph = torch.cuda.CUDAGraph()
        # captured on the stream the warm-up ran on: what the wrappers keep between forwards is kept per stream
        with torch.cuda.graph(graph, stream=side):
            y1 = sim.model(x1)
    lat["sim_hip_graph_replay_ms"] = timed(graph.replay)
    with torch.no_grad():
        ref1 = sim.model(x1)
    # (the convolutions of this model are not run-to-run deterministic, so two eager passes differ as much)
    lat["graph_vs_eager_max_abs_diff"] = float((y1 - ref1).abs().max())
    del graph
    wrappers = list(sim.quant_wrappers())
    n_act = sum(q.enabled for _, w in wrappers for q in w.input_quantizers + w.output_quantizers)
    n_par = sum(q.enabled for _, w in wrappers for q in w.param_quantizers.values())
    return {"model": "ResNet-50-shaped conv net (Conv2d/ReLU/Add, no BN), random init", "batch": batch,
            "activation_quantizers": int(n_act), "param_quantizers": int(n_par),
            "fp32_forward_ms": fp32_ms, "quantsim_forward_ms": sim_ms,
            "qdq_overhead_ms": sim_ms - fp32_ms, "qdq_overhead_pct_of_fp32": 100.0 * (sim_ms - fp32_ms) / fp32_ms,
            "quantsim_forward_requantizing_params_ms": sim_requant_ms,
            "qdq_overhead_requantizing_params_ms": sim_requant_ms - fp32_ms,
            "all_weights_qdq": weights,
            "images_per_s": batch / (sim_ms / 1e3), "fp32_images_per_s": batch / (fp32_ms / 1e3),
            "latency_batch1": lat}


def bench_end_to_end(torch, ops):
    """The two entry points a user calls, timed whole: QuantizationSimModel.compute_encodings on the ResNet-50-shaped
    net (TF-Enhanced analyzers on every activation, per-channel on every weight) against the plain forward over the
    same batches, and Adaround.apply_adaround on a small multi-layer model against the isolated iteration loop.
    "host" is the time until the Python call has queued everything (the device may still be working), "wall" the time
    until the device is done as well: where the two agree, the host paces the run."""
    import tempfile
    from aimet_amd.v1.quantsim import QuantizationSimModel
    dev = torch.device("cuda", 0)
    out = {}
    # ---- compute_encodings
    model = _resnet50_shaped(torch).to(dev)
    g = torch.Generator(device=dev).manual_seed(1004)
    num_batches, batch = 4, 64
    data = [torch.randn(batch, 3, 224, 224, device=dev, generator=g) for _ in range(num_batches)]
    cfg = {"defaults": {"ops": {"is_output_quantized": "True"},
                        "params": {"is_quantized": "True", "is_symmetric": "True"},
                        "strict_symmetric": "False", "per_channel_quantization": "True"},
           "params": {"bias": {"is_quantized": "False"}},
           "op_type": {"Flatten": {"is_output_quantized": "False"}},
           "supergroups": [{"op_list": ["Conv", "Relu"]}, {"op_list": ["Add", "Relu"]}],
           "model_input": {"is_input_quantized": "True"}, "model_output": {}}
    with tempfile.NamedTemporaryFile("w", suffix=".json", delete=False) as f:
        json.dump(cfg, f)
    sim = QuantizationSimModel(model, dummy_input=data[0][:2], quant_scheme='tf_enhanced', default_output_bw=8,
                               default_param_bw=8, config_file=f.name)
    os.unlink(f.name)

    def passes(m, batches):
        for xb in batches:
            m(xb)

    seen = {"elements": 0, "updates": 0}
    real_update = ops.Analyzer.update_stats

    def counting(self, x):
        seen["elements"] += x.numel()
        seen["updates"] += 1
        return real_update(self, x)

    with torch.no_grad():
        for _ in range(2):
            passes(model, data)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        passes(model, data)
        host_fp32 = time.perf_counter() - t0
        torch.cuda.synchronize()
        wall_fp32 = time.perf_counter() - t0
    sim.compute_encodings(passes, data[:1])                     # warm-up (kernels, allocator)
    ops.Analyzer.update_stats = counting
    try:
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        sim.compute_encodings(passes, data)
        host_cal = time.perf_counter() - t0
        torch.cuda.synchronize()
        wall_cal = time.perf_counter() - t0
    finally:
        ops.Analyzer.update_stats = real_update
    n_act = sum(q.enabled for _, w in sim.quant_wrappers() for q in w.input_quantizers + w.output_quantizers)
    n_par = sum(q.enabled for _, w in sim.quant_wrappers() for q in w.param_quantizers.values())
    out["compute_encodings_resnet50_shaped"] = {
        "scheme": "tf_enhanced", "batches": num_batches, "batch": batch, "activation_analyzers": int(n_act),
        "param_quantizers_per_channel": int(n_par), "activation_updates": seen["updates"],
        "activation_elements_observed": seen["elements"],
        "plain_forward_wall_ms": wall_fp32 * 1e3, "plain_forward_host_ms": host_fp32 * 1e3,
        "compute_encodings_wall_ms": wall_cal * 1e3, "compute_encodings_host_ms": host_cal * 1e3,
        "calibration_overhead_pct_of_forward": 100.0 * (wall_cal - wall_fp32) / wall_fp32,
        "observed_elements_per_s": seen["elements"] / wall_cal,
        "note": "compute_encodings reads every encoding back at its end, so its host time includes the device's"}
    del sim
    import gc
    gc.collect()          # the simulation model is a web of reference cycles: collected here, not inside a timed region

    # ---- the same through the v2 classes (SQNR analyzers with 2048-bin observers on every activation and, per
    # channel, on every weight), and its simulated forward afterwards
    from aimet_amd.v2.quantsim import QuantizationSimModel as V2Sim
    sim2 = V2Sim(model, dummy_input=data[0][:2], quant_scheme='tf_enhanced', default_output_bw=8, default_param_bw=8,
                 config_file=cfg)
    sim2.compute_encodings(passes, data[:1])
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    sim2.compute_encodings(passes, data)
    host_v2 = time.perf_counter() - t0
    torch.cuda.synchronize()
    wall_v2 = time.perf_counter() - t0

    def per_forward(fn, steps=10):
        with torch.no_grad():
            for _ in range(5):
                fn()
            torch.cuda.synchronize()
            t1 = time.perf_counter()
            for _ in range(steps):
                fn()
            torch.cuda.synchronize()
        return (time.perf_counter() - t1) * 1e3 / steps

    x1 = data[0][:1].clone()
    out["v2_resnet50_shaped"] = {
        "scheme": "tf_enhanced (SqnrEncodingAnalyzer)", "batches": num_batches, "batch": batch,
        "compute_encodings_wall_ms": wall_v2 * 1e3, "compute_encodings_host_ms": host_v2 * 1e3,
        "plain_forward_wall_ms": wall_fp32 * 1e3,
        "sim_forward_batch64_ms": per_forward(lambda: sim2.model(data[0])),
        "fp32_forward_batch64_ms": per_forward(lambda: model(data[0])),
        "sim_forward_batch1_ms": per_forward(lambda: sim2.model(x1)),
        "fp32_forward_batch1_ms": per_forward(lambda: model(x1))}
    # ---- a training step through the simulation (forward + backward at batch 32; quantization-aware training): in
    # training mode a v1 wrapper recomputes its parameter encodings in every forward
    xt = data[0][:32].clone()

    def training_step(m):
        def run():
            m.zero_grad(set_to_none=True)
            m(xt).float().pow(2).mean().backward()
        for _ in range(3):
            run()
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        for _ in range(5):
            run()
        torch.cuda.synchronize()
        return (time.perf_counter() - t1) * 1e3 / 5

    _, sim_tf, _ = quantsim_resnet50_shaped(torch, 32)
    steps = {"fp32_ms": training_step(model.train())}
    steps["v1_sim_ms"] = training_step(sim_tf.model.train())
    from aimet_amd.v1.tensor_quantizer import StaticGridPerChannelQuantizer
    StaticGridPerChannelQuantizer.compute_tf_encodings_on_device = False
    try:
        steps["v1_sim_encodings_through_the_host_ms"] = training_step(sim_tf.model)
    finally:
        StaticGridPerChannelQuantizer.compute_tf_encodings_on_device = True
    steps["v2_sim_ms"] = training_step(sim2.model.train())
    steps["note"] = ("min/max per-channel weight encodings; a v1 wrapper in training mode recomputes them in every "
                     "forward (as the reference does): one launch here, one host computation per channel there")
    # ---- the same step while the ranges learn (the range-learning quant schemes): every quantizer's grid follows
    # its encoding min / max, and backward returns their gradients
    from aimet_amd.common.defs import QuantScheme
    from aimet_amd.v1 import quantsim_straight_through_grad as ste
    from aimet_amd.v2.quantization.affine import QuantizeDequantize
    del sim_tf
    gc.collect()
    learning = QuantScheme.training_range_learning_with_tf_init
    _, sim_rl, _ = quantsim_resnet50_shaped(torch, 32, learning)
    steps["v1_range_learning_ms"] = training_step(sim_rl.model.train())
    in_one_launch, ste.grid_in_one_launch = ste.grid_in_one_launch, lambda *_: False
    try:
        steps["v1_range_learning_grid_by_tensor_operations_ms"] = training_step(sim_rl.model)
    finally:
        ste.grid_in_one_launch = in_one_launch
    del sim_rl
    gc.collect()
    _, sim2_rl, _ = quantsim_resnet50_shaped(torch, 32, learning, v2=True)
    steps["v2_range_learning_ms"] = training_step(sim2_rl.model.train())
    QuantizeDequantize.fuse_range_learning = False
    try:
        steps["v2_range_learning_grid_by_tensor_operations_ms"] = training_step(sim2_rl.model)
    finally:
        QuantizeDequantize.fuse_range_learning = True
    del sim2_rl
    steps["range_learning_note"] = (
        "127 quantizers; per quantizer and step the grid is one launch and the encoding gradients leave the backward's "
        "reduction kernel, against about twenty parameter-sized tensor operations")
    out["training_step_batch32_resnet50_shaped"] = steps
    del sim2, model, data
    gc.collect()

    # ---- apply_adaround
    from aimet_amd.v1.adaround.adaround_weight import Adaround, AdaroundParameters
    width, layers, iters = 2048, 3, 500
    torch.manual_seed(1005)
    mods = []
    for k in range(layers):
        mods += [torch.nn.Linear(width, width), torch.nn.ReLU()]
    net = torch.nn.Sequential(*mods[:-1]).eval().to(dev)
    loader = [(torch.randn(256, width, device=dev), torch.zeros(256)) for _ in range(4)]
    params = AdaroundParameters(loader, num_batches=4, default_num_iterations=iters,
                                forward_fn=lambda m, b: m(b[0]))
    with tempfile.TemporaryDirectory() as tmp:
        Adaround.apply_adaround(net, loader[0][0][:2], AdaroundParameters(loader, 4, 20, forward_fn=lambda m, b: m(b[0])),
                                tmp, "warm", default_param_bw=4)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        Adaround.apply_adaround(net, loader[0][0][:2], params, tmp, "bench", default_param_bw=4)
        torch.cuda.synchronize()
        total = time.perf_counter() - t0
    # the isolated loop on one layer of this size (activations cached, nothing else)
    from aimet_amd.v1.adaround.adaround_loss import AdaroundHyperParameters
    from aimet_amd.v1.adaround.adaround_optimizer import AdaroundOptimizer
    wrapper, xs, ys = _adaround_layer(torch, out_features=width, in_features=width, rows=1024)
    hp = AdaroundHyperParameters(iters, 0.01, (20, 2), 0.2)
    AdaroundOptimizer.optimize_rounding_on_cached_acts(wrapper, None, xs, ys, AdaroundHyperParameters(20, 0.01, (20, 2), 0.2))
    gc.collect()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    AdaroundOptimizer.optimize_rounding_on_cached_acts(wrapper, None, xs, ys, hp)
    torch.cuda.synchronize()
    loop = time.perf_counter() - t0
    # a small convolutional model through the same entry point (its layers take the general path)
    torch.manual_seed(1005)
    cnet = torch.nn.Sequential(torch.nn.Conv2d(3, 64, 3, padding=1), torch.nn.ReLU(), torch.nn.Conv2d(64, 64, 3, padding=1),
                               torch.nn.ReLU(), torch.nn.Conv2d(64, 128, 3, stride=2, padding=1), torch.nn.ReLU(),
                               torch.nn.Conv2d(128, 128, 1), torch.nn.ReLU(), torch.nn.Conv2d(128, 256, 3, stride=2, padding=1),
                               torch.nn.ReLU(), torch.nn.Conv2d(256, 256, 3, padding=1)).eval().to(dev)
    cloader = [(torch.randn(64, 3, 32, 32, device=dev), torch.zeros(64)) for _ in range(4)]
    conv_iters = 200
    with tempfile.TemporaryDirectory() as tmp:
        Adaround.apply_adaround(cnet, cloader[0][0][:2], AdaroundParameters(cloader, 4, 10, forward_fn=lambda m, b: m(b[0])),
                                tmp, "warm", default_param_bw=4)
        gc.collect()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        Adaround.apply_adaround(cnet, cloader[0][0][:2],
                                AdaroundParameters(cloader, 4, conv_iters, forward_fn=lambda m, b: m(b[0])), tmp, "bench",
                                default_param_bw=4)
        torch.cuda.synchronize()
        conv_total = time.perf_counter() - t0
    # a deep chain through apply_adaround and through apply_adaround_with_cache (groups of four layers whose inputs are
    # kept on the device): sampling a layer's activations costs a pass through every layer before it in the first
    # and a pass through its own group in the second
    depth, dwidth, deep_iters = 48, 1024, 50
    torch.manual_seed(1005)
    chain = []
    for k in range(depth):
        chain += [torch.nn.Linear(dwidth, dwidth), torch.nn.ReLU()]
    deep = torch.nn.Sequential(*chain[:-1]).eval().to(dev)
    dloader = [(torch.randn(256, dwidth, device=dev), torch.zeros(256)) for _ in range(4)]
    unpack = lambda m, b: m(b[0]) if isinstance(b, (list, tuple)) else m(b)
    names = [str(i) for i in range(len(deep))]
    groups = {str(g): names[g * 8:(g + 1) * 8] for g in range((len(names) + 7) // 8)}
    with tempfile.TemporaryDirectory() as tmp:
        cfg = os.path.join(tmp, "checkpoints.json")
        with open(cfg, "w") as f:
            json.dump({"grouped_modules": groups, "include_static_inputs": ["False"] * len(groups),
                        "cache_on_cpu": "False"}, f)
        deep_s = {}
        for label, call in (("apply_adaround_s", lambda it, pre: Adaround.apply_adaround(
                                 deep, dloader[0][0][:2], AdaroundParameters(dloader, 4, it, forward_fn=unpack), tmp, pre,
                                 default_param_bw=4)),
                            ("apply_adaround_with_cache_s", lambda it, pre: Adaround.apply_adaround_with_cache(
                                 deep, dloader[0][0][:2], AdaroundParameters(dloader, 4, it, forward_fn=unpack), tmp, pre,
                                 default_param_bw=4, checkpoints_config=cfg))):
            call(2, "warm")
            gc.collect()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            call(deep_iters, "bench")
            torch.cuda.synchronize()
            deep_s[label] = time.perf_counter() - t0
    out["apply_adaround_48x_linear_1024_whole_model_passes_against_kept_group_inputs"] = {
        "layers": depth, "layer": [dwidth, dwidth], "samples": 1024, "iterations_per_layer": deep_iters,
        "groups": len(groups), **deep_s}
    out["apply_adaround_6_convolutions"] = {
        "layers": 6, "input": [64, 3, 32, 32], "batches": 4, "iterations_per_layer": conv_iters, "bitwidth": 4,
        "apply_adaround_s": conv_total, "s_per_layer": conv_total / 6,
        "ms_per_iteration_end_to_end": conv_total / 6 / conv_iters * 1e3}
    out["apply_adaround_3x_linear_2048"] = {
        "layers": layers, "layer": [width, width], "samples": 1024, "iterations_per_layer": iters, "bitwidth": 4,
        "apply_adaround_s": total, "s_per_layer": total / layers,
        "ms_per_iteration_end_to_end": total / layers / iters * 1e3,
        "isolated_loop_s_per_layer": loop, "isolated_ms_per_iteration": loop / iters * 1e3,
        "outside_the_loop_s_per_layer": total / layers - loop,
        "note": "outside the loop: building the simulation model, weight encodings, sampling the layer's input and "
                "output activations through both models, writing the encodings file"}
    return out


def bench_sqnr(torch, ops, reps=5):
    """v2 SQNR analyzer on the calibration workload: 16 batches of [32,256,28,28] through the 2048-bin histogram
    observer (finite min/max + one dual-range binning pass per batch), then the 8-bit asymmetric search."""
    from aimet_amd.v2.quantization.encoding_analyzer import SqnrEncodingAnalyzer
    dev = torch.device("cuda", 0)
    n = 32 * 256 * 28 * 28
    batches = []
    for b in range(16):
        g = torch.Generator(device=dev).manual_seed(1003 + b)
        x = torch.randn(n, device=dev, generator=g).abs_()
        u = torch.rand(n, device=dev, generator=g)
        t = torch.rand(n, device=dev, generator=g)
        batches.append(torch.where(u < 0.005, (1 - t).rsqrt(), x).contiguous())
    an = SqnrEncodingAnalyzer((1,))
    acc_ms, search_ms = [], []
    for r in range(reps + 1):
        an.reset_stats()
        e = [torch.cuda.Event(enable_timing=True) for _ in range(4)]
        torch.cuda.synchronize()
        e[0].record()
        for x in batches:
            an.update_stats(x)
        e[1].record()
        e[2].record()
        mn, mx = an.compute_encodings(255.0, False)
        e[3].record()
        torch.cuda.synchronize()
        if r:
            acc_ms.append(e[0].elapsed_time(e[1]))
            search_ms.append(e[2].elapsed_time(e[3]))
    acc = sum(acc_ms) / len(acc_ms)
    srch = sum(search_ms) / len(search_ms)
    elems = 16 * n
    # per output channel of the [11008, 4096] weight: one 2048-bin histogram per row, then the symmetric 8-bit search
    w = _laplace_weights(torch, (11008, 4096), 1004, dev)
    first, later, search = [], [], []
    for r in range(3):
        chan = SqnrEncodingAnalyzer((11008, 1))
        t = []
        for step in (lambda: chan.update_stats(w), lambda: chan.update_stats(w),
                     lambda: chan.compute_encodings(255.0, True)):
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            step()
            torch.cuda.synchronize()
            t.append((time.perf_counter() - t0) * 1e3)
        first.append(t[0]), later.append(t[1]), search.append(t[2])
    # an update of running statistics reads its batch once: 4 B/element moved (the min/max-then-bin formulation of
    # the reference reads it twice: that figure is given separately and is not what the memory system saw)
    return {"elements": elems, "num_bins": 2048, "accumulate_ms": acc, "search_ms": srch,
            "elements_per_s": elems / ((acc + srch) / 1e3), "accumulate_GBps": 4.0 * elems / acc / 1e6,
            "accumulate_frac_hbm": 4.0 * elems / acc / 1e6 / HBM_PEAK_GBPS,
            "accumulate_GBps_on_two_pass_formulation": 8.0 * elems / acc / 1e6,
            "encoding": [float(mn), float(mx)],
            "per_channel_11008x4096": {"first_update_ms": min(first), "later_update_ms": min(later),
                                       "search_ms": min(search), "timing": "wall clock around one call"}}


def bench_v2_range_learning(torch, ops, steps=50):
    """v2 quantize-dequantize backward with learnable scale and offset: the one-pass kernel (tensor_grad + both
    parameter sums; 12 B per element) against the torch elementwise ops + reductions of the same expressions, on the
    main weight shape (per channel), the activation shape (per tensor) and a blockwise weight (blocks of 128)."""
    dev = torch.device("cuda", 0)
    out = {}
    for name, shape, c in (("per_channel_11008x4096", (11008, 4096), 11008), ("per_tensor_32x64x56x56", (32, 64, 56, 56), 1),
                           ("blockwise_4096x4096_block128", (4096, 4096), 4096 * 32)):
        g = torch.Generator(device=dev).manual_seed(1006)
        n = 1
        for d in shape:
            n *= d
        npc = n // c
        sets = [(torch.randn(c, npc, device=dev, generator=g) * 0.05, torch.randn(c, npc, device=dev, generator=g))
                for _ in range(3)]
        scale = (sets[0][0].abs().amax(dim=1) / 127).clamp_min(1e-6).contiguous()
        offset = torch.zeros(c, device=dev)

        def fused(k):
            x, gr = sets[k % 3]
            return ops.v2_qdq_bwd_params(x, gr, c, npc, scale, offset, -128, 127)

        def torch_ops(k):
            x, gr = sets[k % 3]
            s, o = scale.view(-1, 1), offset.view(-1, 1)
            q = x / s
            r = torch.round(q)
            mask = (-128 <= r - o) & (r - o <= 127)
            return (gr * mask, (gr * (r.clamp(o - 128, o + 127) - q * mask)).sum(dim=1),
                    (gr * (~mask * s)).sum(dim=1))

        def timed(fn):
            for k in range(5):
                fn(k)
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            torch.cuda.synchronize()
            e0.record()
            for k in range(steps):
                fn(k)
            e1.record()
            torch.cuda.synchronize()
            return e0.elapsed_time(e1) / steps

        t_fused, t_torch = timed(fused), timed(torch_ops)
        out[name] = {"elements": n, "one_pass_ms": t_fused, "torch_ops_ms": t_torch,
                     "one_pass_GBps": 12.0 * n / t_fused / 1e6, "frac_hbm": 12.0 * n / t_fused / 1e6 / HBM_PEAK_GBPS,
                     "speedup_vs_torch_ops": t_torch / t_fused}
    return out


def cpu_baseline_qdq(seconds=10.0):
    """Single-threaded oracle (C restatement of the reference CPU loops) on a [1024, 4096] slice of the workload."""
    import numpy as np
    import oracle
    o = oracle.lib
    rng = np.random.default_rng(1004)
    c, npc = 1024, 4096
    u = rng.random((c, npc)) - 0.5
    w = (-0.02 * np.sign(u) * np.log1p(-2 * np.abs(u))).astype(np.float32)
    g = rng.standard_normal((c, npc)).astype(np.float32)
    amax = np.abs(w).max(axis=1).astype(np.float64)
    encs = [o.tf_compute_encoding(-a, a, 8, sym=True) for a in amax]
    emin, emax = np.array([e.min for e in encs]), np.array([e.max for e in encs])
    params = o.per_channel_params(emin, emax, 8)
    emn32, emx32 = emin.astype(np.float32), emax.astype(np.float32)
    n, reps = c * npc, 0
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < seconds:
        o.qdq_per_channel(w, c, npc, params)
        o.ste_bwd_per_channel(w, g, c, npc, emn32, emx32)
        reps += 1
    dt = time.perf_counter() - t0
    return {"value": 20.0 * n * reps / dt / 1e9, "unit": "GB/s", "cores": 1, "kind": "port",
            "sample": f"{reps} fwd+bwd passes over a [1024,4096] fp32 slice of the workload, {dt:.1f} s, "
                      "single-threaded C restatement of the reference CPU loops (oracle/miq_oracle.c)"}


def cpu_reference_qdq_forward(seconds=5.0):
    """The reference's own compiled C++ per-channel quantize-dequantize (oracle/_ref, built from the reference tree where
    that tree exists) on the same [1024, 4096] slice: forward only (its backward is Python)."""
    import numpy as np
    import oracle
    if oracle.ref is None:
        return None
    o, r = oracle.lib, oracle.ref
    rng = np.random.default_rng(1004)
    c, npc = 1024, 4096
    u = rng.random((c, npc)) - 0.5
    w = (-0.02 * np.sign(u) * np.log1p(-2 * np.abs(u))).astype(np.float32)
    amax = np.abs(w).max(axis=1).astype(np.float64)
    encs = [o.tf_compute_encoding(-a, a, 8, sym=True) for a in amax]
    params = o.per_channel_params(np.array([e.min for e in encs]), np.array([e.max for e in encs]), 8)
    n, reps = c * npc, 0
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < seconds:
        r.qdq_per_channel(w, c, npc, params)
        reps += 1
    dt = time.perf_counter() - t0
    return {"value": 8.0 * n * reps / dt / 1e9, "unit": "GB/s", "cores": 1, "kind": "reference",
            "sample": f"{reps} forward passes over a [1024,4096] fp32 slice, {dt:.1f} s, the reference's "
                      "quantizeDequantizeTensorPerChannel compiled from its own sources"}


def cpu_baseline_calibration(seconds=5.0):
    import numpy as np
    import oracle
    o = oracle.lib
    x = np.abs(np.random.default_rng(1003).standard_normal(32 * 256 * 28 * 28 // 4)).astype(np.float32)
    pdf = o.new_pdf()
    reps = 0
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < seconds:
        pdf.update(x)
        reps += 1
    dt = time.perf_counter() - t0
    return {"value": x.size * reps / dt, "unit": "elements/s", "cores": 1, "kind": "port",
            "sample": f"{reps} histogram updates of a quarter batch ({x.size} elements), {dt:.1f} s"}


def bench_per_channel_calibration(torch, ops):
    """Per-output-channel TF-Enhanced calibration of the [11008, 4096] weight: every channel's PDF and symmetric 8-bit
    encoding from one device object (one update, one search), beside the reference's flow of one analyzer object per
    channel fed slice by slice -- that one measured on 128 channels and scaled."""
    dev = torch.device("cuda", 0)
    c, npc = 11008, 4096
    w = _laplace_weights(torch, (c, npc), 1004, dev)
    an = ops.ChannelAnalyzer(1, c, dev)
    an.update_stats(w, npc)
    an.compute_encodings(8, True)
    upd, srch = [], []
    for _ in range(3):
        an.reset()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        an.update_stats(w, npc)
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        encs, valid = an.compute_encodings(8, True)
        t2 = time.perf_counter()
        upd.append((t1 - t0) * 1e3)
        srch.append((t2 - t1) * 1e3)
    sub = 128
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for ch in range(sub):
        a1 = ops.Analyzer(1, dev)
        a1.update_stats(w[ch].contiguous())
        a1.compute_encoding(8, True)
    t_loop = (time.perf_counter() - t0) * 1e3 / sub
    return {"shape": [c, npc], "channels": c, "update_ms": min(upd), "search_and_readback_ms": min(srch),
            "update_GBps": 4.0 * c * npc / min(upd) / 1e6,
            "one_object_per_channel_ms_per_channel": t_loop, "one_object_per_channel_ms_scaled": t_loop * c,
            "speedup_vs_one_object_per_channel": t_loop * c / (min(upd) + min(srch)),
            "first_encoding": [encs[0].min, encs[0].max, encs[0].delta, encs[0].offset]}


def parity_checks(torch, ops):
    """One cheap comparison per leg against the CPU oracle, outside every timed region: the checker confirms that the
    kernels being timed produce the reference's results on this machine (the full comparisons are the GPU tests).
    Returns {leg: bool}."""
    import numpy as np
    import oracle
    from oracle import adaround_oracle as ada
    from oracle import sqnr_oracle as sq
    o = oracle.lib
    dev = torch.device("cuda", 0)
    out = {}
    rng = np.random.default_rng(7)
    # per-tensor QDQ forward + STE backward (cfg1 arithmetic, 1 M samples)
    x = rng.standard_normal(1 << 20).astype(np.float32)
    g = rng.standard_normal(1 << 20).astype(np.float32)
    enc = o.tf_compute_encoding(float(x.min()), float(x.max()), 8)
    y = ops.qdq_per_tensor(torch.from_numpy(x).to(dev), enc.min, enc.max, 8).cpu().numpy()
    gin = ops.ste_bwd_per_tensor(torch.from_numpy(x).to(dev), torch.from_numpy(g).to(dev), enc.min, enc.max).cpu().numpy()
    out["per_tensor_act_int8"] = bool(
        np.array_equal(y.view(np.uint32), o.qdq_per_tensor(x, enc.min, enc.max, 8).view(np.uint32)) and
        np.array_equal(gin, o.ste_bwd_per_tensor(x, g, np.float32(enc.min), np.float32(enc.max))))
    # per-channel symmetric int8 / int4, fp32 and bf16 storage ([256, 4096] rows of the main workload's distribution)
    c, npc = 256, 4096
    u = rng.random((c, npc)) - 0.5
    w = (-0.02 * np.sign(u) * np.log1p(-2 * np.abs(u))).astype(np.float32)
    ok = True
    for bw in (8, 4):
        amax = np.abs(w).max(axis=1).astype(np.float64)
        encs = [o.tf_compute_encoding(-a, a, bw, sym=True) for a in amax]
        emin, emax = np.array([e.min for e in encs]), np.array([e.max for e in encs])
        params = o.per_channel_params(emin, emax, bw)
        steps = 2 ** bw - 1 - (1 if emin[0] == -emax[0] else 0)
        gp = ops.per_channel_params(torch.from_numpy(emin.astype(np.float32)).to(dev),
                                    torch.from_numpy(emax.astype(np.float32)).to(dev), steps)
        wg = torch.from_numpy(w).to(dev)
        ok &= np.array_equal(ops.qdq_per_channel(wg, c, npc, *gp).cpu().numpy().view(np.uint32),
                             o.qdq_per_channel(w, c, npc, params).view(np.uint32))
        wb = torch.from_numpy(w).to(torch.bfloat16)
        got = ops.qdq_per_channel(wb.to(dev), c, npc, *gp).cpu().view(torch.int16).numpy().view(np.uint16)
        ok &= np.array_equal(got, o.qdq_per_channel_bf16(wb.view(torch.int16).numpy().view(np.uint16), c, npc, params))
        gr = rng.standard_normal((c, npc)).astype(np.float32)
        emn32, emx32 = emin.astype(np.float32), emax.astype(np.float32)
        gin = ops.ste_bwd_per_channel(wg, torch.from_numpy(gr).to(dev), c, npc, torch.from_numpy(emn32).to(dev),
                                      torch.from_numpy(emx32).to(dev)).cpu().numpy()
        ok &= np.array_equal(gin, o.ste_bwd_per_channel(w, gr, c, npc, emn32, emx32))
    out["per_channel_cells"] = bool(ok)
    # TF-Enhanced calibration: two batches of the calibration distribution, PDF bits and the chosen encoding
    an, pdf = ops.Analyzer(1, dev), o.new_pdf()
    for seed in (1, 2):
        a = np.abs(np.random.default_rng(seed).standard_normal(1 << 20)).astype(np.float32)
        a[::200] = (1.0 / np.sqrt(1.0 - np.random.default_rng(seed + 9).random(a[::200].size))).astype(np.float32)
        an.update_stats(torch.from_numpy(a).to(dev))
        pdf.update(a)
    xl, p = an.get_stats_histogram()
    e, _ = an.compute_encoding(8)
    out["tf_enhanced_calibration"] = bool(np.array_equal(p.view(np.uint64), pdf.pdf().view(np.uint64)) and
                                          (e.min, e.max, e.delta, e.offset, e.bw) == pdf.compute_encoding(8)[0].astuple())
    # per-channel TF-Enhanced: 64 rows
    ca = ops.ChannelAnalyzer(1, 64, dev)
    ca.update_stats(torch.from_numpy(w[:64]).to(dev), npc)
    encs, _ = ca.compute_encodings(8, True)
    ok = True
    for ch in (0, 17, 63):
        pc = o.new_pdf()
        pc.update(w[ch])
        ok &= (encs[ch].min, encs[ch].max, encs[ch].delta, encs[ch].offset, encs[ch].bw) == \
            pc.compute_encoding(8, True)[0].astuple()
    out["per_channel_tf_enhanced"] = bool(ok)
    # v2 SQNR observer: histogram of one batch and the chosen range
    from aimet_amd.v2.quantization.encoding_analyzer import SqnrEncodingAnalyzer
    xs = torch.randn(1 << 20) * 1.5 + 0.2
    an2, ref2 = SqnrEncodingAnalyzer((1,)), sq.SqnrAnalyzer()
    an2.update_stats(xs.to(dev))
    ref2.update_stats(xs)
    qmin, qmax = an2.compute_encodings(255.0, False)
    rmin, rmax, _ = ref2.compute_encodings(255.0, False)
    out["v2_sqnr_calibration"] = bool(torch.equal(an2.observer.get_stats()[0].histogram.cpu(), ref2.stats[0].histogram) and
                                      torch.allclose(qmin.cpu(), rmin, rtol=1e-6) and torch.allclose(qmax.cpu(), rmax, rtol=1e-6))
    # v2 backward with learnable scale / offset: input gradient bit for bit, parameter sums to 2e-5
    xw = (rng.standard_normal((64, 1024)) * 0.5).astype(np.float32)
    gw = rng.standard_normal((64, 1024)).astype(np.float32)
    sc = (np.abs(xw).max(axis=1) / 127).astype(np.float32)
    of = np.zeros(64, np.float32)
    gi, gs, go = ops.v2_qdq_bwd_params(torch.from_numpy(xw).to(dev), torch.from_numpy(gw).to(dev), 64, 1024,
                                       torch.from_numpy(sc).to(dev), torch.from_numpy(of).to(dev), -128, 127)
    want_gi = o.v2_qdq_bwd(xw, gw, 64, 1024, sc, of, -128, 127)
    xt = torch.from_numpy(xw)
    s_, o_ = torch.from_numpy(sc).view(-1, 1), torch.from_numpy(of).view(-1, 1)
    q = xt / s_
    r = torch.round(q)
    mask = (-128 <= r - o_) & (r - o_ <= 127)
    want_gs = (torch.from_numpy(gw) * (r.clamp(o_ - 128, o_ + 127) - q * mask)).double().sum(dim=1)
    out["v2_range_learning_backward"] = bool(np.array_equal(gi.cpu().numpy().view(np.uint32), want_gi.view(np.uint32)) and
                                             torch.allclose(gs.double().cpu(), want_gs, rtol=2e-5, atol=1e-4))
    # AdaRound fused Linear path: three iterations on a [64, 256] layer against the torch-CPU restatement
    torch.manual_seed(0)
    wt = torch.randn(64, 256) * 0.05
    delta = (wt.abs().amax(dim=1) * 2 / 15).float()
    offset = torch.full((64,), -8.0)
    alpha0 = ada.generate_alpha(wt, ada.broadcast(delta, wt, 0))
    xs_, ys_ = torch.randn(96, 256), None
    ys_ = ada.layer_output("linear", xs_, wt) + 0.02 * torch.randn(96, 64)
    bts = [torch.randperm(96)[:32] for _ in range(3)]
    a_ref, _, _, _ = ada.optimize_rounding("linear", wt, alpha0, delta, offset, 0, 15, xs_, ys_, bts, 3, 0.01, (20, 2), 0.2)
    wg_, dg, og, xg, yg = (t.to(dev) for t in (wt, delta, offset, xs_, ys_))
    alpha = ops.adaround_init_alpha(wg_, 64, 256, dg)
    fl = ops.adaround_floor(wg_, 64, 256, dg)
    m_, v_ = torch.zeros_like(alpha), torch.zeros_like(alpha)
    ws = ops.adaround_linear_workspace(64, 256, dev)
    gout = torch.empty(32, 64, device=dev)
    for k_, idx in enumerate(bts):
        beta = -1.0 if k_ < 0.2 * 3 else ada.compute_beta(3, k_, (20, 2), 0.2)
        ig = idx.to(torch.int32).to(dev)
        ops.adaround_linear_fwd(fl, alpha, xg, ig, yg, None, 64, dg, og, 0, 15, 0, ws, gout)
        ops.adaround_linear_bwd_adam(fl, gout, xg, ig, alpha, m_, v_, 64, dg, og, 0, 15, 0.01, beta, 1e-3, 0.9, 0.999,
                                     1e-8, k_ + 1)
    out["adaround_linear_4096"] = bool(torch.allclose(alpha.cpu(), a_ref, atol=5e-5))
    return out


def cpu_baseline_adaround(iterations=3):
    """The AdaRound iteration of the configuration ([4096,4096], 32 of 2048 cached rows, 4-bit) as the reference runs it
    on the CPU: torch ops + autograd + torch.optim.Adam (oracle/adaround_oracle.py), all host threads."""
    import torch
    from oracle import adaround_oracle as ada
    g = torch.Generator().manual_seed(1005)
    wt = torch.randn(4096, 4096, generator=g) * 0.02
    xs = torch.randn(2048, 4096, generator=g)
    ys = torch.nn.functional.linear(xs, wt)
    delta = (wt.abs().amax(dim=1) / 7.0).float()
    offset = torch.full((4096,), -8.0)
    alpha0 = ada.generate_alpha(wt, ada.broadcast(delta, wt, 0))
    bts = [torch.randperm(2048, generator=g)[:32] for _ in range(iterations + 1)]
    ada.optimize_rounding("linear", wt, alpha0, delta, offset, 0, 15, xs, ys, bts[:1], 1000, 0.01, (20, 2), 0.2,
                          first_iteration=300)
    t0 = time.perf_counter()
    ada.optimize_rounding("linear", wt, alpha0, delta, offset, 0, 15, xs, ys, bts[1:], 1000, 0.01, (20, 2), 0.2,
                          first_iteration=300)
    dt = time.perf_counter() - t0
    return {"value": dt * 1e3 / iterations, "unit": "ms/iteration", "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"{iterations} iterations of the [4096,4096] layer, batch 32, torch CPU ops + autograd + Adam"}


def cpu_baseline_v2(passes=3):
    """The v2 formulas as torch CPU ops with all host threads: quantize-dequantize forward + backward of the
    [11008,4096] weight (per channel), and one update of the 2048-bin histogram observer on a calibration batch."""
    import torch
    from oracle import sqnr_oracle as sq
    g = torch.Generator().manual_seed(1006)
    x = torch.randn(11008, 4096, generator=g) * 0.05
    gr = torch.randn(11008, 4096, generator=g)
    s = (x.abs().amax(dim=1, keepdim=True) / 127).clamp_min(1e-6)

    def one():
        q = x / s
        r = torch.round(q)
        mask = (-128 <= r) & (r <= 127)
        y = r.clamp(-128, 127) * s
        return y, gr * mask

    one()
    t0 = time.perf_counter()
    for _ in range(passes):
        one()
    dt = (time.perf_counter() - t0) / passes
    batch = torch.randn(32 * 256 * 28 * 28, generator=g).abs_()
    obs = sq.SqnrAnalyzer()
    obs.update_stats(batch)
    t0 = time.perf_counter()
    obs.update_stats(batch)
    t_obs = time.perf_counter() - t0
    n = x.numel()
    return {"qdq_fwd_bwd": {"value": 20.0 * n / dt / 1e9, "unit": "GB/s", "cores": torch.get_num_threads(),
                            "kind": "port", "sample": f"{passes} fwd+bwd passes over [11008,4096] fp32, torch CPU ops"},
            "histogram_observer_update": {"value": batch.numel() / t_obs, "unit": "elements/s",
                                          "cores": torch.get_num_threads(), "kind": "port",
                                          "sample": "one update of a [32,256,28,28] batch, torch.histc on the CPU"}}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--full", action="store_true", help="(kept for old command lines: every cell is measured anyway)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--only", default=None,
                    help="run a subset of the legs, comma separated (main|pt|fp8|calib|chcalib|sqnr|learn|quantsim|e2e|seqmse|adaround|floors|copyref), for profiling")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this path has no multi-GPU leg (run with --gpus 1)", file=sys.stderr)
        sys.exit(2)

    if not os.path.exists(os.path.join(ROOT, "aimet_amd", "libmiq.so")):
        import __graft_entry__
        __graft_entry__.build()
    import gc
    import torch
    from aimet_amd import ops
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    gc.disable()
    torch.cuda.set_device(0)

    main_shape = (11008, 4096)
    extra = {}
    res = None
    legs = None if args.only is None else set(args.only.split(","))

    def want(leg):
        # Python's cycle collector is off while a leg runs (as timeit does) and is run between legs: a full collection
        # walks every object the earlier legs left behind (a simulation model holds tens of thousands of encoding
        # objects) and lands in whichever host-paced region happens to be timed then -- 6 ms on a 4 ms forward
        gc.collect()
        return leg in legs if legs is not None else leg != "copyref"

    if want("copyref"):
        # a plain elementwise kernel of known traffic (reads 4 B, writes 4 B per element of the main shape): the
        # yardstick that hardware-counter readings of the kernels above are scaled by
        a = torch.randn(main_shape, device="cuda")
        b = torch.empty_like(a)
        for _ in range(10):
            torch.add(a, 1.0, out=b)
        torch.cuda.synchronize()
        extra["copyref"] = {"elements": a.numel(), "bytes_read": 4 * a.numel(), "bytes_written": 4 * a.numel()}
    if want("floors"):
        extra["launch_floors"] = bench_launch_floors(torch, ops)
    if want("main"):
        res = bench_per_channel(torch, ops, main_shape, torch.float32, 8, args.steps, args.warmup, 1004)
    if want("pt"):
        extra["per_tensor_act_int8"] = bench_per_tensor(torch, ops, max(20, args.steps), args.warmup)
    if want("fp8"):
        extra["fp8_simulation"] = bench_fp8(torch, ops, max(20, args.steps), args.warmup)
    if want("calib"):
        extra["tf_enhanced_calibration"] = bench_calibration(torch, ops, 5)
    if want("chcalib"):
        extra["per_channel_tf_enhanced"] = bench_per_channel_calibration(torch, ops)
    if want("sqnr"):
        extra["v2_sqnr_calibration"] = bench_sqnr(torch, ops)
    if want("learn"):
        extra["v2_range_learning_backward"] = bench_v2_range_learning(torch, ops)
    if want("quantsim"):
        extra["quantsim_resnet50_shaped"] = bench_quantsim(torch)
    if want("e2e"):
        extra["end_to_end"] = bench_end_to_end(torch, ops)
    if want("seqmse"):
        extra["sequential_mse"] = bench_seq_mse(torch, ops)
    if want("adaround"):
        extra["adaround_linear_4096"] = bench_adaround(torch, ops, 1000 if args.only is None else args.steps)
        extra["adaround_linear_4096"]["torch_ops_same_gpu"] = torch_ops_adaround_baseline(torch)
    if args.only is None:
        # every shape x dtype x bit-width cell of the weight configuration (the main cell is the headline above)
        cells = [(s, d, b) for s in ((512, 512, 3, 3), (4096, 4096), (11008, 4096))
                 for d in (torch.float32, torch.bfloat16) for b in (8, 4)]
        extra["per_channel_cells"] = [
            bench_per_channel(torch, ops, s, d, b, max(20, args.steps // 2), 5, 1002 + {512: 0, 4096: 1, 11008: 2}[s[0]])
            for (s, d, b) in cells if not (s == main_shape and d == torch.float32 and b == 8)]
        for cell in extra["per_channel_cells"]:
            cell["frac_hbm"] = cell["fwd_bwd_GBps"] / HBM_PEAK_GBPS
        extra["parity_checked"] = parity_checks(torch, ops)
    if res is None:
        print(json.dumps({"extra": extra}))
        return

    n = res["elements"]
    line = {
        "metric": "QDQ fwd+bwd GB/s & % of HBM peak; TF-Enhanced calib elems/s (1 GPU)",
        "value": res["fwd_bwd_GBps"], "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": res["ms_per_step"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": "per-channel symmetric int8 weight QDQ fwd + STE bwd, [11008,4096] fp32, rotated buffers",
                   "data": "Laplace(0,0.02) + 0.1% x20 outliers, 3+ buffer sets rotated so that every read comes from HBM",
                   "elements_per_step": n, "algorithmic_bytes_per_step": 20 * n,
                   "cpu_baseline_slice": "[1024,4096] of the [11008,4096] weight (the loop is single-threaded)",
                   "saved_mask_ms_per_step": res["saved_mask"]["ms_per_step"],
                   "saved_mask_bytes_moved_per_step": res["saved_mask"]["bytes_moved_per_step"],
                   "saved_mask_GBps_moved": res["saved_mask"]["fwd_bwd_GBps_moved"]},
        "pct_hbm_peak": 100.0 * res["fwd_bwd_GBps"] / HBM_PEAK_GBPS,
        "roofline": {"bound": "hbm", "kernel": "ew_vec_kernel<float, OpV1Ste, per-channel> (STE backward)",
                     "achieved": res["bwd_GBps"], "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": res["bwd_GBps"] / HBM_PEAK_GBPS,
                     "traffic": MEASURED_TRAFFIC_BYTES["ste_bwd_per_channel_f32"],
                     "avg_launch_ms": res["bwd_ms"], "algorithmic_bytes_per_launch": 12 * n,
                     "forward_kernel": {"achieved": res["fwd_GBps"], "frac": res["fwd_GBps"] / HBM_PEAK_GBPS,
                                        "avg_launch_ms": res["fwd_ms"], "algorithmic_bytes_per_launch": 8 * n,
                                        "traffic": MEASURED_TRAFFIC_BYTES["qdq_fwd_per_channel_f32"]}},
    }
    line["saved_mask_step"] = dict(res["saved_mask"], fwd_traffic=MEASURED_TRAFFIC_BYTES["qdq_mask_fwd_per_channel_f32"],
                                   bwd_traffic=MEASURED_TRAFFIC_BYTES["ste_mask_bwd_f32"], note="the same fwd+bwd step with the forward writing the "
                                   "straight-through mask (1 bit per element) and the backward reading it instead of x")
    if "tf_enhanced_calibration" in extra:
        # the metric's second half, as flat keys of the roofline object: hist_kernel over the 16 + 1 passes of the
        # calibration configuration (16 batches of [32,256,28,28] and the range discovery of the first)
        cal = extra["tf_enhanced_calibration"]
        line["calib_elements_per_s"] = cal["elements_per_s"]
        line["roofline"].update({
            "secondary_kernel": "hist_kernel (TF-Enhanced 512-bucket histogram, 16 x [32,256,28,28] fp32)",
            "secondary_achieved": cal["accumulate_GBps"], "secondary_frac": cal["accumulate_frac_hbm"],
            "secondary_algorithmic_bytes": 17 * 4 * cal["elements"] // 16,
            "calib_elements_per_s": cal["elements_per_s"], "calib_elements": cal["elements"],
            "calib_accumulate_ms": cal["accumulate_ms"], "calib_search_us": cal["search_ms_wall"] * 1e3,
            "calib_total_ms": cal["total_ms_wall"]})
    if not args.no_cpu:
        line["cpu_baseline"] = cpu_baseline_qdq()
        extra["cpu_baseline_calibration"] = cpu_baseline_calibration()
        ref_fwd = cpu_reference_qdq_forward()
        if ref_fwd is not None:
            extra["cpu_reference_qdq_forward"] = ref_fwd
        if args.only is None:
            extra["cpu_baseline_adaround"] = cpu_baseline_adaround()
            extra["cpu_baseline_v2"] = cpu_baseline_v2()
    line["extra"] = extra
    print(json.dumps(line))


if __name__ == "__main__":
    main()
