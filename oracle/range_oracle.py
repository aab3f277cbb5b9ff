"""CPU restatement of range learning's parameter-sized arithmetic -- TEST INFRASTRUCTURE, never imported by the product.

numpy float32, one rounding per operation, following

  v1  TrainingExtensions/torch/src/python/aimet_torch/v1/quantsim_straight_through_grad.py
        grid_v1              :121-162   get_computed_encodings (its operands are tensors: every "/" divides)
        range_grads_v1       :251-292   asymmetric_gradients (the part after the two sums), :296-325 symmetric_gradients
      TrainingExtensions/torch/src/python/aimet_torch/v1/tensor_quantizer.py
        ordered_range        :1347-1359 set_encoding_min_max_gating_threshold
  v2  TrainingExtensions/torch/src/python/aimet_torch/v2/quantization/affine/quantizer.py
        grid_v2              :404-436   get_scale, get_offset
        range_grads_v2       what autograd makes of them, written out: with u = min / scale,
                             d offset / d min = 1 / scale, d offset / d scale = -u / scale (round is straight-through),
                             d scale / d max = 1 / steps = -d scale / d min

The two sums every gradient formula starts from are those of the quantize-dequantize backward
(v2_qdq_bwd_params in miq_oracle.c): sum_s = d loss / d scale, sum_o = d loss / d offset, per channel.

Pinned by tests/test_oracle_range.py: the v2 gradients against float64 autograd of the reference's own expressions,
the v1 grid against the properties get_computed_encodings exists for (zero is a grid point, the range is covered), the
ordering against its three stated invariants.  The v1 gradient formulas are pinned end to end by the reference's own
check, autograd of the explicit expression (tests/test_gpu_range_learning.py).
"""
import math

import numpy as np

F32 = np.float32


def ordered_range(enc_min, enc_max):
    """min <= 0 <= max and max >= min + 1e-5; NaN stays NaN (torch.clamp and torch.maximum keep it)."""
    mn, mx = np.asarray(enc_min, F32).copy(), np.asarray(enc_max, F32).copy()
    mn = np.where(mn > 0, F32(0), mn)
    mx = np.where(mx < 0, F32(0), mx)
    with np.errstate(invalid="ignore"):
        mx = np.maximum(mx, mn + F32(1e-5))            # np.maximum propagates NaN, as torch.maximum does
    return mn.astype(F32), mx.astype(F32)


def grid_v1(enc_min, enc_max, bitwidth, symmetric, strict_symmetric, unsigned_symmetric):
    """(delta, offset, num_steps)"""
    mn, mx = np.asarray(enc_min, F32), np.asarray(enc_max, F32)
    num_steps = 2 ** bitwidth - 1 - (1 if symmetric and strict_symmetric else 0)
    steps, half = F32(num_steps), num_steps / 2
    with np.errstate(all="ignore"):
        if symmetric and not unsigned_symmetric:
            delta = mx / F32(math.floor(half))
            offset = np.full_like(mn, -F32(math.ceil(half)))
        else:
            delta = (mx - mn) / steps
            if symmetric:
                offset = mn / delta
            else:
                zero_point = np.rint(-mn / delta)
                offset = -np.minimum(steps, np.maximum(F32(0), zero_point))
    return delta.astype(F32), offset.astype(F32), num_steps


def grid_v2(enc_min, enc_max, qmin, qmax, symmetric, divide=True):
    """(scale, offset).  divide=False forms "/ steps" as the product with float32(1 / steps), which is what torch's
    device kernels do when a tensor is divided by a number; torch's CPU kernels divide."""
    mn, mx = np.asarray(enc_min, F32), np.asarray(enc_max, F32)
    steps = F32(qmax - qmin)
    with np.errstate(all="ignore"):
        scale = (mx - mn) / steps if divide else (mx - mn) * (F32(1) / steps)
        offset = np.zeros_like(mn) if symmetric else np.rint(mn / scale) - F32(qmin)
    return scale.astype(F32), offset.astype(F32)


def range_grads_v1(sum_s, sum_o, enc_min, enc_max, num_steps, symmetric):
    """(grad_min, grad_max) from the two channel sums"""
    s, o = np.asarray(sum_s, F32), np.asarray(sum_o, F32)
    mn, mx = np.asarray(enc_min, F32), np.asarray(enc_max, F32)
    steps = F32(num_steps)
    if symmetric:
        grad_max = s / F32(num_steps // 2)
        return (-grad_max).astype(F32), grad_max.astype(F32)
    term1 = s / steps
    width = mx - mn
    term2 = steps / (width * width) * o
    return (-term1 + mx * term2).astype(F32), (term1 - mn * term2).astype(F32)


def range_grads_v2(sum_s, sum_o, enc_min, scale, qmin, qmax, symmetric, divide=True):
    """(grad_min, grad_max) from the two channel sums; `divide` as in grid_v2"""
    s, o = np.asarray(sum_s, F32), np.asarray(sum_o, F32)
    mn, sc = np.asarray(enc_min, F32), np.asarray(scale, F32)
    steps = F32(qmax - qmin)

    def by_steps(t):
        return t / steps if divide else t * (F32(1) / steps)
    if symmetric:
        grad_max = by_steps(s)
        return (-grad_max).astype(F32), grad_max.astype(F32)
    through_scale = s + (-o) * ((mn / sc) / sc)
    grad_max = by_steps(through_scale)
    return (o / sc + (-grad_max)).astype(F32), grad_max.astype(F32)
