"""Straight-through-estimator gradient of the v1 path.

compute_dloss_by_dx mirrors TrainingExtensions/torch/src/python/aimet_torch/v1/quantsim_straight_through_grad.py:91-118:
grad * ((encoding_min <= x) & (x <= encoding_max)), one fused kernel instead of three elementwise passes and a bool
temporary.

Range learning (:121-346): get_computed_encodings, the quantize-dequantize forward and the gradients w.r.t. the input
and the learnable encoding min / max.  The reference keeps x_quant, delta, offset and a bool mask at full tensor size
for backward and forms the encoding gradients from five more full-size products; here forward is one kernel, and
backward is one kernel that re-derives grid position and mask from the saved input and returns the input gradient
together with the two per-channel sums the encoding gradients are made of.
"""
import functools
import math

import torch

from .. import ops


def broadcast_to_tensor(tensor, encoding, ch_axis):
    """1-d per-channel encoding values -> shape broadcastable against `tensor` (reference :66-88)."""
    if not isinstance(encoding, torch.Tensor):
        encoding = torch.tensor(encoding).to(tensor.device)
    assert len(encoding.shape) <= 1
    if encoding.numel() == 1:
        return encoding
    assert encoding.numel() == tensor.shape[ch_axis]
    shape = tuple(dim if axis == ch_axis else 1 for axis, dim in enumerate(tensor.shape))
    return encoding.view(shape)


def compute_dloss_by_dx(x, grad, encoding_min, encoding_max, ch_axis=0):
    """dL/dx = grad where encoding_min <= x <= encoding_max (both ends inclusive), 0 elsewhere.

    encoding_min / encoding_max: python floats (per-tensor), or sequences / 1-d tensors with one value per channel
    along `ch_axis`.
    """
    per_channel = isinstance(encoding_min, (list, tuple)) or \
        (isinstance(encoding_min, torch.Tensor) and encoding_min.numel() > 1)
    if not per_channel:
        mn = float(encoding_min[0] if isinstance(encoding_min, (list, tuple, torch.Tensor)) else encoding_min)
        mx = float(encoding_max[0] if isinstance(encoding_max, (list, tuple, torch.Tensor)) else encoding_max)
        if x.dtype != torch.float32:
            # the reference compares against a 0-dim tensor, which torch's type promotion casts to x's dtype
            mn = float(torch.tensor(mn, dtype=torch.float32).to(x.dtype))
            mx = float(torch.tensor(mx, dtype=torch.float32).to(x.dtype))
        if x.dtype == torch.float16:
            # the kernels take float32 and bfloat16: a float16 value is the same number in float32, and the bounds
            # have just been rounded to float16 as the reference's comparison rounds them
            return ops.ste_bwd_per_tensor(x.float(), grad.float(), mn, mx).to(x.dtype)
        return ops.ste_bwd_per_tensor(x, grad, mn, mx)
    mn = torch.as_tensor(encoding_min, dtype=torch.float32).to(x.device)
    mx = torch.as_tensor(encoding_max, dtype=torch.float32).to(x.device)
    num_channel = x.shape[ch_axis]
    assert mn.numel() == num_channel and mx.numel() == num_channel
    n_per_channel = functools.reduce(lambda a, b: a * b, x.shape[ch_axis + 1:], 1)
    if x.dtype == torch.float16:
        # (one bound per channel is a tensor with a dimension: the reference's comparison promotes x to float32)
        return ops.ste_bwd_per_channel(x.float(), grad.float(), num_channel, n_per_channel, mn, mx).to(x.dtype)
    return ops.ste_bwd_per_channel(x, grad, num_channel, n_per_channel, mn, mx)


# ------------------------------------------------------------------------------------------------- range learning
def get_computed_encodings(bitwidth, encoding_min, encoding_max, use_symmetric_encodings, use_strict_symmetric,
                           is_unsigned_symmetric):
    """(delta, offset, num_steps) from learnable encoding min / max tensors (reference :121-162, which follows the
    C++ getComputedEncodings): signed symmetric -> delta = max / floor(steps / 2), offset = -ceil(steps / 2);
    unsigned symmetric -> delta = (max - min) / steps, offset = min / delta; asymmetric -> the zero point
    round(-min / delta) clamped to the grid."""
    num_steps = 2 ** bitwidth - 1
    if use_symmetric_encodings and use_strict_symmetric:
        num_steps -= 1
    half = num_steps / 2
    steps = torch.full_like(encoding_min, float(num_steps))
    if use_symmetric_encodings and not is_unsigned_symmetric:
        # a tensor as divisor, as in the reference: torch's device kernels multiply by the reciprocal of a number
        delta = encoding_max / torch.full_like(encoding_min, float(math.floor(half)))
        offset = torch.full_like(encoding_min, -float(math.ceil(half)))
    else:
        delta = (encoding_max - encoding_min) / steps
        if use_symmetric_encodings:
            offset = encoding_min / delta
        else:
            offset = -torch.clamp(torch.round(-encoding_min / delta), 0.0, float(num_steps))
    return delta, offset, steps


def _channel_geometry(tensor, num_param, ch_axis):
    if num_param == 1:
        return 1, max(tensor.numel(), 1)
    assert num_param == tensor.shape[ch_axis]
    return num_param, max(math.prod(tensor.shape[ch_axis + 1:]), 1)


def range_mode(tensor_quantizer) -> int:
    """Which of the library's grid formulas a learned-grid quantizer follows (get_computed_encodings' three cases)."""
    if tensor_quantizer.use_symmetric_encodings:
        return ops.RANGE_V1_UNSIGNED_SYMMETRIC if tensor_quantizer.is_unsigned_symmetric \
            else ops.RANGE_V1_SIGNED_SYMMETRIC
    return ops.RANGE_V1_ASYMMETRIC


def _grid_key(tensor_quantizer, encoding_min, encoding_max):
    # pylint: disable=protected-access
    return (id(encoding_min), encoding_min._version, id(encoding_max), encoding_max._version,
            tensor_quantizer.bitwidth, range_mode(tensor_quantizer), tensor_quantizer.use_strict_symmetric,
            ops.current_stream_handle(encoding_min.device))


def grid_in_one_launch(encoding_min, encoding_max) -> bool:
    """The library forms delta / offset itself for float32 ranges held contiguously on the GPU."""
    return encoding_min is not None and encoding_max is not None and encoding_min.is_cuda and \
        encoding_min.dtype == encoding_max.dtype == torch.float32 and encoding_min.is_contiguous() and \
        encoding_max.is_contiguous() and encoding_min.numel() == encoding_max.numel() and \
        encoding_min.device == encoding_max.device


def gate_and_prepare_grid(tensor_quantizer, encoding_min, encoding_max):
    """The wrapper's ordering of a learned range (min <= 0 <= max, max >= min + 1e-5), in place, and the grid that
    range gives -- one launch.  The grid is left with the quantizer for the forward pass that follows."""
    grid = ops.range_to_grid(encoding_min.detach().reshape(-1), encoding_max.detach().reshape(-1), 0,
                             _num_steps(tensor_quantizer), range_mode(tensor_quantizer), gate=True)
    tensor_quantizer.__dict__['_prepared_grid'] = (_grid_key(tensor_quantizer, encoding_min, encoding_max), grid)


def _grid_of(tensor_quantizer, encoding_min, encoding_max):
    prepared = tensor_quantizer.__dict__.pop('_prepared_grid', None)
    if prepared is not None and prepared[0] == _grid_key(tensor_quantizer, encoding_min, encoding_max):
        return prepared[1]
    return ops.range_to_grid(encoding_min.detach().reshape(-1), encoding_max.detach().reshape(-1), 0,
                             _num_steps(tensor_quantizer), range_mode(tensor_quantizer))


def learned_grid_forward(tensor, tensor_quantizer, encoding_min, encoding_max):
    """Forward of range learning (reference calculate_forward_pass :185-249):
    x_dequant = (clamp(round(x / delta) - offset, 0, steps) + offset) * delta, in one kernel.  Returns the output and
    what backward needs -- no full-size intermediates are kept: the backward kernel recomputes the grid position and
    the mask from the saved input.  What backward needs is (grid, steps, channels, elements per channel), grid being
    the library's [4, C] table of delta, offset and the min / max they were made from, or, for ranges the library
    does not take (not float32, not on the GPU), (delta, offset, steps, channels, elements per channel)."""
    if tensor.dtype not in (torch.float32, torch.float16, torch.bfloat16):
        raise RuntimeError("Invalid input data type. Expected torch.float32 or torch.float16. "
                           f"Got {tensor.dtype}.")
    if not tensor.dtype == encoding_min.dtype == encoding_max.dtype:
        raise RuntimeError("Data type mismatch. Expected the input and encoding min & max to be of same dtype."
                           f"Got {tensor.dtype} input, {encoding_min.dtype} encoding_min, "
                           f"and {encoding_max.dtype} encoding_max")
    if tensor_quantizer.bitwidth >= 32:
        raise RuntimeError(f'Invalid bitwidth: {tensor_quantizer.bitwidth}')
    num_steps = _num_steps(tensor_quantizer)
    x = tensor if tensor.dtype != torch.float16 else tensor.float()
    if grid_in_one_launch(encoding_min, encoding_max) and tensor.is_cuda:
        grid = _grid_of(tensor_quantizer, encoding_min, encoding_max)
        c, npc = _channel_geometry(tensor, grid.shape[1], tensor_quantizer.channel_axis)
        out = ops.v2_qdq(x, c, npc, grid[0], grid[1], 0, num_steps)
        return out.to(tensor.dtype), (grid, num_steps, c, npc)
    delta, offset, _ = get_computed_encodings(tensor_quantizer.bitwidth, encoding_min.detach().float(),
                                              encoding_max.detach().float(),
                                              tensor_quantizer.use_symmetric_encodings,
                                              tensor_quantizer.use_strict_symmetric,
                                              tensor_quantizer.is_unsigned_symmetric)
    c, npc = _channel_geometry(tensor, delta.numel(), tensor_quantizer.channel_axis)
    out = ops.v2_qdq(x, c, npc, delta, offset, 0, num_steps)
    return out.to(tensor.dtype), (delta, offset, num_steps, c, npc)


def _num_steps(tensor_quantizer) -> int:
    n = 2 ** tensor_quantizer.bitwidth - 1
    if tensor_quantizer.use_symmetric_encodings and tensor_quantizer.use_strict_symmetric:
        n -= 1
    return n


def learned_grid_backward(tensor, grad, saved, encoding_min, encoding_max, is_symmetric, want_tensor_grad,
                          want_encoding_grads):
    """Backward of range learning (reference asymmetric_gradients :253-297, symmetric_gradients :301-331).  One pass
    over (tensor, grad) yields grad * mask and, per channel, S = sum(grad * (x_quant + offset - x * mask / delta)) and
    O = sum(delta * grad * ~mask); then

        asymmetric:  t1 = S / steps, t2 = steps / (max - min)^2 * O
                     d/dmin = -t1 + max * t2,  d/dmax = t1 - min * t2
        symmetric:   d/dmax = S / floor(steps / 2),  d/dmin = -d/dmax
    """
    x = tensor if tensor.dtype != torch.float16 else tensor.float()
    g = grad.to(x.dtype)
    if len(saved) == 4:
        # the library's grid: the encoding gradients leave the kernel that adds up the channel sums
        grid, num_steps, c, npc = saved
        if not want_encoding_grads:
            return ops.v2_qdq_bwd(x, g, c, npc, grid[0], grid[1], 0, num_steps).to(tensor.dtype), None, None
        mode = ops.RANGE_V1_SIGNED_SYMMETRIC if is_symmetric else ops.RANGE_V1_ASYMMETRIC
        tensor_grad, grad_min, grad_max = ops.qdq_bwd_range(x, g, c, npc, grid, 0, num_steps, mode,
                                                            want_grad_in=want_tensor_grad)
        if tensor_grad is not None:
            tensor_grad = tensor_grad.to(tensor.dtype)
        return (tensor_grad, grad_min.to(encoding_min.dtype).view_as(encoding_min),
                grad_max.to(encoding_max.dtype).view_as(encoding_max))
    delta, offset, num_steps, c, npc = saved
    if not want_encoding_grads:
        return ops.v2_qdq_bwd(x, g, c, npc, delta, offset, 0, num_steps).to(tensor.dtype), None, None
    tensor_grad, s_sum, o_sum = ops.v2_qdq_bwd_params(x, g, c, npc, delta, offset, 0, num_steps,
                                                      want_grad_in=want_tensor_grad)
    if tensor_grad is not None:
        tensor_grad = tensor_grad.to(tensor.dtype)
    emin, emax = encoding_min.detach().float().reshape(-1), encoding_max.detach().float().reshape(-1)
    steps = torch.full_like(s_sum, float(num_steps))      # tensors as divisors, as in the reference
    if is_symmetric:
        grad_max = s_sum / torch.full_like(s_sum, float(num_steps // 2))
        grad_min = -grad_max
    else:
        term1 = s_sum / steps
        term2 = steps / (emax - emin) ** 2 * o_sum
        grad_min = -term1 + emax * term2
        grad_max = term1 - emin * term2
    return (tensor_grad, grad_min.to(encoding_min.dtype).view_as(encoding_min),
            grad_max.to(encoding_max.dtype).view_as(encoding_max))
