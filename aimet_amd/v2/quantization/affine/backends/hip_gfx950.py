"""``hip_gfx950``: the v2 affine quantization backend on hand-written HIP kernels.

Same functions, argument meaning and error behaviour as the reference's torch_builtins backend
(TrainingExtensions/torch/src/python/aimet_torch/v2/quantization/affine/backends/torch_builtins.py:52-344):

    quantize            out = clamp(round_half_even(x / scale) - offset, qmin, qmax)
    dequantize          out = (x + offset) * scale
    quantize_dequantize out = (clamp(round_half_even(x / scale) - offset, qmin, qmax) + offset) * scale

The forward of quantize / quantize_dequantize is one fused kernel (the reference runs about seven elementwise ATen
kernels and saves a bool mask); the input gradient is one fused kernel: from a one-bit-per-element mask the forward
wrote when only the input wants a gradient, else recomputing the mask from the saved input.  float32 and bfloat16 tensors are computed in float32, as the reference does for 4- and 8-bit grids; other
float types are upcast to float32.

Scale / offset may be per-tensor, per-channel, vary along several axes, or be blockwise (`block_size`, reference
:347-399).  The kernels index parameters as channel(i) = (i / n_per_channel) % num_channel over the flat tensor, which
covers every layout whose varying axes are adjacent in memory (per-channel along any one axis; blocks cutting the
last varying axis, e.g. weight [out, in] with scale [out, in / block]) without a copy; other layouts take one permuted
copy each way.

Gradients w.r.t. scale and offset (range learning, :329-344) come from one fused pass over the input and the
incoming gradient, together with the input gradient.  For the quantizer modules, whose scale and offset are functions
of a learnable min / max, quantize_dequantize_learned_range() takes min / max themselves and returns their gradients.
"""
import functools
from typing import List, Optional

import torch

from ..... import ops
from ....utils import (_is_expandable, channel_view, channel_view_restore, get_encoding_shape_with_blocks,
                       reshape_tensor_for_blocks)


def _is_value_representable(dtype: torch.dtype, value: int) -> bool:
    r = torch.tensor(value, dtype=dtype)
    return bool(r.isfinite()) and int(r.long()) == value


@functools.lru_cache(maxsize=256)
def _is_grid_representable(dtype: torch.dtype, qmin: int, qmax: int) -> bool:
    return all(_is_value_representable(dtype, v) for v in (qmax, qmax - 1, qmin + 1, qmin))


def _validate_arguments(tensor, scale, offset, qmin=None, qmax=None, block_size=None):
    if block_size is not None:
        if len(scale.shape) != len(block_size):
            raise RuntimeError(f'Length of scale shape {scale.shape} must equal length of block size {block_size}')
        if len(block_size) > tensor.dim():
            raise RuntimeError(f'Block size {block_size} has more dimensions than the tensor of shape {tensor.shape}')
        for i in range(1, len(block_size) + 1):
            if block_size[-i] == -1:
                if tensor.shape[-i] % scale.shape[-i] != 0:
                    raise RuntimeError(f'Each tensor dimension size for tensor shape {tensor.shape} must divide '
                                       f'evenly with corresponding scale dimension value for scale shape '
                                       f'{scale.shape}')
            elif block_size[-i] * scale.shape[-i] != tensor.shape[-i]:
                raise RuntimeError(f'Each tensor dimension size for tensor shape {tensor.shape} must equal the '
                                   f'corresponding scale dimension size * block size for scale shape {scale.shape} '
                                   f'and block size {block_size}')
    elif not _is_expandable(scale.shape, tensor.shape):
        raise RuntimeError(f"Scale of shape {scale.shape} cannot be expanded like input tensor of shape "
                           f"{tensor.shape}")
    if tensor.device != scale.device or tensor.device != offset.device:
        raise RuntimeError(f"Expected all tensors to be on the same device, but found {tensor.device}, "
                           f"{scale.device} and {offset.device}")
    if qmin is not None and qmax is not None and qmin > qmax:
        raise RuntimeError(f"qmin ({qmin}) must be smaller than or equal to qmax ({qmax})")


def _channel_geometry(tensor_shape, scale_shape):
    """(num_channel, n_per_channel) of a tensor laid out [outer, num_channel, n_per_channel] by channel_view."""
    assert len(tensor_shape) == 3 and tuple(scale_shape) == (tensor_shape[1], 1)
    return tensor_shape[1], max(tensor_shape[2], 1)


def _apply_per_channel(func, tensor, scale, offset, qmin, qmax, block_size):
    """Runs an autograd function of (tensor3, scale[C, 1], offset[C, 1]) on the channel layout of the tensor.  The
    re-layout is made of differentiable views / copies, so gradients flow back in the callers' shapes."""
    shape = tensor.shape
    if scale.shape != offset.shape:
        scale, offset = torch.broadcast_tensors(scale, offset)
    expanded = reshape_tensor_for_blocks(tensor, scale.shape, block_size)
    tensor3, perm = channel_view(expanded, get_encoding_shape_with_blocks(scale.shape, block_size))
    c = tensor3.shape[1]
    if func is _QuantDequantFunc and not torch.is_grad_enabled():
        # inference: the same kernel without the autograd.Function machinery around it
        out = ops.v2_qdq(tensor3, c, max(tensor3.shape[2], 1), scale.reshape(c, 1), offset.reshape(c, 1), qmin, qmax)
    else:
        out = func.apply(tensor3, scale.reshape(c, 1), offset.reshape(c, 1), qmin, qmax)
    return channel_view_restore(out, expanded.shape, perm).reshape(shape)


def _geometry_as_it_is(tensor: torch.Tensor, param: torch.Tensor):
    """(num_channel, n_per_channel) of a tensor that _as_it_is() accepts"""
    count = param.numel()
    return count, max(tensor.numel() // count, 1)


def _as_it_is(tensor: torch.Tensor, param: torch.Tensor, block_size) -> bool:
    """True for a contiguous tensor whose parameter is one number, or one number per slice along the first axis (every
    activation and every weight quantized per output channel): memory already is [channel][run], and the reshapes of
    _apply_per_channel -- two view nodes forward, two backward -- have nothing to do."""
    if block_size is not None or not tensor.is_contiguous() or tensor.numel() == 0:
        return False
    count = param.numel()
    if count == 1:
        return True
    shape = param.shape
    return len(shape) == tensor.dim() and shape[0] == tensor.shape[0] == count


def _reduce_like(grad: torch.Tensor, shape) -> torch.Tensor:
    return grad.sum_to_size(shape) if tuple(grad.shape) != tuple(shape) else grad


class _QuantDequantFunc(torch.autograd.Function):
    # When only the input wants a gradient (static scale / offset) the forward writes the backward's mask itself, one
    # bit per element, and keeps that instead of the input; the reference keeps the same mask as a bool tensor, one
    # byte per element (torch_builtins.py:303-327).  False: keep the input and recompute the mask in backward.
    save_mask = True

    @staticmethod
    def forward(ctx, tensor, scale, offset, qmin, qmax, geometry=None):  # pylint: disable=arguments-differ
        # geometry: (channels, elements per channel) of a tensor handed over as it is; None: channel_view's layout
        c, npc = geometry or _channel_geometry(tensor.shape, scale.shape)
        ctx.geom = (c, npc, qmin, qmax)
        ctx.masked = _QuantDequantFunc.save_mask and ctx.needs_input_grad[0] and \
            not (ctx.needs_input_grad[1] or ctx.needs_input_grad[2])
        if ctx.masked:
            out, mask = ops.v2_qdq_mask(tensor, c, npc, scale, offset, qmin, qmax)
            ctx.save_for_backward(mask)
            return out
        out = ops.v2_qdq(tensor, c, npc, scale, offset, qmin, qmax)
        ctx.save_for_backward(tensor, scale, offset)
        return out

    @staticmethod
    def backward(ctx, grad):  # pylint: disable=arguments-differ
        if ctx.masked:
            mask, = ctx.saved_tensors
            return ops.ste_bwd_mask(mask, grad), None, None, None, None, None
        tensor, scale, offset = ctx.saved_tensors
        c, npc, qmin, qmax = ctx.geom
        tensor_grad = scale_grad = offset_grad = None
        if ctx.needs_input_grad[1] or ctx.needs_input_grad[2]:
            # x and grad are read once: tensor_grad and both parameter sums come out of the same pass
            tensor_grad, sg, og = ops.v2_qdq_bwd_params(tensor, grad, c, npc, scale, offset, qmin, qmax,
                                                        want_grad_in=ctx.needs_input_grad[0])
            scale_grad = sg.reshape(scale.shape).to(scale.dtype) if ctx.needs_input_grad[1] else None
            offset_grad = og.reshape(offset.shape).to(offset.dtype) if ctx.needs_input_grad[2] else None
        elif ctx.needs_input_grad[0]:
            tensor_grad = ops.v2_qdq_bwd(tensor, grad, c, npc, scale, offset, qmin, qmax)
        return tensor_grad, scale_grad, offset_grad, None, None, None


class _LearnedRangeFunc(torch.autograd.Function):
    """Quantize-dequantize as a function of (tensor, encoding min, encoding max): the grid is made from min / max by
    one small launch, and backward returns the gradients of min / max straight from the kernel that reduces the
    channel sums -- what autograd otherwise assembles from get_scale() / get_offset(), about ten tensor operations of
    parameter size forward and as many backward, per quantizer and step."""

    @staticmethod
    def forward(ctx, tensor, enc_min, enc_max, qmin, qmax, symmetric, geometry=None):  # pylint: disable=arguments-differ
        c, npc = geometry or (tensor.shape[1], max(tensor.shape[2], 1))
        mode = ops.RANGE_V2_SYMMETRIC if symmetric else ops.RANGE_V2_ASYMMETRIC
        grid = ops.range_to_grid(enc_min.reshape(-1), enc_max.reshape(-1), qmin, qmax, mode)
        ctx.geom = (c, npc, qmin, qmax, mode, enc_min.shape, enc_max.shape)
        ctx.save_for_backward(tensor, grid)
        return ops.v2_qdq(tensor, c, npc, grid[0], grid[1], qmin, qmax)

    @staticmethod
    def backward(ctx, grad):  # pylint: disable=arguments-differ
        tensor, grid = ctx.saved_tensors
        c, npc, qmin, qmax, mode, min_shape, max_shape = ctx.geom
        tensor_grad, grad_min, grad_max = ops.qdq_bwd_range(tensor, grad, c, npc, grid, qmin, qmax, mode,
                                                            want_grad_in=ctx.needs_input_grad[0])
        return tensor_grad, (grad_min.reshape(min_shape) if ctx.needs_input_grad[1] else None), \
            (grad_max.reshape(max_shape) if ctx.needs_input_grad[2] else None), None, None, None, None


def takes_learned_range(tensor: torch.Tensor, enc_min: torch.Tensor, enc_max: torch.Tensor) -> bool:
    """True where quantize_dequantize_learned_range() applies: float32 min / max of one shape, held contiguously on
    the tensor's GPU."""
    return tensor.is_cuda and tensor.is_floating_point() and enc_min.dtype == enc_max.dtype == torch.float32 and \
        enc_min.shape == enc_max.shape and enc_min.device == enc_max.device == tensor.device and \
        enc_min.is_contiguous() and enc_max.is_contiguous() and tensor.numel() > 0


def quantize_dequantize_learned_range(tensor: torch.Tensor, enc_min: torch.Tensor, enc_max: torch.Tensor, qmin: int,
                                      qmax: int, symmetric: bool, block_size: Optional[List] = None) -> torch.Tensor:
    """quantize_dequantize(tensor, scale, offset, ...) with scale = (max - min) / (qmax - qmin) and
    offset = round(min / scale) - qmin (0 for a symmetric quantizer), differentiable w.r.t. tensor, min and max: the
    training-time forward of a quantizer with learnable range (reference affine/quantizer.py:404-436 followed by
    :720-745)."""
    _validate_arguments(tensor, enc_min, enc_max, qmin, qmax, block_size)
    if not _is_grid_representable(torch.float32, qmin, qmax):
        raise RuntimeError(f"{torch.float32} is unable to represent quantized output of range [{qmin}, {qmax}].")
    x, orig = _prepare(tensor, enc_min, enc_max)
    if _as_it_is(x, enc_min, block_size):
        out = _LearnedRangeFunc.apply(x, enc_min, enc_max, qmin, qmax, bool(symmetric),
                                      _geometry_as_it_is(x, enc_min))
        return out.to(orig) if orig is not None else out
    shape = x.shape
    expanded = reshape_tensor_for_blocks(x, enc_min.shape, block_size)
    tensor3, perm = channel_view(expanded, get_encoding_shape_with_blocks(enc_min.shape, block_size))
    out = _LearnedRangeFunc.apply(tensor3, enc_min, enc_max, qmin, qmax, bool(symmetric))
    out = channel_view_restore(out, expanded.shape, perm).reshape(shape)
    return out.to(orig) if orig is not None else out


class _QuantizeFunc(torch.autograd.Function):
    @staticmethod
    def forward(ctx, tensor, scale, offset, qmin, qmax):  # pylint: disable=arguments-differ
        c, npc = _channel_geometry(tensor.shape, scale.shape)
        x = tensor.to(torch.float32)
        _, codes = ops.v2_qdq(x, c, npc, scale, offset, qmin, qmax, want_codes=True)
        ctx.geom = (c, npc, qmin, qmax)
        ctx.save_for_backward(tensor, scale, offset)
        return codes.to(tensor.dtype)

    @staticmethod
    def backward(ctx, grad):  # pylint: disable=arguments-differ
        tensor, scale, offset = ctx.saved_tensors
        c, npc, qmin, qmax = ctx.geom
        # torch_builtins.py:236-246: masked_grad = grad * mask; d/dx = masked / scale;
        # d/dscale = -(masked / scale) * (x / scale); d/doffset = -masked
        masked = ops.v2_qdq_bwd(tensor.to(torch.float32), grad.to(torch.float32), c, npc, scale, offset, qmin, qmax)
        s = scale.to(torch.float32)
        tensor_grad = (masked / s).to(tensor.dtype) if ctx.needs_input_grad[0] else None
        scale_grad = _reduce_like(-(masked / s) * (tensor.to(torch.float32) / s), scale.shape).to(scale.dtype) \
            if ctx.needs_input_grad[1] else None
        offset_grad = _reduce_like(-masked, offset.shape).to(offset.dtype) if ctx.needs_input_grad[2] else None
        return tensor_grad, scale_grad, offset_grad, None, None


def _prepare(tensor, scale, offset):
    if not tensor.is_cuda:
        raise RuntimeError("the hip_gfx950 backend computes on the GPU only; got a tensor on " + str(tensor.device))
    if tensor.dtype not in (torch.float32, torch.bfloat16):
        if not tensor.is_floating_point():
            raise RuntimeError(f"expected a floating point tensor, got {tensor.dtype}")
        return tensor.to(torch.float32), tensor.dtype
    return tensor, None


def quantize(tensor: torch.Tensor, scale: torch.Tensor, offset: torch.Tensor, qmin: int, qmax: int,
             block_size: Optional[List] = None) -> torch.Tensor:
    """Differentiable quantization: integer-valued output in the input's dtype."""
    _validate_arguments(tensor, scale, offset, qmin, qmax, block_size)
    if not _is_grid_representable(tensor.dtype, qmin, qmax):
        raise RuntimeError(f"{tensor.dtype} is unable to represent quantized output of range [{qmin}, {qmax}].")
    x, orig = _prepare(tensor, scale, offset)
    out = _apply_per_channel(_QuantizeFunc, x, scale, offset, qmin, qmax, block_size)
    return out.to(orig) if orig is not None else out


def quantize_dequantize(tensor: torch.Tensor, scale: torch.Tensor, offset: torch.Tensor, qmin: int, qmax: int,
                        block_size: Optional[List] = None) -> torch.Tensor:
    """Differentiable quantize-dequantize (fake quantization)."""
    if block_size is None and not torch.is_grad_enabled() and scale.numel() == 1 and offset.numel() == 1 and \
            tensor.is_cuda and tensor.dtype in (torch.float32, torch.bfloat16) and tensor.is_contiguous() and \
            tensor.numel() > 0 and scale.device == tensor.device and offset.device == tensor.device and qmin <= qmax and \
            _is_grid_representable(torch.float32, qmin, qmax):
        # inference with one scale for the whole tensor (every activation quantizer): none of the re-layout below has
        # anything to do, and every check it makes has just been made
        return ops.v2_qdq(tensor, 1, tensor.numel(), scale, offset, qmin, qmax)
    _validate_arguments(tensor, scale, offset, qmin, qmax, block_size)
    if not _is_grid_representable(torch.float32, qmin, qmax):
        raise RuntimeError(f"{torch.float32} is unable to represent quantized output of range [{qmin}, {qmax}].")
    x, orig = _prepare(tensor, scale, offset)
    if scale.shape == offset.shape and _as_it_is(x, scale, block_size) and torch.is_grad_enabled():
        out = _QuantDequantFunc.apply(x, scale, offset, qmin, qmax, _geometry_as_it_is(x, scale))
    else:
        out = _apply_per_channel(_QuantDequantFunc, x, scale, offset, qmin, qmax, block_size)
    return out.to(orig) if orig is not None else out


def dequantize(tensor: torch.Tensor, scale: torch.Tensor, offset: torch.Tensor,
               block_size: Optional[List] = None) -> torch.Tensor:
    """(x + offset) * scale on an already quantized tensor; not a hot op (two elementwise tensor ops)."""
    _validate_arguments(tensor, scale, offset, block_size=block_size)
    shape = tensor.shape
    expanded = reshape_tensor_for_blocks(tensor, scale.shape, block_size)
    pshape = get_encoding_shape_with_blocks(scale.shape, block_size)
    out = (expanded + offset.to(tensor.dtype).reshape(pshape)) * scale.to(tensor.dtype).reshape(pshape)
    return out.reshape(shape)
