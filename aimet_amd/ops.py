"""Tensor-level entry points over the libmiq C ABI.

Every function takes CUDA(HIP) tensors, launches on torch's *current* stream of the tensor's device and returns
without synchronising (except the analyzer read-backs, which must).  torch is used for device memory and streams
only; there is no torch-op fallback: tensors that are not on a GPU are rejected.
"""
import ctypes as C

import numpy as np
import torch

from . import _lib
from ._lib import Encoding, check, lib

_F32, _BF16 = torch.float32, torch.bfloat16


# torch.cuda.current_stream() builds a Stream object (about 3 us per call, as much as queueing a kernel); the raw
# handle of the same stream is available without it
_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)  # pylint: disable=protected-access


def _stream_of(device):
    """HIP stream handle (an integer) of torch's current stream on `device`."""
    if _raw_stream is not None and device.index is not None:
        return _raw_stream(device.index)
    return torch.cuda.current_stream(device).cuda_stream


def _stream(t):
    return _stream_of(t.device)


current_stream_handle = _stream_of


class _OnDevice:
    """`with torch.cuda.device(d)` only when d is not already the current device: the context manager costs several
    microseconds per call, as much as queueing the kernel, and the devices nearly always agree."""
    __slots__ = ("_guard",)

    def __init__(self, device):
        self._guard = None
        if device.index is not None and device.index != torch.cuda.current_device():
            self._guard = torch.cuda.device(device)

    def __enter__(self):
        if self._guard is not None:
            self._guard.__enter__()

    def __exit__(self, *exc):
        if self._guard is not None:
            self._guard.__exit__(*exc)
        return False


def _ptr(t):
    # (a plain integer converts to a void* argument without building a ctypes object)
    return t.data_ptr() if t is not None else None


def _require_gpu(*tensors):
    """Every tensor given lives on one GPU (Tensor.get_device() is an int, -1 off the GPU: no device objects built)."""
    index = tensors[0].get_device()
    for t in tensors:
        if t is None:
            continue
        i = t.get_device()
        if i != index or i < 0:
            if not t.is_cuda:
                raise RuntimeError("aimet_amd kernels run on the GPU only; got a tensor on " + str(t.device))
            raise RuntimeError(f"tensors are on different devices: {t.device} vs {tensors[0].device}")


def _suffix(t):
    if t.dtype == _F32:
        return "f32"
    if t.dtype == _BF16:
        return "bf16"
    raise RuntimeError(f"unsupported dtype {t.dtype}: float32 and bfloat16 are implemented")


def _params_f32(t, like):
    if t.dtype is _F32 and t.is_contiguous() and t.get_device() == like.get_device():
        return t
    return t.to(device=like.device, dtype=_F32).contiguous()


# ---------------------------------------------------------------------------------------------------------- host math
def fill_encoding_info(bw, enc_min, enc_max):
    e = Encoding()
    check(lib.miq_fill_encoding_info(int(bw), float(enc_min), float(enc_max), C.byref(e)))
    return e


def get_computed_encodings(bw, mn, mx, symmetric, strict_symmetric, unsigned_symmetric):
    e = Encoding()
    check(lib.miq_get_computed_encodings(int(bw), float(mn), float(mx), int(symmetric), int(strict_symmetric),
                                         int(unsigned_symmetric), C.byref(e)))
    return e


# ------------------------------------------------------------------------------------------------------------ v1 QDQ
def set_stochastic_seed(seed: int):
    """Seed of the stochastic rounding mode (the counterpart of srand for the reference's CPU path); restarts the
    library's count of stochastic launches."""
    check(lib.miq_set_stochastic_seed(int(seed) & 0xFFFFFFFFFFFFFFFF))


def stochastic_state():
    """(seed, number of stochastic launches since the seed was set)."""
    seed, calls = C.c_uint64(), C.c_uint64()
    check(lib.miq_get_stochastic_state(C.byref(seed), C.byref(calls)))
    return seed.value, calls.value


def qdq_per_tensor(x, enc_min, enc_max, bw, rounding_mode=_lib.ROUND_NEAREST, out=None):
    """DlQuantization per-tensor quantize-dequantize; float32 or bfloat16 storage, float32 arithmetic."""
    _require_gpu(x, out)
    x = x.contiguous()
    out = torch.empty_like(x) if out is None else out
    fn = getattr(lib, "miq_qdq_per_tensor_" + _suffix(x))
    with _OnDevice(x.device):
        check(fn(_ptr(x), _ptr(out), x.numel(), float(enc_min), float(enc_max), int(bw), int(rounding_mode),
                 _stream(x)))
    return out


def fp16_round_trip(x, out=None):
    """float(half(x)) in one pass over a float32 tensor: the float16 data type of the simulation."""
    _require_gpu(x, out)
    if x.dtype != _F32:
        raise RuntimeError("fp16_round_trip takes float32 tensors")
    x = x.contiguous()
    out = torch.empty_like(x) if out is None else out
    with _OnDevice(x.device):
        check(lib.miq_fp16_round_trip_f32(_ptr(x), _ptr(out), x.numel(), _stream(x)))
    return out


def float_grid(maxval, exponent_bits: int, mantissa_bits: int, host_constants: bool = False, host_bias=None):
    """(maxval, bias, steps) device tensors that describe the float grid of `exponent_bits` and `mantissa_bits` ending at
    `maxval` (a one-element tensor, or one value per channel): bias of the format, and for every channel the step
    2^((e - M) - bias) of each exponent e = 0 .. 2^E, all in float32 as the reference's expression evaluates them
    (aimet_torch/fp_quantization.py:171-209).  Reusable for as long as maxval does not change.

    The expression meets its constants in two ways.  The v1 path passes the mantissa bits as a device tensor, so
    2^E and log2(2 - 2^-M) are torch float32 results (the default here).  The v2 float quantizer passes Python
    numbers: log2(2 - 2^-M) is then numpy's float64 value, rounded to float32 where it meets the tensor
    (`host_constants`), and when maxval too is a Python number the whole bias is a float64 that is rounded once
    (`host_bias` = that number)."""
    if not isinstance(maxval, torch.Tensor) or not maxval.is_cuda:
        raise RuntimeError("maxval must be a tensor on the GPU")
    if not 1 <= exponent_bits <= 8 or mantissa_bits < 1:
        raise RuntimeError("float grids take 1 to 8 exponent bits and at least one mantissa bit")
    maxval = maxval.detach().to(_F32).reshape(-1).contiguous()
    key = (maxval.device, exponent_bits, mantissa_bits)
    if key not in _FLOAT_GRID_CONSTANTS:
        m = torch.tensor([float(mantissa_bits)], dtype=_F32, device=maxval.device)
        e = torch.tensor([float(exponent_bits)], dtype=_F32, device=maxval.device)
        exponents = torch.arange((1 << exponent_bits) + 1, dtype=_F32, device=maxval.device)
        # 2^E, log2(2 - 2^-M) and e - M, each as torch's float32 kernels on this device give them
        _FLOAT_GRID_CONSTANTS[key] = (2 ** e, torch.log2(2 - 2 ** (-m)), exponents - m)
    two_to_e, log2_top, e_minus_m = _FLOAT_GRID_CONSTANTS[key]
    # the bias of the format follows from its largest value: maxval = (2 - 2^-M) * 2^(2^E - 1 - bias)
    if host_bias is not None:
        bias = torch.full_like(maxval, float(host_bias))
    elif host_constants:
        bias = (2 ** exponent_bits - torch.log2(maxval) + float(np.log2(2 - 2 ** (-mantissa_bits))) - 1).contiguous()
    else:
        bias = (two_to_e - torch.log2(maxval) + log2_top - 1).contiguous()
    steps = (2. ** (e_minus_m.unsqueeze(0) - bias.unsqueeze(1))).contiguous()
    return maxval, bias, steps


def fp8_grid(maxval, mantissa_bits: int = 3):
    """float_grid() of the 8-bit format with `mantissa_bits` mantissa and 7 - mantissa_bits exponent bits."""
    return float_grid(maxval, 7 - mantissa_bits, mantissa_bits)


_FLOAT_GRID_CONSTANTS = {}


def float_fake_cast(x, maxval, exponent_bits: int, mantissa_bits: int, ch_axis: int = 0, out=None, grid=None):
    """Rounds a float32 tensor to the float grid of `exponent_bits` (1 to 8) and `mantissa_bits` whose largest value is
    `maxval`: a one-element tensor for the whole tensor, or a 1-d tensor with one value per channel along `ch_axis`
    (reference aimet_torch/fp_quantization.py:171-209, fake_cast_to_ieee_float).  `grid` = float_grid(maxval,
    exponent_bits, mantissa_bits) computed earlier saves recomputing it."""
    _require_gpu(x, out)
    if x.dtype != _F32:
        raise RuntimeError("float_fake_cast takes float32 tensors")
    x = x.contiguous()
    if grid is None:
        grid = float_grid(torch.as_tensor(maxval, dtype=_F32, device=x.device), exponent_bits, mantissa_bits)
    maxval, bias, steps = grid
    channels = maxval.numel()
    inner = x.numel()
    if channels > 1:
        if x.dim() <= ch_axis or x.shape[ch_axis] != channels:
            raise RuntimeError(f"maxval has {channels} entries but dimension {ch_axis} of the tensor has "
                               f"{x.shape[ch_axis] if x.dim() > ch_axis else 'no'} channels")
        inner = 1
        for d in x.shape[ch_axis + 1:]:
            inner *= d
    out = torch.empty_like(x) if out is None else out
    with _OnDevice(x.device):
        check(lib.miq_float_fake_cast_f32(_ptr(x), _ptr(out), x.numel(), channels, max(inner, 1), _ptr(maxval),
                                          _ptr(bias), _ptr(steps), steps.shape[1], _stream(x)))
    return out


def fp8_fake_cast(x, maxval, mantissa_bits: int = 3, ch_axis: int = 0, out=None, grid=None):
    """float_fake_cast() on the 8-bit grid with `mantissa_bits` mantissa and 7 - mantissa_bits exponent bits
    (reference aimet_torch/fp_quantization.py:133-169, quantize_to_fp8)."""
    if not 1 <= mantissa_bits <= 6:
        raise RuntimeError("mantissa_bits must be in [1, 6]")
    return float_fake_cast(x, maxval, 7 - mantissa_bits, mantissa_bits, ch_axis, out, grid)


def bf16_round_trip(x, out=None):
    """float(bfloat16(x)) for a float32 tensor, in one pass."""
    _require_gpu(x, out)
    if x.dtype != _F32:
        raise RuntimeError("bf16_round_trip takes float32 tensors")
    x = x.contiguous()
    out = torch.empty_like(x) if out is None else out
    with _OnDevice(x.device):
        check(lib.miq_bf16_round_trip_f32(_ptr(x), _ptr(out), x.numel(), _stream(x)))
    return out


def quantize_per_tensor(x, enc_min, enc_max, bw, shift_to_signed, rounding_mode=_lib.ROUND_NEAREST):
    """Float-valued grid indices (minus 2^(bw-1) when shift_to_signed)."""
    _require_gpu(x)
    x = x.to(_F32).contiguous()
    out = torch.empty_like(x)
    with _OnDevice(x.device):
        check(lib.miq_quantize_per_tensor_f32(_ptr(x), _ptr(out), x.numel(), float(enc_min), float(enc_max), int(bw),
                                              int(rounding_mode), int(bool(shift_to_signed)), _stream(x)))
    return out


def qdq_codes_per_tensor(x, enc_min, enc_max, bw, shift_to_signed=False, want_dequant=True):
    """One pass producing (dequantized or None, byte codes): uint8 grid index, or int8 when shift_to_signed."""
    _require_gpu(x)
    x = x.to(_F32).contiguous()
    out = torch.empty_like(x) if want_dequant else None
    codes = torch.empty(x.shape, dtype=torch.int8 if shift_to_signed else torch.uint8, device=x.device)
    with _OnDevice(x.device):
        check(lib.miq_qdq_codes_per_tensor_f32(_ptr(x), _ptr(out), _ptr(codes), x.numel(), float(enc_min),
                                               float(enc_max), int(bw), int(bool(shift_to_signed)), _stream(x)))
    return out, codes


def tf_encodings_per_channel(minmax, bw, symmetric, strict_symmetric, unsigned_symmetric):
    """minmax: float32 GPU tensor [2, C] of per-channel running minima and maxima.  Returns (enc, params): enc a
    float64 GPU tensor [C, 4] = (min, max, delta, offset) of every channel's TF encoding, params the six float32
    vectors (min, max, delta, offset, raw_min, raw_max) the per-channel kernels take.  Nothing waits for the device."""
    _require_gpu(minmax)
    if minmax.dtype != _F32 or minmax.dim() != 2 or minmax.size(0) != 2 or not minmax.is_contiguous():
        raise RuntimeError("minmax must be a contiguous float32 tensor [2, C]")
    c = minmax.size(1)
    enc = torch.empty(c, 4, dtype=torch.float64, device=minmax.device)
    outs = torch.empty(6, c, dtype=_F32, device=minmax.device)
    with _OnDevice(minmax.device):
        check(lib.miq_tf_encodings_per_channel_f32(_ptr(minmax[0]), _ptr(minmax[1]), c, int(bw), int(bool(symmetric)),
                                                   int(bool(strict_symmetric)), int(bool(unsigned_symmetric)),
                                                   _ptr(enc), *(_ptr(outs[k]) for k in range(6)), _stream(minmax)))
    return enc, tuple(outs[k] for k in range(6))


def per_channel_params(enc_min, enc_max, num_steps):
    """(min, max, delta, offset) float32 device vectors from raw per-channel min/max (float32 tensors on the GPU)."""
    _require_gpu(enc_min, enc_max)
    enc_min, enc_max = enc_min.to(_F32).contiguous(), enc_max.to(_F32).contiguous()
    c = enc_min.numel()
    outs = torch.empty(4, c, dtype=_F32, device=enc_min.device)
    with _OnDevice(enc_min.device):
        check(lib.miq_per_channel_params_f32(_ptr(enc_min), _ptr(enc_max), c, float(num_steps), _ptr(outs[0]),
                                             _ptr(outs[1]), _ptr(outs[2]), _ptr(outs[3]), _stream(enc_min)))
    return outs[0], outs[1], outs[2], outs[3]


def qdq_per_channel(x, num_channel, n_per_channel, mn, mx, delta, offset, rounding_mode=_lib.ROUND_NEAREST,
                    out=None):
    _require_gpu(x, mn, mx, delta, offset, out)
    x = x.contiguous()
    out = torch.empty_like(x) if out is None else out
    fn = getattr(lib, "miq_qdq_per_channel_" + _suffix(x))
    mn, mx, delta, offset = (_params_f32(p, x) for p in (mn, mx, delta, offset))
    with _OnDevice(x.device):
        check(fn(_ptr(x), _ptr(out), int(num_channel), x.numel(), int(n_per_channel), _ptr(mn), _ptr(mx),
                 _ptr(delta), _ptr(offset), int(rounding_mode), _stream(x)))
    return out


def qdq_codes_per_channel(x, num_channel, n_per_channel, mn, mx, delta, offset, bw, shift_to_signed=False,
                          want_dequant=True):
    _require_gpu(x, mn, mx, delta, offset)
    x = x.to(_F32).contiguous()
    out = torch.empty_like(x) if want_dequant else None
    codes = torch.empty(x.shape, dtype=torch.int8 if shift_to_signed else torch.uint8, device=x.device)
    mn, mx, delta, offset = (_params_f32(p, x) for p in (mn, mx, delta, offset))
    with _OnDevice(x.device):
        check(lib.miq_qdq_codes_per_channel_f32(_ptr(x), _ptr(out), _ptr(codes), int(num_channel), x.numel(),
                                                int(n_per_channel), _ptr(mn), _ptr(mx), _ptr(delta), _ptr(offset),
                                                int(bool(shift_to_signed)), int(bw), _stream(x)))
    return out, codes


def qdq_broadcast(x, input_strides, encoding_strides, mn, mx, delta, offset):
    _require_gpu(x, mn, mx, delta, offset)
    x = x.to(_F32).contiguous()
    out = torch.empty_like(x)
    nd = len(input_strides)
    ist = (C.c_int64 * nd)(*[int(v) for v in input_strides])
    est = (C.c_int64 * nd)(*[int(v) for v in encoding_strides])
    mn, mx, delta, offset = (_params_f32(p, x) for p in (mn, mx, delta, offset))
    with _OnDevice(x.device):
        check(lib.miq_qdq_broadcast_f32(_ptr(x), _ptr(out), x.numel(), nd, ist, est, _ptr(mn), _ptr(mx), _ptr(delta),
                                        _ptr(offset), _stream(x)))
    return out


def ste_bwd_per_tensor(x, grad_out, enc_min, enc_max, out=None):
    _require_gpu(x, grad_out, out)
    x, grad_out = x.contiguous(), grad_out.to(x.dtype).contiguous()
    gin = torch.empty_like(x) if out is None else out
    fn = getattr(lib, "miq_ste_bwd_per_tensor_" + _suffix(x))
    with _OnDevice(x.device):
        check(fn(_ptr(x), _ptr(grad_out), _ptr(gin), x.numel(), float(enc_min), float(enc_max), _stream(x)))
    return gin


def ste_bwd_per_channel(x, grad_out, num_channel, n_per_channel, enc_min, enc_max, out=None):
    _require_gpu(x, grad_out, enc_min, enc_max, out)
    x, grad_out = x.contiguous(), grad_out.to(x.dtype).contiguous()
    gin = torch.empty_like(x) if out is None else out
    fn = getattr(lib, "miq_ste_bwd_per_channel_" + _suffix(x))
    enc_min, enc_max = _params_f32(enc_min, x), _params_f32(enc_max, x)
    with _OnDevice(x.device):
        check(fn(_ptr(x), _ptr(grad_out), _ptr(gin), int(num_channel), x.numel(), int(n_per_channel), _ptr(enc_min),
                 _ptr(enc_max), _stream(x)))
    return gin


# ---------------------------------------------------------------------------------------- several tensors, one launch
class QdqMulti:
    """A prepared quantize-dequantize of several tensors in one launch (nearest rounding, v1 arithmetic).

    entries: (x, num_channel, n_per_channel, enc_min, enc_max, enc_delta, enc_offset) with x a contiguous float32 (or
    all bfloat16) GPU tensor and the four parameter vectors as qdq_per_channel takes them (one-element vectors for a
    per-tensor encoding).  Outputs are allocated once (`outputs`, same order) and rewritten by every call.  Raises
    RuntimeError when an entry cannot take part (tiny channels, unaligned data): quantize that one by itself."""
    MAX_SEGMENTS = 256

    def __init__(self, entries, outputs=None):
        entries = list(entries)
        if not 1 <= len(entries) <= self.MAX_SEGMENTS:
            raise RuntimeError(f"1 .. {self.MAX_SEGMENTS} tensors per launch")
        first = entries[0][0]
        _require_gpu(*[t for e in entries for t in (e[0],) + tuple(e[3:7])])
        self.device = first.device
        self._suffix = _suffix(first)
        self.outputs = [torch.empty_like(e[0]) for e in entries] if outputs is None else list(outputs)
        self._keep = []
        table = (_lib.QdqSegment * len(entries))()
        for seg, entry, out in zip(table, entries, self.outputs):
            x, c, npc = entry[0], int(entry[1]), int(entry[2])
            if x.dtype != first.dtype or not x.is_contiguous() or out.shape != x.shape or out.dtype != x.dtype:
                raise RuntimeError("the tensors of one launch share a dtype and are contiguous")
            params = [_params_f32(p, x).reshape(-1) for p in entry[3:7]]
            if any(p.numel() != c for p in params):
                raise RuntimeError("parameter vectors must hold one value per channel")
            self._keep.append((x, out, params))
            seg.in_, seg.out, seg.num_element, seg.num_channel, seg.num_element_per_channel = \
                x.data_ptr(), out.data_ptr(), x.numel(), c, npc
            seg.enc_min, seg.enc_max, seg.enc_delta, seg.enc_offset = (p.data_ptr() for p in params)
        self._tiles = int(lib.miq_qdq_multi_plan(table, len(entries), first.element_size()))
        if self._tiles < 0:
            raise _lib.MiqError(lib.miq_last_error().decode())
        self._count = len(entries)
        self.elements = sum(e[0].numel() for e in entries)
        host = torch.frombuffer(bytearray(bytes(table)), dtype=torch.uint8)
        self._table = host.to(self.device)
        self._fn = getattr(lib, "miq_qdq_per_channel_multi_" + self._suffix)

    def __call__(self):
        with _OnDevice(self.device):
            check(self._fn(self._table.data_ptr(), self._count, self._tiles, _stream_of(self.device)))
        return self.outputs


# ------------------------------------------------------------------------------------- saved straight-through mask
def _new_mask(x):
    """Device buffer for the one-bit-per-element straight-through mask of `x` (int64 words, never initialised: the
    forward writes every word the backward reads)."""
    nbytes = int(lib.miq_ste_mask_bytes(x.numel(), x.element_size()))
    return torch.empty(nbytes // 8, dtype=torch.int64, device=x.device)


def _out_and_mask(x, out, mask):
    if mask is not None and (mask.dtype != torch.int64 or
                             mask.numel() * 8 != int(lib.miq_ste_mask_bytes(x.numel(), x.element_size()))):
        raise RuntimeError("the mask buffer does not fit a tensor of this size and dtype")
    return (torch.empty_like(x) if out is None else out), (_new_mask(x) if mask is None else mask)


def qdq_mask_per_tensor(x, enc_min, enc_max, bw, mask_min=None, mask_max=None, out=None, mask=None):
    """qdq_per_tensor (nearest rounding) that also returns the mask ste_bwd_mask multiplies the gradient with:
    mask_min <= x <= mask_max, by default the encoding's bounds as ste_bwd_per_tensor would take them."""
    _require_gpu(x, out, mask)
    x = x.contiguous()
    out, mask = _out_and_mask(x, out, mask)
    fn = getattr(lib, "miq_qdq_mask_per_tensor_" + _suffix(x))
    mask_min = float(enc_min) if mask_min is None else float(mask_min)
    mask_max = float(enc_max) if mask_max is None else float(mask_max)
    with _OnDevice(x.device):
        check(fn(_ptr(x), _ptr(out), _ptr(mask), x.numel(), float(enc_min), float(enc_max), int(bw), mask_min,
                 mask_max, _stream(x)))
    return out, mask


def qdq_mask_per_channel(x, num_channel, n_per_channel, mn, mx, delta, offset, raw_min, raw_max, out=None, mask=None):
    """qdq_per_channel (nearest rounding) + mask; raw_min / raw_max are the stored encodings' bounds, the ones
    ste_bwd_per_channel compares with."""
    _require_gpu(x, mn, mx, delta, offset, raw_min, raw_max, out, mask)
    x = x.contiguous()
    out, mask = _out_and_mask(x, out, mask)
    fn = getattr(lib, "miq_qdq_mask_per_channel_" + _suffix(x))
    raw_min, raw_max = _params_f32(raw_min, x), _params_f32(raw_max, x)
    with _OnDevice(x.device):
        check(fn(_ptr(x), _ptr(out), _ptr(mask), int(num_channel), x.numel(), int(n_per_channel), _ptr(mn), _ptr(mx),
                 _ptr(delta), _ptr(offset), _ptr(raw_min), _ptr(raw_max), _stream(x)))
    return out, mask


def v2_qdq_mask(x, num_channel, n_per_channel, scale, offset, qmin, qmax, out=None, mask=None):
    """v2_qdq + the mask of its backward (qmin <= round(x / scale) - offset <= qmax)."""
    _require_gpu(x, scale, offset)
    x = x.contiguous()
    scale, offset = _params_f32(scale, x).reshape(-1), _params_f32(offset, x).reshape(-1)
    out, mask = _out_and_mask(x, out, mask)
    fn = getattr(lib, "miq_v2_qdq_mask_" + _suffix(x))
    with _OnDevice(x.device):
        check(fn(_ptr(x), _ptr(out), _ptr(mask), int(num_channel), x.numel(), int(n_per_channel), _ptr(scale),
                 _ptr(offset), int(qmin), int(qmax), _stream(x)))
    return out, mask


def ste_bwd_mask(mask, grad_out, out=None):
    """grad_out * bit, from the mask a *_mask forward wrote for a tensor of grad_out's dtype and element count."""
    _require_gpu(grad_out, mask, out)
    grad_out = grad_out.contiguous()
    if mask.dtype != torch.int64 or mask.numel() * 8 != int(lib.miq_ste_mask_bytes(grad_out.numel(),
                                                                                   grad_out.element_size())):
        raise RuntimeError("the mask does not belong to a tensor of this size and dtype")
    gin = torch.empty_like(grad_out) if out is None else out
    fn = getattr(lib, "miq_ste_bwd_mask_" + _suffix(grad_out))
    with _OnDevice(grad_out.device):
        check(fn(_ptr(mask), _ptr(grad_out), _ptr(gin), grad_out.numel(), _stream(grad_out)))
    return gin


# ------------------------------------------------------------------------------------------------------------ v2 QDQ
def v2_qdq(x, num_channel, n_per_channel, scale, offset, qmin, qmax, want_codes=False):
    _require_gpu(x, scale, offset)
    x = x.contiguous()
    scale, offset = _params_f32(scale, x).reshape(-1), _params_f32(offset, x).reshape(-1)
    out = torch.empty_like(x)
    with _OnDevice(x.device):
        if x.dtype == _F32:
            codes = torch.empty(x.shape, dtype=torch.int32, device=x.device) if want_codes else None
            check(lib.miq_v2_qdq_f32(_ptr(x), _ptr(out), _ptr(codes), int(num_channel), x.numel(), int(n_per_channel),
                                     _ptr(scale), _ptr(offset), int(qmin), int(qmax), _stream(x)))
            return (out, codes) if want_codes else out
        if x.dtype == _BF16 and not want_codes:
            check(lib.miq_v2_qdq_bf16(_ptr(x), _ptr(out), int(num_channel), x.numel(), int(n_per_channel),
                                      _ptr(scale), _ptr(offset), int(qmin), int(qmax), _stream(x)))
            return out
    raise RuntimeError(f"unsupported dtype {x.dtype} for v2 quantize-dequantize")


def v2_qdq_bwd(x, grad_out, num_channel, n_per_channel, scale, offset, qmin, qmax):
    _require_gpu(x, grad_out, scale, offset)
    x, grad_out = x.contiguous(), grad_out.to(x.dtype).contiguous()
    scale, offset = _params_f32(scale, x).reshape(-1), _params_f32(offset, x).reshape(-1)
    gin = torch.empty_like(x)
    fn = getattr(lib, "miq_v2_qdq_bwd_" + _suffix(x))
    with _OnDevice(x.device):
        check(fn(_ptr(x), _ptr(grad_out), _ptr(gin), int(num_channel), x.numel(), int(n_per_channel), _ptr(scale),
                 _ptr(offset), int(qmin), int(qmax), _stream(x)))
    return gin


def v2_qdq_bwd_params(x, grad_out, num_channel, n_per_channel, scale, offset, qmin, qmax, want_grad_in=True):
    """(grad_in or None, scale_grad[C], offset_grad[C]) of the v2 quantize-dequantize in one pass; float32 sums."""
    _require_gpu(x, grad_out, scale, offset)
    x, grad_out = x.contiguous(), grad_out.to(x.dtype).contiguous()
    scale, offset = _params_f32(scale, x).reshape(-1), _params_f32(offset, x).reshape(-1)
    c, npc = int(num_channel), int(n_per_channel)
    gin = torch.empty_like(x) if want_grad_in else None
    grads = torch.empty(2, c, dtype=_F32, device=x.device)
    ws = torch.empty(int(lib.miq_v2_qdq_bwd_params_workspace_bytes(c, x.numel(), npc)), dtype=torch.uint8,
                     device=x.device)
    fn = getattr(lib, "miq_v2_qdq_bwd_params_" + _suffix(x))
    with _OnDevice(x.device):
        check(fn(_ptr(x), _ptr(grad_out), _ptr(gin) if want_grad_in else None, c, x.numel(), npc, _ptr(scale),
                 _ptr(offset), int(qmin), int(qmax), _ptr(grads[0]), _ptr(grads[1]), _ptr(ws), _stream(x)))
    return gin, grads[0], grads[1]


def adaround_recon_grad(out, target_all, index, activation):
    """dLoss/dout of AdaRound's reconstruction loss, (act(out) - act(target_all[index])) * 2 / (elements per channel)
    [* (act(out) > 0) under ReLU], in one pass: `out` [batch, ...] float32 layer output, `target_all` the cached
    float32 outputs of all samples [samples, ...], `index` int64 device tensor of `batch` sample numbers (None: the
    first `batch` samples), activation 0 (none) or 1 (ReLU)."""
    _require_gpu(out, target_all)
    if out.dtype != _F32 or target_all.dtype != _F32 or not out.is_contiguous() or not target_all.is_contiguous():
        raise ValueError("out and target_all must be contiguous float32 tensors")
    batch = out.shape[0]
    per_sample = out.numel() // max(batch, 1)
    if tuple(out.shape[1:]) != tuple(target_all.shape[1:]):
        raise ValueError(f"a sample of out is {tuple(out.shape[1:])}, of target_all {tuple(target_all.shape[1:])}")
    if index is not None:
        _require_gpu(index)
        if index.dtype != torch.int64 or index.numel() != batch or not index.is_contiguous():
            raise ValueError("index must hold one int64 sample number per row of out")
    grad = torch.empty_like(out)
    scale = 2.0 / (out.numel() // out.shape[1]) if out.numel() else 0.0
    with _OnDevice(out.device):
        check(lib.miq_adaround_recon_grad_f32(_ptr(out), _ptr(target_all), _ptr(index) if index is not None else None,
                                              batch, target_all.shape[0], per_sample, int(activation), scale,
                                              _ptr(grad), _stream(out)))
    return grad


# ---------------------------------------------------------------------------------------------------- sequential MSE
COLUMN_ERROR_SQUARED, COLUMN_ERROR_ABSOLUTE, COLUMN_ERROR_SQUARED_AND_SIGNAL = range(3)


def column_error(a, b, kind):
    """Per block and column, an error between `a` and `b` ([blocks, rows, cols] float32, contiguous) summed over rows,
    both read once: squared (kind 0) or absolute (kind 1) differences -> [blocks, cols]; kind 2 -> [2, blocks, cols],
    the squared differences and the squares of `b`."""
    _require_gpu(a, b)
    if a.dtype != _F32 or b.dtype != _F32 or a.dim() != 3 or a.shape != b.shape or not a.is_contiguous() \
            or not b.is_contiguous():
        raise ValueError("a and b must be contiguous float32 tensors of one shape [blocks, rows, cols]")
    blocks, rows, cols = a.shape
    planes = 2 if kind == COLUMN_ERROR_SQUARED_AND_SIGNAL else 1
    if a.numel() == 0:
        return a.new_zeros((planes, blocks, cols) if planes == 2 else (blocks, cols))
    splits = lib.miq_column_error_splits(blocks, rows, cols)
    partial = torch.empty((splits, planes, blocks, cols), dtype=_F32, device=a.device)
    with _OnDevice(a.device):
        check(lib.miq_column_error_f32(_ptr(a), _ptr(b), blocks, rows, cols, int(kind), splits, _ptr(partial),
                                       _stream(a)))
    total = partial[0] if splits == 1 else partial.sum(0)
    return total if planes == 2 else total[0]


# ---------------------------------------------------------------------------------------------------- range learning
RANGE_V2_ASYMMETRIC, RANGE_V2_SYMMETRIC, RANGE_V1_ASYMMETRIC, RANGE_V1_SIGNED_SYMMETRIC, \
    RANGE_V1_UNSIGNED_SYMMETRIC = range(5)


def range_to_grid(enc_min, enc_max, qmin, qmax, mode, gate=False):
    """float32 device tensor [4, C]: scale, offset and the encoding min / max they were made from, for the learnable
    float32 min / max tensors of one quantizer (C elements each, contiguous).  gate=True first puts min <= 0 <= max and
    max >= min + 1e-5 into the two tensors themselves, the way the v1 wrappers order their ranges before a forward
    pass; their version counters are moved, as an in-place torch operation would move them."""
    _require_gpu(enc_min, enc_max)
    if enc_min.dtype != _F32 or enc_max.dtype != _F32 or not enc_min.is_contiguous() or not enc_max.is_contiguous() \
            or enc_min.numel() != enc_max.numel():
        raise ValueError("encoding min / max must be contiguous float32 tensors of one size")
    c = enc_min.numel()
    grid = torch.empty(4, c, dtype=_F32, device=enc_min.device)
    with _OnDevice(enc_min.device):
        check(lib.miq_range_to_grid_f32(_ptr(enc_min), _ptr(enc_max), c, int(qmin), int(qmax), int(mode),
                                        1 if gate else 0, _ptr(grid), _stream(enc_min)))
    if gate:
        torch.autograd.graph.increment_version(enc_min)
        torch.autograd.graph.increment_version(enc_max)
    return grid


def qdq_bwd_range(x, grad_out, num_channel, n_per_channel, grid, qmin, qmax, mode, want_grad_in=True):
    """(grad_in or None, grad_min[C], grad_max[C]) of a quantize-dequantize whose grid range_to_grid() made: the
    backward pass over x and grad_out, the channel sums and their conversion into the gradients of the encoding
    min / max, in the two launches of v2_qdq_bwd_params (one where a channel is a single workgroup's work)."""
    _require_gpu(x, grad_out, grid)
    x, grad_out = x.contiguous(), grad_out.to(x.dtype).contiguous()
    c, npc = int(num_channel), int(n_per_channel)
    if grid.dtype != _F32 or tuple(grid.shape) != (4, c) or not grid.is_contiguous():
        raise ValueError(f"grid must be the contiguous float32 [4, {c}] tensor of range_to_grid()")
    gin = torch.empty_like(x) if want_grad_in else None
    grads = torch.empty(2, c, dtype=_F32, device=x.device)
    ws = torch.empty(int(lib.miq_v2_qdq_bwd_params_workspace_bytes(c, x.numel(), npc)), dtype=torch.uint8,
                     device=x.device)
    fn = getattr(lib, "miq_qdq_bwd_range_" + _suffix(x))
    with _OnDevice(x.device):
        check(fn(_ptr(x), _ptr(grad_out), _ptr(gin) if want_grad_in else None, c, x.numel(), npc, _ptr(grid),
                 int(qmin), int(qmax), int(mode), _ptr(grads[0]), _ptr(grads[1]), _ptr(ws), _stream(x)))
    return gin, grads[0], grads[1]


# -------------------------------------------------------------------------------------------------------- statistics
def _minmax_workspace(num_channel, n, n_per_channel, device):
    nbytes = int(lib.miq_minmax_workspace_bytes(int(num_channel), int(n), int(n_per_channel)))
    return torch.empty(nbytes, dtype=torch.uint8, device=device)


def minmax(x):
    """float32 device tensor [min, max] of x (NaN ignored); asynchronous."""
    _require_gpu(x)
    x = x.to(_F32).contiguous()
    out = torch.empty(2, dtype=_F32, device=x.device)
    ws = _minmax_workspace(1, x.numel(), max(x.numel(), 1), x.device)
    with _OnDevice(x.device):
        check(lib.miq_minmax_f32(_ptr(x), x.numel(), _ptr(out), _ptr(ws), _stream(x)))
    return out


def minmax_per_channel(x, num_channel, n_per_channel):
    """float32 device tensor [2, C]: row 0 = per-channel min, row 1 = per-channel max."""
    _require_gpu(x)
    x = x.to(_F32).contiguous()
    out = torch.empty(2, num_channel, dtype=_F32, device=x.device)
    ws = _minmax_workspace(num_channel, x.numel(), n_per_channel, x.device)
    with _OnDevice(x.device):
        check(lib.miq_minmax_per_channel_f32(_ptr(x), int(num_channel), x.numel(), int(n_per_channel), _ptr(out),
                                             _ptr(ws), _stream(x)))
    return out


# ------------------------------------------------------------------------------------- v2 histogram observer / SQNR
def v2_hist_workspace(num_hist, n_per_hist, num_bins, device):
    nbytes = int(lib.miq_v2_hist_workspace_bytes(int(num_hist), int(n_per_hist), int(num_bins)))
    # zero-filled: the library keeps counters in it that are zero between updates
    return torch.zeros((nbytes + 3) // 4, dtype=torch.int32, device=device)


def v2_hist_update(data, num_hist, num_bins, has_stats, state_hist, state_minmax, bad_flag, workspace,
                   want_batch_hist=True):
    """collect_stats + merge_stats of the v2 histogram observer for one batch; returns (batch_hist, batch_minmax)
    (batch_hist is None when want_batch_hist is False)."""
    _require_gpu(data, state_hist, state_minmax, bad_flag, workspace)
    if data.dtype != _F32 or not data.is_contiguous():
        raise RuntimeError("the histogram observer takes contiguous float32 data")
    n_per_hist = data.numel() // num_hist
    batch_hist = torch.empty(num_hist, num_bins, dtype=_F32, device=data.device) if want_batch_hist else None
    batch_minmax = torch.empty(num_hist, 2, dtype=_F32, device=data.device) if want_batch_hist else None
    with _OnDevice(data.device):
        check(lib.miq_v2_hist_update_f32(_ptr(data), int(num_hist), int(n_per_hist), int(num_bins), int(has_stats),
                                         int(bool(want_batch_hist)), _ptr(state_hist), _ptr(state_minmax),
                                         _ptr(batch_hist), _ptr(batch_minmax), _ptr(bad_flag), _ptr(workspace),
                                         _stream(data)))
    return batch_hist, batch_minmax


class V2HistRepeat:
    """A prepared v2_hist_update for running per-tensor statistics (one histogram, has_stats, no batch histogram):
    everything but the data pointer and the stream is fixed, so the calibration loop's call costs one check and one
    foreign call.  Holds the state tensors it points into."""
    __slots__ = ("_device", "_numel", "_args", "_keep")

    def __init__(self, like, num_bins, state_hist, state_minmax, bad_flag, workspace):
        self._device = like.get_device()
        self._numel = like.numel()
        self._keep = (state_hist, state_minmax, bad_flag, workspace)
        self._args = (1, self._numel, int(num_bins), 1, 0, state_hist.data_ptr(), state_minmax.data_ptr(), None, None,
                      bad_flag.data_ptr(), workspace.data_ptr())

    def matches(self, data):
        return (data.get_device() == self._device and data.numel() == self._numel and data.dtype == _F32
                and data.is_contiguous() and torch.cuda.current_device() == self._device)

    def __call__(self, data):
        check(lib.miq_v2_hist_update_f32(data.data_ptr(), *self._args, _stream_of(data.device)))


def v2_sqnr_num_candidates(num_steps, symmetric, asym_deltas, sym_deltas, offset_candidates):
    n = int(lib.miq_v2_sqnr_num_candidates(float(num_steps), int(symmetric), int(asym_deltas), int(sym_deltas),
                                           int(offset_candidates)))
    if n < 0:
        raise _lib.MiqError(lib.miq_last_error().decode())
    return n


def v2_sqnr_search(hist, minmax, num_steps, symmetric, gamma, asym_deltas, sym_deltas, offset_candidates,
                   want_details=False):
    """SQNR search over the candidate grid; returns (min, max) device vectors [num_hist] (+ noise, best index)."""
    _require_gpu(hist, minmax)
    hist, minmax = hist.contiguous(), minmax.contiguous()
    num_hist, num_bins = hist.shape
    ncand = v2_sqnr_num_candidates(num_steps, symmetric, asym_deltas, sym_deltas, offset_candidates)
    out = torch.empty(2, num_hist, dtype=_F32, device=hist.device)
    noise = torch.empty(num_hist, ncand, dtype=torch.float64, device=hist.device)
    best = torch.empty(num_hist, dtype=torch.int32, device=hist.device) if want_details else None
    with _OnDevice(hist.device):
        check(lib.miq_v2_sqnr_search_f32(_ptr(hist), _ptr(minmax), num_hist, num_bins, float(num_steps),
                                         int(symmetric), float(gamma), int(asym_deltas), int(sym_deltas),
                                         int(offset_candidates), _ptr(out[0]), _ptr(out[1]), _ptr(noise), _ptr(best),
                                         _stream(hist)))
    if want_details:
        return out[0], out[1], noise, best
    return out[0], out[1]


# ----------------------------------------------------------------------------------------------------------- AdaRound
def _ada_check(weight, *others):
    _require_gpu(weight, *others)
    for t in (weight,) + others:
        if t is None:
            continue
        if t.dtype != _F32 or not t.is_contiguous():
            raise RuntimeError("AdaRound kernels take contiguous float32 tensors")


def adaround_soft_round(weight, alpha, num_channel, n_per_channel, delta, offset, clip_min, clip_max,
                        use_soft_rounding=True, out=None):
    """(clamp(floor(w / delta) + h(alpha) - offset, clip_min, clip_max) + offset) * delta."""
    _ada_check(weight, alpha, out)
    out = torch.empty_like(weight) if out is None else out
    with _OnDevice(weight.device):
        check(lib.miq_adaround_soft_round_f32(_ptr(weight), _ptr(alpha), _ptr(out), int(num_channel), weight.numel(),
                                              int(n_per_channel), _ptr(delta), _ptr(offset), float(clip_min),
                                              float(clip_max), int(bool(use_soft_rounding)), _stream(weight)))
    return out


def adaround_floor(weight, num_channel, n_per_channel, delta):
    """floor(w / delta): the alpha-independent part of apply_adaround, input of the fused Linear kernels."""
    _ada_check(weight)
    out = torch.empty_like(weight)
    with _OnDevice(weight.device):
        check(lib.miq_adaround_floor_f32(_ptr(weight), _ptr(out), int(num_channel), weight.numel(),
                                         int(n_per_channel), _ptr(delta), _stream(weight)))
    return out


def adaround_floor_int(weight, num_channel, n_per_channel, delta, offset, clip_min, clip_max, dtype=torch.int8):
    """floor(w / delta) as int8 or int16, saturated per channel to the window outside which its value cannot matter
    (offset + clip_min - 2 .. offset + clip_max + 1), or None when some channel's window does not fit the type.
    Reads one flag back from the device (once per layer)."""
    _ada_check(weight)
    fn = {torch.int8: lib.miq_adaround_floor_i8, torch.int16: lib.miq_adaround_floor_i16}[dtype]
    out = torch.empty(weight.shape, dtype=dtype, device=weight.device)
    unfit = torch.zeros(1, dtype=torch.int32, device=weight.device)
    with _OnDevice(weight.device):
        check(fn(_ptr(weight), _ptr(out), int(num_channel), weight.numel(), int(n_per_channel), _ptr(delta),
                 _ptr(offset), float(clip_min), float(clip_max), _ptr(unfit), _stream(weight)))
    return None if int(unfit.item()) else out


def adaround_floor_i8(weight, num_channel, n_per_channel, delta, offset, clip_min, clip_max):
    return adaround_floor_int(weight, num_channel, n_per_channel, delta, offset, clip_min, clip_max, torch.int8)


def adaround_floor_packed(weight, num_channel, n_per_channel, delta, offset, clip_min, clip_max):
    """The narrowest integer form of floor(w / delta) that fits (int8, then int16), or None."""
    for dtype in (torch.int8, torch.int16):
        out = adaround_floor_int(weight, num_channel, n_per_channel, delta, offset, clip_min, clip_max, dtype)
        if out is not None:
            return out
    return None


def adaround_init_alpha(weight, num_channel, n_per_channel, delta):
    """alpha such that h(alpha) equals the fractional part of w / delta."""
    _ada_check(weight)
    alpha = torch.empty_like(weight)
    with _OnDevice(weight.device):
        check(lib.miq_adaround_init_alpha_f32(_ptr(weight), _ptr(alpha), int(num_channel), weight.numel(),
                                              int(n_per_channel), _ptr(delta), _stream(weight)))
    return alpha


def adaround_blocks(num_element):
    return int(lib.miq_adaround_blocks(int(num_element)))


def adaround_eval_terms(values, what, beta=2.0):
    """The kernels' own per-element AdaRound terms, for accuracy measurements.

    what = 0: `values` is alpha; returns (sigmoid(alpha), h(alpha), dh/dalpha).
    what = 1: `values` is h; returns (1 - |2h - 1|^beta, its derivative with respect to h)."""
    _ada_check(values)
    n = values.numel()
    out = torch.empty((3 if what == 0 else 2, n), dtype=_F32, device=values.device)
    with _OnDevice(values.device):
        check(lib.miq_adaround_eval_terms_f32(_ptr(values), _ptr(out), n, int(what), float(beta), _stream(values)))
    return tuple(out[i] for i in range(out.size(0)))


def adaround_bwd(weight, grad_weight, alpha, num_channel, n_per_channel, delta, offset, clip_min, clip_max,
                 reg_param=0.0, beta=-1.0, reg_partial=None):
    """dLoss/dW' -> dLoss/dalpha (rounding regulariser included when beta >= 0); returns the gradient."""
    _ada_check(weight, grad_weight, alpha)
    grad_alpha = torch.empty_like(alpha)
    with _OnDevice(weight.device):
        check(lib.miq_adaround_bwd_f32(_ptr(weight), _ptr(grad_weight), _ptr(alpha), _ptr(grad_alpha),
                                       int(num_channel), weight.numel(), int(n_per_channel), _ptr(delta),
                                       _ptr(offset), float(clip_min), float(clip_max), float(reg_param), float(beta),
                                       _ptr(reg_partial), _stream(weight)))
    return grad_alpha


def adaround_bwd_adam(weight, grad_weight, alpha, exp_avg, exp_avg_sq, num_channel, n_per_channel, delta, offset,
                      clip_min, clip_max, reg_param, beta, lr, beta1, beta2, eps, step, reg_partial=None,
                      grad_alpha=None):
    """dLoss/dW' -> Adam update of alpha (in place), rounding regulariser included when beta >= 0."""
    _ada_check(weight, grad_weight, alpha, exp_avg, exp_avg_sq)
    if reg_partial is not None and reg_partial.numel() < adaround_blocks(weight.numel()):
        raise RuntimeError("reg_partial is too small")
    with _OnDevice(weight.device):
        check(lib.miq_adaround_bwd_adam_f32(_ptr(weight), _ptr(grad_weight), _ptr(alpha), _ptr(exp_avg),
                                            _ptr(exp_avg_sq), _ptr(grad_alpha), int(num_channel), weight.numel(), int(n_per_channel),
                                            _ptr(delta), _ptr(offset), float(clip_min), float(clip_max),
                                            float(reg_param), float(beta), float(lr), float(beta1), float(beta2),
                                            float(eps), int(step), _ptr(reg_partial), _stream(weight)))


def adaround_linear_supported(out_features, in_features, batch):
    """Shapes the MFMA-fused Linear path takes."""
    return batch in (32, 64, 128, 256) and out_features % 32 == 0 and in_features % 128 == 0 and \
        out_features * in_features < 2 ** 31


def adaround_linear_workspace(out_features, in_features, device, batch=32):
    nbytes = int(lib.miq_adaround_linear_workspace_bytes(int(out_features), int(in_features), int(batch)))
    return torch.empty(nbytes // 4, dtype=_F32, device=device)


def adaround_linear_blocks(out_features, in_features):
    return int(lib.miq_adaround_linear_blocks(int(out_features), int(in_features)))


def _floor_variant(weight_floor, alpha, prefix):
    """Entry point for the storage type of floor(W / delta): float32, int8 or int16 (adaround_floor_int)."""
    suffix = {_F32: "f32", torch.int8: "i8", torch.int16: "i16"}.get(weight_floor.dtype)
    if suffix is None or not weight_floor.is_contiguous() or weight_floor.shape != alpha.shape or \
            not weight_floor.is_cuda:
        raise RuntimeError("weight_floor must be a contiguous float32, int8 or int16 GPU tensor of alpha's shape")
    return getattr(lib, prefix + suffix)


def _ada_batch(grad_out, out_features, row_index):
    """Rows per iteration of the fused Linear path: grad_out is [batch, out_features]."""
    if grad_out.dim() != 2 or grad_out.size(1) != out_features:
        raise RuntimeError("grad_out must be [batch, out_features]")
    batch = grad_out.size(0)
    if row_index is not None and (row_index.dtype != torch.int32 or row_index.numel() != batch or
                                  not row_index.is_contiguous()):
        raise RuntimeError(f"row_index must hold {batch} int32 row numbers")
    return batch


def adaround_linear_fwd(weight_floor, alpha, x, row_index, target, bias, num_channel, delta, offset, clip_min, clip_max,
                        activation, workspace, grad_out, out=None, loss_partial=None):
    """Fused apply_adaround + Linear forward + reconstruction-loss gradient for the rows of x / target that row_index
    names: as many as grad_out has rows (32, 64, 128 or 256)."""
    _ada_check(alpha, workspace, grad_out, out)
    fn = _floor_variant(weight_floor, alpha, "miq_adaround_linear_fwd_")
    _require_gpu(weight_floor, x, target, bias, row_index)
    if x.dtype != _F32 or target.dtype != _F32 or x.stride(-1) != 1 or target.stride(-1) != 1:
        raise RuntimeError("x and target must be float32 with contiguous rows")
    o, k = weight_floor.shape
    batch = _ada_batch(grad_out, o, row_index)
    if workspace.numel() * 4 < lib.miq_adaround_linear_workspace_bytes(o, k, batch) or \
            (out is not None and out.numel() < batch * o):
        raise RuntimeError("workspace or out is too small for this batch")
    with _OnDevice(weight_floor.device):
        check(fn(_ptr(weight_floor), _ptr(alpha), _ptr(x), _ptr(row_index), batch, min(x.size(0), target.size(0)),
                 x.stride(0),
                 _ptr(target), target.stride(0),
                 _ptr(bias), o, k, int(num_channel), _ptr(delta), _ptr(offset), float(clip_min), float(clip_max),
                 int(activation), _ptr(workspace), _ptr(out), _ptr(grad_out), _ptr(loss_partial), _stream(weight_floor)))


def adaround_linear_bwd_adam(weight_floor, grad_out, x, row_index, alpha, exp_avg, exp_avg_sq, num_channel, delta, offset,
                             clip_min, clip_max, reg_param, beta, lr, beta1, beta2, eps, step, reg_partial=None,
                             grad_alpha=None):
    """Fused dLoss/dW' = grad_out^T x (MFMA) + alpha gradient + regulariser + Adam update (alpha, moments in place)."""
    _ada_check(grad_out, alpha, exp_avg, exp_avg_sq, grad_alpha)
    fn = _floor_variant(weight_floor, alpha, "miq_adaround_linear_bwd_adam_")
    _require_gpu(weight_floor, x, row_index)
    o, k = weight_floor.shape
    batch = _ada_batch(grad_out, o, row_index)
    if x.dtype != _F32 or x.stride(-1) != 1:
        raise RuntimeError("x must be float32 with contiguous rows")
    with _OnDevice(weight_floor.device):
        check(fn(_ptr(weight_floor), _ptr(grad_out), _ptr(x), _ptr(row_index), batch, x.size(0), x.stride(0), _ptr(alpha),
                 _ptr(exp_avg),
                 _ptr(exp_avg_sq), _ptr(grad_alpha), o, k, int(num_channel), _ptr(delta), _ptr(offset), float(clip_min),
                 float(clip_max), float(reg_param), float(beta), float(lr), float(beta1), float(beta2), float(eps),
                 int(step), _ptr(reg_partial), _stream(weight_floor)))


class _StateOwner:
    """Keeps a device-state tensor (torch's caching allocator) safe when the object is used on several streams: the
    allocator may hand the block to someone else as soon as the tensor dies, unless it knows which streams used it."""

    def _init_state(self, nbytes):
        self._state = torch.empty(int(nbytes) // 8 + 1, dtype=torch.float64, device=self.device)
        self._last_stream = torch.cuda.current_stream(self.device)
        self._last_handle = self._last_stream.cuda_stream
        self._streams_seen = {self._last_handle}

    def _note_stream(self, handle):
        """Called with the stream handle of every call that queues work on the state.  The object's host-side
        bookkeeping (pending batch, sequence numbers, whether the range is known) assumes that its launches run in the
        order they were queued; when the caller moves to another stream, that stream is made to wait for everything
        queued on the previous one."""
        if handle != self._last_handle:
            current = torch.cuda.current_stream(self.device)
            current.wait_event(self._last_stream.record_event())
            self._last_stream, self._last_handle = current, handle
            if handle not in self._streams_seen:
                self._streams_seen.add(handle)
                self._state.record_stream(current)


# Destroying an analyzer frees pinned host memory (and, for some modes, device memory): calls the HIP runtime refuses
# while a stream capture is under way -- they invalidate the capture.  The garbage collector can run a destructor in the
# middle of somebody's `torch.cuda.graph(...)` block, so a handle that dies while the current stream is capturing is
# parked and destroyed by the next creation or destruction that happens outside a capture.
_parked_handles = []


def _capturing() -> bool:
    try:
        return torch.cuda.is_current_stream_capturing()
    except Exception:                             # pylint: disable=broad-except
        return False                              # interpreter shutdown, or no usable device any more


def _destroy_parked():
    while _parked_handles and lib is not None:
        destroy, handle = _parked_handles.pop()
        destroy(handle)


def _destroy_handle(destroy, handle):
    if _capturing():
        _parked_handles.append((destroy, handle))
        return
    _destroy_parked()
    destroy(handle)


class Analyzer(_StateOwner):
    """Device-resident encoding analyzer: mode 0 = TF min/max, 1 = TF-Enhanced (512-bucket PDF + SQNR search),
    2 = percentile on the same PDF, 3 = least squared error over pairs of bucket edges of the same PDF, 4 = least KL
    divergence over windows of a 512-bin histogram that follows the range of the data."""

    def __init__(self, mode, device=None):
        self.mode = int(mode)
        self.device = torch.device("cuda", torch.cuda.current_device()) if device is None else torch.device(device)
        if self.device.type != "cuda":
            raise RuntimeError("an Analyzer lives on a GPU")
        if self.device.index is None:
            self.device = torch.device("cuda", torch.cuda.current_device())
        h = C.c_void_p()
        if not _capturing():
            _destroy_parked()
        # the device state comes from torch's caching allocator
        self._init_state(lib.miq_analyzer_state_bytes())
        with torch.cuda.device(self.device):
            check(lib.miq_analyzer_create_in(self.mode, _ptr(self._state), C.byref(h)))
        self._h = h

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h and lib is not None:                 # at interpreter shutdown the module's globals may already be gone
            _destroy_handle(lib.miq_analyzer_destroy, h)

    def _s(self):
        handle = _stream_of(self.device)
        if handle != self._last_handle:
            self._note_stream(handle)
        return C.c_void_p(handle)

    def reset(self):
        with torch.cuda.device(self.device):
            check(lib.miq_analyzer_reset(self._h, self._s()))

    def set_percentile(self, percentile: float):
        check(lib.miq_analyzer_set_percentile(self._h, float(percentile)))

    def update_stats(self, x):
        """Queue one batch.  Lean on purpose: a batch of a few MB takes microseconds on the device, so the Python
        cost of this call is what bounds calibration throughput."""
        if not x.is_cuda or x.device != self.device:
            raise RuntimeError(f"analyzer lives on {self.device}, tensor on {x.device}")
        if x.dtype != _F32 or not x.is_contiguous():
            x = x.to(_F32).contiguous()
        # x was produced on (or converted on) the current stream and the kernels are queued on the same stream, so
        # the caching allocator cannot hand its memory to anyone else before they have run
        if torch.cuda.current_device() == self.device.index:
            stream = _stream_of(self.device)
            if stream != self._last_handle:
                self._note_stream(stream)
            check(lib.miq_analyzer_update_stats_f32(self._h, x.data_ptr(), x.numel(), stream))
        else:
            with torch.cuda.device(self.device):
                check(lib.miq_analyzer_update_stats_f32(self._h, x.data_ptr(), x.numel(), self._s()))

    def queue_encoding(self, bw, symmetric=False, strict_symmetric=False, unsigned_symmetric=False):
        """Queue the device work of the next compute_encoding call with these arguments without waiting for it."""
        with torch.cuda.device(self.device):
            check(lib.miq_analyzer_queue_encoding(self._h, int(bw), int(bool(symmetric)), int(bool(strict_symmetric)),
                                                  int(bool(unsigned_symmetric)), self._s()))

    def compute_encoding(self, bw, symmetric=False, strict_symmetric=False, unsigned_symmetric=False):
        """returns (Encoding, is_valid)"""
        e, valid = Encoding(), C.c_int(0)
        with torch.cuda.device(self.device):
            check(lib.miq_analyzer_compute_encoding(self._h, int(bw), int(bool(symmetric)),
                                                    int(bool(strict_symmetric)), int(bool(unsigned_symmetric)),
                                                    C.byref(e), C.byref(valid), self._s()))
        return e, bool(valid.value)

    def get_stats_histogram(self):
        import numpy as np
        xl, pdf = np.zeros(_lib.PDF_SIZE), np.zeros(_lib.PDF_SIZE)
        n = C.c_int(0)
        with torch.cuda.device(self.device):
            check(lib.miq_analyzer_get_stats_histogram(self._h, xl.ctypes.data, pdf.ctypes.data, C.byref(n),
                                                       self._s()))
        return xl[:n.value], pdf[:n.value]

    def entropy_histogram(self):
        """Entropy analyzer only: (512 counts, (min, max) of the range they span, whether a batch other than all zeros
        has been seen, number of batches counted)."""
        import numpy as np
        counts, span = np.zeros(_lib.PDF_SIZE), np.zeros(2)
        seen, batches = C.c_int(0), C.c_int(0)
        with torch.cuda.device(self.device):
            check(lib.miq_analyzer_entropy_histogram(self._h, counts.ctypes.data, span.ctypes.data, C.byref(seen),
                                                     C.byref(batches), self._s()))
        return counts, (float(span[0]), float(span[1])), bool(seen.value), batches.value

    def last_batch_counts(self):
        import numpy as np
        counts = np.zeros(_lib.PDF_SIZE, np.uint32)
        with torch.cuda.device(self.device):
            check(lib.miq_analyzer_last_batch_counts(self._h, counts.ctypes.data, self._s()))
        return counts

    def last_search(self):
        import numpy as np
        cap = 512
        d, o, c = np.zeros(cap, np.float32), np.zeros(cap, np.int32), np.zeros(cap, np.float64)
        n, best = C.c_int(0), C.c_int(-1)
        with torch.cuda.device(self.device):
            check(lib.miq_analyzer_last_search(self._h, d.ctypes.data, o.ctypes.data, c.ctypes.data, cap, C.byref(n),
                                               C.byref(best), self._s()))
        return d[:n.value], o[:n.value], c[:n.value], best.value


class ChannelAnalyzer(_StateOwner):
    """Device-resident per-channel TF-Enhanced (mode 1) / percentile (mode 2) analyzer: one 512-bucket PDF per channel of
    a tensor laid out [outer][channels][n_per_channel], one launch sequence per update, one search launch for all
    channels.  Channel c behaves like an `Analyzer` fed ``tensor.select(axis, c)``.  The state is a torch tensor
    (torch's caching allocator); nothing is allocated per channel."""

    def __init__(self, mode, num_channel, device=None):
        self.mode, self.num_channel = int(mode), int(num_channel)
        self.device = torch.device("cuda", torch.cuda.current_device()) if device is None else torch.device(device)
        if self.device.type != "cuda":
            raise RuntimeError("a ChannelAnalyzer lives on a GPU")
        if self.device.index is None:
            self.device = torch.device("cuda", torch.cuda.current_device())
        self._init_state(lib.miq_channel_analyzer_state_bytes(self.num_channel))
        h = C.c_void_p()
        with torch.cuda.device(self.device):
            check(lib.miq_channel_analyzer_create(self.mode, self.num_channel, _ptr(self._state), self._s(),
                                                  C.byref(h)))
        self._h = h

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h and lib is not None:
            _destroy_handle(lib.miq_channel_analyzer_destroy, h)

    def _s(self):
        handle = _stream_of(self.device)
        if handle != self._last_handle:
            self._note_stream(handle)
        return C.c_void_p(handle)

    def reset(self):
        with torch.cuda.device(self.device):
            check(lib.miq_channel_analyzer_reset(self._h, self._s()))

    def set_percentile(self, percentile: float):
        check(lib.miq_channel_analyzer_set_percentile(self._h, float(percentile)))

    def update_stats(self, x, n_per_channel):
        """x: float32 GPU tensor whose flat layout is [outer][num_channel][n_per_channel]."""
        if not x.is_cuda or x.device != self.device:
            raise RuntimeError(f"analyzer lives on {self.device}, tensor on {x.device}")
        if x.dtype != _F32 or not x.is_contiguous():
            x = x.to(_F32).contiguous()
        ws = _minmax_workspace(self.num_channel, x.numel(), int(n_per_channel), x.device)
        with torch.cuda.device(self.device):
            self._note_stream(_stream_of(self.device))
            check(lib.miq_channel_analyzer_update_stats_f32(self._h, _ptr(x), x.numel(), int(n_per_channel), _ptr(ws),
                                                            self._s()))

    def compute_encodings(self, bw, symmetric=False, strict_symmetric=False, unsigned_symmetric=False):
        """returns (ctypes array of Encoding, one per channel: indexable and iterable; is_valid)"""
        encs = (Encoding * self.num_channel)()
        valid = C.c_int(0)
        with torch.cuda.device(self.device):
            check(lib.miq_channel_analyzer_compute_encodings(self._h, int(bw), int(bool(symmetric)),
                                                             int(bool(strict_symmetric)),
                                                             int(bool(unsigned_symmetric)), encs, C.byref(valid),
                                                             self._s()))
        return encs, bool(valid.value)

    def compute_encodings_on_device(self, bw, symmetric=False, strict_symmetric=False, unsigned_symmetric=False):
        """The search with its results left on the device: (enc, params) as tf_encodings_per_channel returns them, or
        None when the analyzer has no statistics yet.  Nothing waits."""
        c = self.num_channel
        enc = torch.empty(c, 4, dtype=torch.float64, device=self.device)
        outs = torch.empty(6, c, dtype=_F32, device=self.device)
        valid = C.c_int(0)
        with torch.cuda.device(self.device):
            check(lib.miq_channel_analyzer_compute_encodings_device(
                self._h, int(bw), int(bool(symmetric)), int(bool(strict_symmetric)), int(bool(unsigned_symmetric)),
                _ptr(enc), *(_ptr(outs[k]) for k in range(6)), C.byref(valid), self._s()))
        if not valid.value:
            return None
        return enc, tuple(outs[k] for k in range(6))

    def get_stats_histogram(self, channel):
        import numpy as np
        xl, pdf = np.zeros(_lib.PDF_SIZE), np.zeros(_lib.PDF_SIZE)
        n = C.c_int(0)
        with torch.cuda.device(self.device):
            check(lib.miq_channel_analyzer_get_stats_histogram(self._h, int(channel), xl.ctypes.data, pdf.ctypes.data,
                                                               C.byref(n), self._s()))
        return xl[:n.value], pdf[:n.value]
