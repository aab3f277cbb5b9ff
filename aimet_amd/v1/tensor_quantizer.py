"""v1 tensor quantizers: static grid (post-training) and learned grid (range learning).

Mirrors TrainingExtensions/torch/src/python/aimet_torch/v1/tensor_quantizer.py (TensorQuantizer :61-123,
StaticGridTensorQuantizer :143-395, StaticGridPerTensorQuantizer :398-480, StaticGridPerChannelQuantizer :483-570,
autograd functions QuantizeDequantize / Quantize :1098-1277; LearnedGridTensorQuantizer :573-895,
QuantizeDequantizeFunc :898-986, initialize_learned_grid_quantizer_attributes :1285-1345): same class names,
attributes, method names and semantics.  What differs is below the interface:

* per-channel quantizers keep their per-channel (min, max, delta, offset) as four device vectors built once per
  encoding, instead of rebuilding a host vector and copying it to the device on every forward;
* per-channel min/max (TF) statistics are one fused kernel over the whole weight instead of one
  select().contiguous() copy plus two reductions per channel;
* bfloat16 tensors go through the kernels directly (conversion fused) instead of .to(float32) / .to(dtype) passes;
* the per-channel straight-through backward works (the reference's QuantizeDequantize.backward reads ``.min`` of a
  list for per-channel quantizers).
"""
import functools
import io
import math
from typing import List, Optional, Tuple, Union

import torch

from .. import ops
from ..common import libpymo
from ..common.AimetTensorQuantizer import AimetTensorQuantizer
from ..common.defs import MAP_QUANT_SCHEME_TO_PYMO, QuantizationDataType, QuantScheme
from . import quantsim_straight_through_grad as grad_fn


class TensorQuantizer:
    """Base class: simulation of quantization for one tensor (a parameter, a layer input or a layer output)."""

    def __init__(self, bitwidth: int, round_mode: libpymo.RoundingMode, quant_scheme: QuantScheme,
                 use_symmetric_encodings: bool, enabled_by_default: bool,
                 data_type: QuantizationDataType = QuantizationDataType.int):
        super().__init__()
        self.round_mode = round_mode
        self._quant_scheme = quant_scheme
        self.use_symmetric_encodings = use_symmetric_encodings
        self.use_strict_symmetric = False
        self.use_unsigned_symmetric = False
        self.is_unsigned_symmetric = False
        self.bitwidth = bitwidth
        self.enabled = enabled_by_default
        self.data_type = data_type
        self.is_const = False
        self.is_singleton = False
        self._encoding_min_max_fixed_vals = None
        self._is_encoding_frozen = False

    @property
    def quant_scheme(self):
        return self._quant_scheme

    @property
    def is_encoding_frozen(self):
        return self._is_encoding_frozen

    @property
    def channel_axis(self):
        return None

    @property
    def encoding_min_max_fixed_vals(self) -> Optional[Tuple[float, float]]:
        return self._encoding_min_max_fixed_vals


class StaticGridTensorQuantizer(TensorQuantizer):
    """Simulates quantization for the given tensor post training."""

    def __init__(self, bitwidth, round_mode, quant_scheme, use_symmetric_encodings, enabled_by_default,
                 data_type=QuantizationDataType.int):
        if data_type == QuantizationDataType.float and bitwidth not in (8, 16, 32):
            raise ValueError("float data_type only supports bitwidth in {16, 8}")
        super().__init__(bitwidth, round_mode, quant_scheme, use_symmetric_encodings, enabled_by_default, data_type)
        self._cppOp = None
        self._encoding = None
        self.fp8_maxval = None        # largest value of the 8-bit float grid: 0-dim tensor, or one entry per channel
        self._fp8_grid = None         # (maxval, bias, steps) device tensors of that grid, and the maxval they are for

    # The list of TfEncoding objects.  A per-channel quantizer whose encodings were computed on the device keeps them
    # there (`_pending_encoding`) and builds the list when somebody reads it: a wrapper in training mode recomputes its
    # parameter encodings in every forward and only ever quantizes with them.
    @property
    def _encoding(self):
        pending = self.__dict__.get('_pending_encoding')
        if pending is not None:
            self.__dict__['_pending_encoding'] = None
            self.__dict__['_encoding_list'] = pending()
            computed_from = self.__dict__.get('_computed_from')
            if computed_from is not None and computed_from[1] is pending:
                self.__dict__['_computed_from'] = (computed_from[0], self.__dict__['_encoding_list'])
        return self.__dict__.get('_encoding_list')

    @_encoding.setter
    def _encoding(self, value):
        self.__dict__['_pending_encoding'] = None
        self.__dict__['_encoding_list'] = value
        self.__dict__['_encoding_serial'] = self.__dict__.get('_encoding_serial', 0) + 1

    def _has_encoding(self) -> bool:
        """bool(self._encoding) without building the list."""
        return self.__dict__.get('_pending_encoding') is not None or bool(self.__dict__.get('_encoding_list'))

    has_encoding = _has_encoding

    def encoding_stamp(self):
        """Changes whenever the encoding does: a count of assignments, plus, where the list exists, the bounds at both
        of its ends (an encoding object edited in place).  Does not build the list."""
        serial = self.__dict__.get('_encoding_serial', 0)
        if self.__dict__.get('_pending_encoding') is not None:
            return ('on device', serial)
        enc = self.__dict__.get('_encoding_list')
        if not enc:
            return (None, serial)
        return (id(enc), serial, len(enc), enc[0].min, enc[0].max, enc[-1].min, enc[-1].max, enc[0].bw)

    # ---- 8-bit float grid (reference tensor_quantizer.py:393-400, :461-468, :544-552; fp_quantization.py:45-122)
    @property
    def _is_fp8(self) -> bool:
        return self.data_type == QuantizationDataType.float and self.bitwidth == 8

    def update_maxval(self, maxval: torch.Tensor):
        """Running estimate of the grid's largest value: the first observation, then 0.9 old + 0.1 new."""
        self.fp8_maxval = maxval if self.fp8_maxval is None else 0.9 * self.fp8_maxval + 0.1 * maxval

    def _fp8_observe(self, tensor: torch.Tensor, per_channel: bool):
        """One calibration step of the 8-bit float grid: the batch's maxval by the rule of the quant scheme (largest
        magnitude for TF; for TF-Enhanced the candidate among 111 between 0.1 and 1.2 times the largest magnitude
        with the smallest mean squared error), folded into fp8_maxval, which also becomes the encoding's max."""
        if self._quant_scheme == QuantScheme.post_training_percentile:
            raise NotImplementedError("Percentile scheme is not supported for FP8")
        tensor = tensor.detach().to(torch.float32)
        axis = self.channel_axis if per_channel else None
        if per_channel:
            other = [d for d in range(tensor.dim()) if d != axis]
            largest = tensor.abs().amax(dim=other) if other else tensor.abs()
        else:
            largest = tensor.abs().max()
        if self._quant_scheme == QuantScheme.post_training_tf:
            maxval = largest
        else:
            # candidates as aimet_torch/fp_quantization.py:78-110 forms them: per channel, 111 float32 values from
            # torch.linspace(0.1 * largest, 1.2 * largest) with Python-float end points
            ends = largest.reshape(-1).cpu().tolist()
            candidates = torch.stack([torch.linspace(0.1 * mx, 1.2 * mx, 111) for mx in ends]).to(tensor.device).t()
            errors = []
            for candidate in candidates:                              # [111, channels]
                cast = ops.fp8_fake_cast(tensor, candidate if per_channel else candidate[0], 3, axis or 0)
                squared = (tensor - cast) ** 2
                errors.append((squared.mean(dim=other) if per_channel and other else squared.mean()).reshape(-1))
            best = torch.stack(errors).argmin(0)
            maxval = candidates.gather(0, best.view(1, -1)).view(largest.shape)
        self.update_maxval(maxval)
        self._encoding = [libpymo.TfEncoding(-float(m), float(m), 0.0, 0.0, 8)
                          for m in self.fp8_maxval.reshape(-1).tolist()]

    def __str__(self):
        stream = io.StringIO(newline='\n')
        stream.write('StaticGrid TensorQuantizer:\n')
        stream.write(f'    quant-scheme:{self._quant_scheme}, round_mode={self.round_mode}, '
                     f'bitwidth={self.bitwidth}, enabled={self.enabled}\n')
        if self._encoding:
            for enc in self._encoding:
                stream.write(f'    min:{enc.min}, max={enc.max}, delta={enc.delta}, offset={enc.offset}\n')
        else:
            stream.write('    no encoding\n')
        return stream.getvalue()

    # pickling: the device objects are dropped and re-created, encodings travel as tuples (reference :182-220)
    def __getstate__(self):
        state = self.__dict__.copy()
        state['_num_ops'] = len(self._cppOp)
        state['_encoding'] = None if self._encoding is None else \
            [(e.min, e.max, e.delta, e.offset, e.bw) for e in self._encoding]
        for key in ('_cppOp', '_dev_params', '_fp8_grid', '_channel_analyzer', '_computed_from', '_encoding_list',
                    '_pending_encoding'):
            state.pop(key, None)
        return state

    def __setstate__(self, state):
        num_ops = state.pop('_num_ops')
        encoding = state.pop('_encoding')
        self.__dict__.update(state)
        self._cppOp = [AimetTensorQuantizer(MAP_QUANT_SCHEME_TO_PYMO[self._quant_scheme]) for _ in range(num_ops)]
        self._encoding = None if encoding is None else [libpymo.TfEncoding(*e) for e in encoding]
        self._dev_params = None
        self._fp8_grid = None
        if '_tf_minmax' in state:
            self._channel_analyzer = None

    @property
    def quant_scheme(self) -> QuantScheme:
        return self._quant_scheme

    @quant_scheme.setter
    def quant_scheme(self, quant_scheme: QuantScheme):
        # re-instantiates the analyzer objects, which also clears accumulated statistics (reference :222-247)
        self._quant_scheme = quant_scheme
        assert self._cppOp
        self._cppOp = [AimetTensorQuantizer(MAP_QUANT_SCHEME_TO_PYMO[quant_scheme]) for _ in self._cppOp]
        self._stats_changed()
        self._drop_fused_stats()

    @property
    def encoding(self):
        return self._encoding

    @encoding.setter
    def encoding(self, encoding) -> None:
        if self._is_encoding_frozen:
            raise RuntimeError("Encoding can be set only when it is not frozen.")
        self._encoding = encoding
        self._dev_params = None

    @TensorQuantizer.encoding_min_max_fixed_vals.setter
    def encoding_min_max_fixed_vals(self, min_max_vals: Tuple[float, float]):
        assert isinstance(min_max_vals, tuple) and len(min_max_vals) == 2, 'Min max vals must be a tuple of two values'
        assert min_max_vals[0] < min_max_vals[1], f'Min value {min_max_vals[0]} is not less than max val ' \
                                                  f'{min_max_vals[1]}'
        if self.quant_scheme != QuantScheme.post_training_tf:
            self.quant_scheme = QuantScheme.post_training_tf
        self._encoding_min_max_fixed_vals = min_max_vals
        self._drop_fused_stats()

    def _drop_fused_stats(self):
        """Statistics a subclass keeps outside the analyzer objects go with them."""

    def _stats_tensor(self, tensor: torch.Tensor) -> torch.Tensor:
        if self.encoding_min_max_fixed_vals is not None:
            return torch.tensor(list(self.encoding_min_max_fixed_vals), dtype=torch.float32, device=tensor.device)
        return tensor

    def _stats_changed(self):
        """Every update / reset of the statistics (and of what turns them into encodings) counts up."""
        self.__dict__['_stats_version'] = self.__dict__.get('_stats_version', 0) + 1

    def _encoding_recipe(self):
        return (self.__dict__.get('_stats_version', 0), self.bitwidth, self.data_type, self.use_symmetric_encodings,
                self.use_strict_symmetric, self.use_unsigned_symmetric, self._quant_scheme,
                self.encoding_min_max_fixed_vals, getattr(self, '_percentile_value', None))

    def compute_encoding(self):
        """Compute the encoding(s) from the accumulated statistics; skipped for bitwidth 32 (reference :280-321)."""
        if self.enabled and not self._is_encoding_frozen:
            # The same statistics and settings give the same encodings: the simulation model asks twice for every
            # parameter (once when the first forward needs the encoding, once at the end of compute_encodings), and
            # a per-channel answer costs a search launch, a read-back and thousands of encoding objects
            recipe, result = self.__dict__.get('_computed_from') or (None, None)
            current = self.__dict__.get('_pending_encoding') or self.__dict__.get('_encoding_list')
            if result is not None and result is current and recipe == self._encoding_recipe():
                return
            self._encoding = []
            self._dev_params = None
            if self.bitwidth == 32 or self.data_type == QuantizationDataType.float:
                # float16 has no encoding (reference :286-290).  The 8-bit float grid is described by fp8_maxval
                # alone; the encoding keeps [-maxval, maxval] for display (the reference leaves an empty one here)
                self._encoding = None
                if self._is_fp8 and self.fp8_maxval is not None:
                    self._encoding = [libpymo.TfEncoding(-float(m), float(m), 0.0, 0.0, 8)
                                      for m in self.fp8_maxval.reshape(-1).tolist()]
                return
            computed = self._compute_op_encodings()
            if callable(computed):
                # every channel's encoding exists, on the device: the list is built when it is first read
                self.__dict__['_pending_encoding'] = computed
                self.__dict__['_encoding_serial'] = self.__dict__.get('_encoding_serial', 0) + 1
            else:
                for encoding, valid in computed:
                    if not valid:
                        self.enabled = False
                    else:
                        self._encoding.append(encoding)
            self.is_unsigned_symmetric = self.use_symmetric_encodings and self.use_unsigned_symmetric and \
                all(enc.min >= 0 and enc.max >= 0 for enc in self._encoding)
            assert not (not self.enabled and self._has_encoding()), \
                'At least one encoding for a multi-encoding quantizer is invalid.'
            current = self.__dict__.get('_pending_encoding') or self.__dict__.get('_encoding_list')
            self.__dict__['_computed_from'] = (self._encoding_recipe(), current) if self.enabled and current else None

    def _compute_op_encodings(self):
        return [op.getEncoding(self.bitwidth, self.use_symmetric_encodings, self.use_strict_symmetric,
                               self.use_unsigned_symmetric) for op in self._cppOp]

    def queue_encoding(self):
        """Queue the device work of the next compute_encoding() call without waiting for it.  An owner of many
        quantizers calls this on all of them first: the read-backs that follow then share one wait for the device."""
        if self.enabled and not self._is_encoding_frozen and self.bitwidth != 32 and \
                self.data_type != QuantizationDataType.float and len(self._cppOp) == 1:
            self._cppOp[0].queueEncoding(self.bitwidth, self.use_symmetric_encodings, self.use_strict_symmetric,
                                         self.use_unsigned_symmetric)

    def quantize_dequantize(self, tensor: torch.Tensor, round_mode: libpymo.RoundingMode) -> torch.Tensor:
        if not torch.is_grad_enabled():
            # inference: the same forward without the autograd.Function machinery (about 10 us per call)
            return QuantizeDequantize.forward(_NoContext(), tensor, self, round_mode)
        return QuantizeDequantize.apply(tensor, self, round_mode)

    def quantize(self, tensor: torch.Tensor, round_mode: libpymo.RoundingMode) -> torch.Tensor:
        return Quantize.apply(tensor, self, round_mode)

    def reset_encoding_stats(self):
        if not self._is_encoding_frozen:
            self._stats_changed()
            for op in self._cppOp:
                op.resetEncodingStats()
            self._encoding = None
            self._dev_params = None

    def get_stats_histogram(self) -> List[List]:
        if self._quant_scheme != QuantScheme.post_training_tf_enhanced:
            raise RuntimeError("get_stats_histogram() can be invoked only when quantization scheme is TF-Enhanced.")
        if not self._encoding:
            raise RuntimeError("get_stats_histogram() can be invoked only when encoding is computed.")
        return [op.getStatsHistogram() for op in self._cppOp]

    def freeze_encoding(self) -> None:
        if not self._encoding:
            raise RuntimeError("Encoding can be frozen only when it is not None.")
        self._is_encoding_frozen = True

    def set_percentile_value(self, percentile_value: float):
        self._stats_changed()
        for op in self._cppOp:
            op.setPercentileValue(percentile_value)


class StaticGridPerTensorQuantizer(StaticGridTensorQuantizer):
    """Per-tensor scale/offset."""

    def __init__(self, bitwidth, round_mode, quant_scheme, use_symmetric_encodings, enabled_by_default,
                 data_type=QuantizationDataType.int):
        super().__init__(bitwidth, round_mode, quant_scheme, use_symmetric_encodings, enabled_by_default, data_type)
        self._cppOp = [AimetTensorQuantizer(MAP_QUANT_SCHEME_TO_PYMO[quant_scheme])]
        self._dev_params = None

    @property
    def encoding(self) -> Union[None, libpymo.TfEncoding]:
        return self._encoding[0] if self._encoding else None

    @encoding.setter
    def encoding(self, encoding):
        if self._is_encoding_frozen:
            raise RuntimeError("Encoding can be set only when it is not frozen.")
        self._encoding = encoding if isinstance(encoding, list) and len(encoding) == 1 else [encoding]

    def update_encoding_stats(self, tensor: torch.Tensor):
        if self.enabled and not self._is_encoding_frozen:
            self._stats_changed()
            if self._is_fp8:
                self._fp8_observe(tensor, per_channel=False)
                return
            if self.bitwidth == 32 or self.data_type == QuantizationDataType.float:
                return
            self._cppOp[0].updateStats(self._stats_tensor(tensor), tensor.is_cuda)


class StaticGridPerChannelQuantizer(StaticGridTensorQuantizer):
    """Per-channel scale/offset along ``ch_axis``."""

    def __init__(self, bitwidth, round_mode, quant_scheme, use_symmetric_encodings, num_channels, enabled_by_default,
                 ch_axis: int = 0, data_type=QuantizationDataType.int):
        super().__init__(bitwidth, round_mode, quant_scheme, use_symmetric_encodings, enabled_by_default, data_type)
        self._cppOp = [AimetTensorQuantizer(MAP_QUANT_SCHEME_TO_PYMO[quant_scheme]) for _ in range(num_channels)]
        self._ch_axis = ch_axis
        self._dev_params = None      # (min, max, delta, offset, raw_min, raw_max) device vectors of the encoding
        self._tf_minmax = None       # fused per-channel running min/max for the TF scheme: device tensor [2, C]
        self._channel_analyzer = None   # TF-Enhanced / percentile: every channel's PDF in one device object
        self._percentile_value = 100.0

    @property
    def channel_axis(self) -> int:
        return self._ch_axis

    def reset_encoding_stats(self):
        if self.__dict__.get('_ops_hold_stats', True):
            super().reset_encoding_stats()           # walks the per-channel objects (thousands of calls)
            self.__dict__['_ops_hold_stats'] = False
        elif not self._is_encoding_frozen:
            # the per-channel objects never saw a tensor: the statistics live in the fused objects below
            self._stats_changed()
            self._encoding = None
            self._dev_params = None
        if not self._is_encoding_frozen:
            self._tf_minmax = None
            if self._channel_analyzer is not None:
                self._channel_analyzer.reset()

    def _drop_fused_stats(self):
        self._tf_minmax = None
        self._channel_analyzer = None

    def set_percentile_value(self, percentile_value: float):
        super().set_percentile_value(percentile_value)
        if self._quant_scheme == QuantScheme.post_training_percentile:
            self._percentile_value = float(percentile_value)
            if self._channel_analyzer is not None:
                self._channel_analyzer.set_percentile(self._percentile_value)

    def get_stats_histogram(self) -> List[List]:
        if self._channel_analyzer is None:
            return super().get_stats_histogram()
        if self._quant_scheme != QuantScheme.post_training_tf_enhanced:
            raise RuntimeError("get_stats_histogram() can be invoked only when quantization scheme is TF-Enhanced.")
        if not self._encoding:
            raise RuntimeError("get_stats_histogram() can be invoked only when encoding is computed.")
        out = []
        for channel in range(self._channel_analyzer.num_channel):
            x_left, pdf = self._channel_analyzer.get_stats_histogram(channel)
            out.append(list(zip(x_left.tolist(), pdf.tolist())))
        return out

    def update_encoding_stats(self, tensor: torch.Tensor):
        if self.enabled and not self._is_encoding_frozen:
            self._stats_changed()
            if self._is_fp8:
                self._fp8_observe(tensor, per_channel=True)
                return
            if self.bitwidth == 32 or self.data_type == QuantizationDataType.float:
                return
            if self.encoding_min_max_fixed_vals is not None:
                fixed = self._stats_tensor(tensor)
                self.__dict__['_ops_hold_stats'] = True
                for op in self._cppOp:
                    op.updateStats(fixed, fixed.is_cuda)
                return
            if tensor.dtype == torch.float16:
                tensor = tensor.to(torch.float32)
            # the reference walks its fixed list of per-channel analyzers (:567-570): a tensor with another number of
            # channels along ch_axis fails there, and statistics gathered so far are never dropped
            if tensor.shape[self._ch_axis] != len(self._cppOp):
                raise RuntimeError(f"the tensor has {tensor.shape[self._ch_axis]} channels along axis {self._ch_axis}; "
                                   f"this quantizer was created for {len(self._cppOp)}")
            if self._quant_scheme == QuantScheme.post_training_tf:
                # one fused pass: per-channel min and max of the whole tensor
                num_channel = tensor.shape[self._ch_axis]
                n_per_channel = functools.reduce(lambda a, b: a * b, tensor.shape[self._ch_axis + 1:], 1)
                mm = ops.minmax_per_channel(tensor, num_channel, n_per_channel)
                if self._tf_minmax is None:
                    self._tf_minmax = mm
                else:
                    self._tf_minmax = torch.stack((torch.minimum(self._tf_minmax[0], mm[0]),
                                                   torch.maximum(self._tf_minmax[1], mm[1])))
                return
            # TF-Enhanced / percentile: the reference feeds one analyzer object per channel with
            # tensor.select(ch_axis, c).contiguous() (:567-570); here one device object holds every channel's PDF and
            # one launch sequence updates them all -- channel c sees exactly the samples of that slice
            if not tensor.is_cuda:
                raise RuntimeError("aimet_amd computes on the GPU only: pass a GPU tensor")
            num_channel = tensor.shape[self._ch_axis]
            n_per_channel = functools.reduce(lambda a, b: a * b, tensor.shape[self._ch_axis + 1:], 1)
            analyzer = self._channel_analyzer
            if analyzer is not None and analyzer.device != tensor.device:
                raise RuntimeError(f"statistics were gathered on {analyzer.device}; this batch is on {tensor.device}")
            if analyzer is None:
                mode = 1 if self._quant_scheme == QuantScheme.post_training_tf_enhanced else 2
                analyzer = ops.ChannelAnalyzer(mode, num_channel, tensor.device)
                analyzer.set_percentile(self._percentile_value)
                self._channel_analyzer = analyzer
            analyzer.update_stats(tensor, n_per_channel)

    def _compute_op_encodings(self):
        if self._channel_analyzer is not None:
            if self.compute_tf_encodings_on_device and self._quant_scheme == QuantScheme.post_training_tf_enhanced:
                found = self._channel_analyzer.compute_encodings_on_device(
                    self.bitwidth, self.use_symmetric_encodings, self.use_strict_symmetric, self.use_unsigned_symmetric)
                if found is not None:
                    return self._encodings_left_on_device(*found)
            encodings, valid = self._channel_analyzer.compute_encodings(
                self.bitwidth, self.use_symmetric_encodings, self.use_strict_symmetric, self.use_unsigned_symmetric)
            return [(libpymo.TfEncoding(e.min, e.max, e.delta, e.offset, e.bw), valid) for e in encodings]
        if self._tf_minmax is None:
            return super()._compute_op_encodings()
        if self.compute_tf_encodings_on_device and self._tf_minmax.is_cuda:
            return self._tf_encodings_on_device()
        # TfEncodingAnalyzer::computeEncoding per channel (DlQuantization/src/TfEncodingAnalyzer.cpp:80-101) on the
        # fused statistics: one small read-back, then the double-precision host recipe
        mm = self._tf_minmax.double().cpu()
        out = []
        for c in range(mm.shape[1]):
            lo, hi = min(0.0, float(mm[0, c])), max(0.0, float(mm[1, c]))
            hi = max(hi, lo + 0.01)
            e = ops.get_computed_encodings(self.bitwidth, lo, hi, self.use_symmetric_encodings,
                                           self.use_strict_symmetric, self.use_unsigned_symmetric)
            out.append((libpymo.TfEncoding(e.min, e.max, e.delta, e.offset, e.bw), True))
        return out

    # The encodings of all channels (TF: min / max; TF-Enhanced: the per-channel search) from one launch, left on the
    # device, instead of one read-back and one host computation or object per channel (thousands per layer, in every
    # forward of a wrapper in training mode).  The numbers are the same: the min / max kernel runs the host recipe's
    # double arithmetic, the search is the one the host path reads back.  False: always the host path.
    compute_tf_encodings_on_device = True

    def _tf_encodings_on_device(self):
        mm = self._tf_minmax.to(torch.float32).contiguous()
        return self._encodings_left_on_device(*ops.tf_encodings_per_channel(
            mm, self.bitwidth, self.use_symmetric_encodings, self.use_strict_symmetric, self.use_unsigned_symmetric))

    def _encodings_left_on_device(self, enc, params):
        """Takes the kernel parameters as they are and returns the builder of the TfEncoding list for
        compute_encoding(): one read-back of [C, 4] doubles when the list is first wanted."""
        self._dev_params = params
        bitwidth = self.bitwidth

        def build():
            return [libpymo.TfEncoding(mn, mx, delta, offset, bitwidth) for mn, mx, delta, offset in enc.cpu().tolist()]
        return build

    def device_params(self, device):
        """Per-channel kernel parameters on `device`, built once per encoding."""
        if self._dev_params is None or self._dev_params[0].device != device:
            mn, mx, delta, offset = AimetTensorQuantizer.channelParams(device, self._encoding)
            raw = torch.tensor([[e.min for e in self._encoding], [e.max for e in self._encoding]],
                               dtype=torch.float32).to(device)
            self._dev_params = (mn, mx, delta, offset, raw[0].contiguous(), raw[1].contiguous())
        return self._dev_params


def _channel_geometry(tensor, ch_axis):
    sizes = [*tensor.shape, 1]
    num_channel = sizes[ch_axis]
    n_per_channel = functools.reduce(lambda x, y: x * y, sizes[ch_axis + 1:])
    return num_channel, n_per_channel


def _is_nearest(round_mode) -> bool:
    value = round_mode.value if isinstance(round_mode, libpymo.RoundingMode) else round_mode
    return int(value) == int(libpymo.RoundingMode.ROUND_NEAREST.value)


class _NoContext:
    """Stands in for the autograd context when QuantizeDequantize.forward is called directly (no gradient)."""
    __slots__ = ("tensor_quantizer", "masked")

    def save_for_backward(self, *_):
        pass


class QuantizeDequantize(torch.autograd.Function):
    """Quantize-dequantize with the straight-through gradient (reference :1098-1212)."""

    @staticmethod
    def _per_tensor_quantize_dequantize(tensor, tensor_quantizer, round_mode):
        # pylint: disable=protected-access
        return tensor_quantizer._cppOp[0].quantizeDequantize(tensor, tensor_quantizer.encoding, round_mode,
                                                             tensor.is_cuda)

    @staticmethod
    def _per_channel_quantize_dequantize(tensor, tensor_quantizer, round_mode):
        num_channel, n_per_channel = _channel_geometry(tensor, tensor_quantizer.channel_axis)
        mn, mx, delta, offset, _, _ = tensor_quantizer.device_params(tensor.device)
        dtype = tensor.dtype
        if dtype not in (torch.float32, torch.bfloat16):
            tensor = tensor.to(torch.float32)
        out = ops.qdq_per_channel(tensor, num_channel, n_per_channel, mn, mx, delta, offset,
                                  round_mode.value if isinstance(round_mode, libpymo.RoundingMode) else round_mode)
        return out.to(dtype)

    @staticmethod
    def _quantize_float(tensor, tensor_quantizer):
        """float16 simulation: tensor.half().float(); 8-bit float simulation: the fake cast to the grid that ends at
        the quantizer's fp8_maxval (reference :1100-1113), each one fused pass for float32 tensors."""
        if tensor_quantizer.bitwidth == 8:
            if tensor_quantizer.fp8_maxval is None:
                raise ValueError('tensor_quantizer.fp8_maxval not present or not initialized!')
            maxval = tensor_quantizer.fp8_maxval
            cached = tensor_quantizer._fp8_grid               # pylint: disable=protected-access
            if cached is None or cached[0] is not maxval or cached[1] != maxval._version:
                cached = (maxval, maxval._version, ops.fp8_grid(maxval.to(tensor.device), 3))
                tensor_quantizer._fp8_grid = cached           # pylint: disable=protected-access
            out = ops.fp8_fake_cast(tensor.to(torch.float32), None, 3, tensor_quantizer.channel_axis or 0,
                                    grid=cached[2])
            return out.to(tensor.dtype)
        if tensor_quantizer.bitwidth != 16:
            raise ValueError('float data_type only supports bitwidth in {16, 8}')
        if tensor.dtype == torch.float32 and tensor.is_cuda:
            return ops.fp16_round_trip(tensor)
        return tensor.half().float()

    # The backward needs one bit per element: whether the input lay inside the stored encoding's range.  When the
    # input wants a gradient the forward writes those bits itself (ops.qdq_mask_*) and keeps them instead of the
    # input -- 1/8 byte per element instead of 4, and the backward reads 1/8 byte instead of the input again.  The
    # reference keeps the input and compares in backward (reference :1186-1212); the results are the same bit for bit
    # as long as the encoding is not changed between the two passes.  False: keep the input, as the reference does.
    save_mask = True

    @staticmethod
    def _masked_forward(tensor, tensor_quantizer):
        """(quantized, mask) through the mask-writing forward, or None where it does not apply."""
        if not (tensor.is_cuda and tensor.dtype in (torch.float32, torch.bfloat16) and tensor.is_contiguous()):
            return None
        if isinstance(tensor_quantizer, StaticGridPerChannelQuantizer):
            num_channel, n_per_channel = _channel_geometry(tensor, tensor_quantizer.channel_axis)
            mn, mx, delta, offset, raw_min, raw_max = tensor_quantizer.device_params(tensor.device)
            return ops.qdq_mask_per_channel(tensor, num_channel, n_per_channel, mn, mx, delta, offset, raw_min,
                                            raw_max)
        enc = tensor_quantizer.encoding
        mask_min, mask_max = enc.min, enc.max
        if tensor.dtype != torch.float32:
            # the reference compares against a 0-dim tensor, which torch's type promotion casts to x's dtype
            mask_min = float(torch.tensor(mask_min, dtype=torch.float32).to(tensor.dtype))
            mask_max = float(torch.tensor(mask_max, dtype=torch.float32).to(tensor.dtype))
        return ops.qdq_mask_per_tensor(tensor, enc.min, enc.max, enc.bw, mask_min, mask_max)

    @staticmethod
    def forward(ctx, tensor, tensor_quantizer, round_mode):  # pylint: disable=arguments-differ
        ctx.masked = False
        if tensor_quantizer.enabled and tensor_quantizer.bitwidth != 32:
            masked = None
            if QuantizeDequantize.save_mask and tensor_quantizer.data_type == QuantizationDataType.int and \
                    getattr(ctx, "needs_input_grad", (False,))[0] and _is_nearest(round_mode):
                masked = QuantizeDequantize._masked_forward(tensor, tensor_quantizer)
            if masked is not None:
                quantized, mask = masked
                ctx.masked = True
                ctx.save_for_backward(mask)
            else:
                if tensor_quantizer.data_type == QuantizationDataType.float:
                    quantized = QuantizeDequantize._quantize_float(tensor, tensor_quantizer)
                elif isinstance(tensor_quantizer, StaticGridPerChannelQuantizer):
                    quantized = QuantizeDequantize._per_channel_quantize_dequantize(tensor, tensor_quantizer,
                                                                                    round_mode)
                else:
                    dtype = tensor.dtype
                    quantized = QuantizeDequantize._per_tensor_quantize_dequantize(tensor, tensor_quantizer,
                                                                                   round_mode).to(dtype)
                ctx.save_for_backward(tensor)
        else:
            quantized = tensor
        ctx.tensor_quantizer = tensor_quantizer
        return quantized

    @staticmethod
    def backward(ctx, output_grad):  # pylint: disable=arguments-differ
        q = ctx.tensor_quantizer
        if ctx.masked:
            mask, = ctx.saved_tensors
            grad = ops.ste_bwd_mask(mask, output_grad)
        elif q.enabled and q.data_type == QuantizationDataType.int and q.bitwidth != 32:
            tensor, = ctx.saved_tensors
            if isinstance(q, StaticGridPerChannelQuantizer):
                _, _, _, _, raw_min, raw_max = q.device_params(tensor.device)
                grad = grad_fn.compute_dloss_by_dx(tensor, output_grad, raw_min, raw_max, q.channel_axis)
            else:
                grad = grad_fn.compute_dloss_by_dx(tensor, output_grad, q.encoding.min, q.encoding.max)
        else:
            grad = output_grad
        return grad, None, None


class Quantize(torch.autograd.Function):
    """Quantize only: float-valued grid indices, signed range by default (reference :1216-1277)."""

    @staticmethod
    def forward(ctx, tensor, tensor_quantizer, round_mode):  # pylint: disable=arguments-differ
        assert tensor_quantizer.enabled, 'Tensor quantizer must be enabled to perform quantize only.'
        assert tensor_quantizer.data_type == QuantizationDataType.int
        assert tensor_quantizer.bitwidth != 32, 'Tensor quantizer bitwidth must be < 32 to perform quantize only.'
        assert tensor_quantizer.encoding is not None, 'Tensor quantizer encoding must be valid.'
        shift_to_signed = not (tensor_quantizer.use_symmetric_encodings and tensor_quantizer.use_unsigned_symmetric)
        # pylint: disable=protected-access
        if isinstance(tensor_quantizer, StaticGridPerChannelQuantizer):
            slices = []
            for index, op in enumerate(tensor_quantizer._cppOp):
                tensor_slice = tensor.select(tensor_quantizer._ch_axis, index).contiguous()
                slices.append(op.quantize(tensor_slice, tensor_quantizer._encoding[index], round_mode,
                                          tensor.is_cuda, shift_to_signed))
            return torch.stack(tuple(slices), dim=tensor_quantizer._ch_axis)
        return tensor_quantizer._cppOp[0].quantize(tensor, tensor_quantizer.encoding, round_mode, tensor.is_cuda,
                                                   shift_to_signed)

    @staticmethod
    def backward(ctx, _output_grad):  # pylint: disable=arguments-differ
        raise AssertionError('Backward pass for quantize only not implemented')


# ------------------------------------------------------------------------------------------------- range learning
def is_non_strict_symmetric(use_symmetric_encodings: bool, use_strict_symmetric: bool,
                            is_unsigned_symmetric: bool) -> bool:
    return use_symmetric_encodings and not use_strict_symmetric and not is_unsigned_symmetric


class LearnedGridTensorQuantizer(TensorQuantizer):
    """Quantization simulation whose encoding min / max are parameters of the owning wrapper, initialised from a
    calibrated encoding and then learned (reference :573-895).  The wrapper holds the parameters under
    '<name>_encoding_min' / '<name>_encoding_max'; this object holds the configuration and computes encodings from
    them."""

    # pylint: disable=too-many-instance-attributes
    def __init__(self, bitwidth: int, round_mode, quant_scheme: QuantScheme, use_symmetric_encodings: bool,
                 enabled_by_default: bool, data_type: QuantizationDataType = QuantizationDataType.int):
        if data_type != QuantizationDataType.int:
            raise ValueError('Only QuantizationDataType.int is supported for LearnedGridTensorQuantizer')
        super().__init__(bitwidth, round_mode, quant_scheme, use_symmetric_encodings, enabled_by_default, data_type)
        self.wrapper_ref = None
        self.name = None
        self.scaling, self.offset = None, None
        self.device = None
        self._ch_axis = 0

    @staticmethod
    def get_n_and_p(bitwidth: int, use_symmetric_encoding: bool, use_strict_symmetric: bool, device=None):
        """Grid bounds n = 0 and p = 2^bitwidth - 1 (one less for strict symmetric) as tensors."""
        if not use_symmetric_encoding and use_strict_symmetric:
            raise ValueError("Strict symmetric can be enabled only when using symmetric encoding")
        p = 2.0 ** bitwidth - 1
        if use_symmetric_encoding and use_strict_symmetric:
            p -= 1
        return torch.tensor([0.0], device=device), torch.tensor([p], device=device)

    def n(self, device=None) -> torch.Tensor:
        return self.get_n_and_p(self.bitwidth, self.use_strict_symmetric, self.use_strict_symmetric,
                                device or self.device)[0]

    def p(self, device=None) -> torch.Tensor:
        return self.get_n_and_p(self.bitwidth, self.use_strict_symmetric, self.use_strict_symmetric,
                                device or self.device)[1]

    def _parameters_of_wrapper(self):
        return getattr(self.wrapper_ref, self.name + '_encoding_min'), \
            getattr(self.wrapper_ref, self.name + '_encoding_max')

    def __getstate__(self):
        # the grid a wrapper prepared for the forward pass in progress is not part of the quantizer
        state = self.__dict__.copy()
        state.pop('_prepared_grid', None)
        return state

    def get_effective_encoding(self):
        """The encoding as the user's quant scheme means it: non-strict symmetric quantizers learn with max == -min
        and report min one step lower (reference :642-686)."""
        if not self.enabled:
            return None
        encodings = self.encoding
        if not encodings:
            return None
        if isinstance(encodings, libpymo.TfEncoding):
            encodings = [encodings]
        if is_non_strict_symmetric(self.use_symmetric_encodings, self.use_strict_symmetric,
                                   self.is_unsigned_symmetric):
            encodings = [libpymo.TfEncoding(e.min - e.delta, e.max, e.delta, e.offset, e.bw) for e in encodings]
        return encodings[0] if len(encodings) == 1 else encodings

    @property
    def encoding(self):
        """The learned encoding(s), recomputed from the current min / max parameters."""
        if not self.enabled or self.bitwidth == 32 or self.data_type == QuantizationDataType.float:
            return None
        return self._compute_updated_encoding()

    @encoding.setter
    def encoding(self, encoding):
        if not self.enabled or self.bitwidth == 32 or self.data_type == QuantizationDataType.float:
            return
        if encoding is None:
            raise RuntimeError("Encodings cannot be None if Quantizer is enabled.")
        bitwidth = encoding[0].bw if isinstance(encoding, list) else encoding.bw
        if bitwidth != self.bitwidth:
            raise RuntimeError(
                f"Bitwidth mismatched. The bitwidth for quantizer is {self.bitwidth}, but the bitwidth in encodings "
                f"is {bitwidth}. If the intent is to change the bitwidth, please set quantizer bitwidth to "
                f"{bitwidth} first.")
        if self._is_encoding_frozen:
            raise RuntimeError("Encoding can be set only when it is not frozen.")
        self._set_encoding_min_max_parameters(encoding)

    @property
    def channel_axis(self) -> int:
        return self._ch_axis

    @TensorQuantizer.encoding_min_max_fixed_vals.setter
    def encoding_min_max_fixed_vals(self, min_max_vals: Optional[Tuple[float, float]]):
        self._encoding_min_max_fixed_vals = min_max_vals

    def __str__(self):
        stream = io.StringIO(newline='\n')
        stream.write('LearnedGrid TensorQuantizer:\n')
        stream.write(f'    quant-scheme:{self._quant_scheme}, round_mode={self.round_mode}, '
                     f'bitwidth={self.bitwidth}, enabled={self.enabled}\n')
        encoding = self.get_effective_encoding() if self.encoding else None
        if encoding:
            for enc in (encoding if isinstance(encoding, list) else [encoding]):
                stream.write(f'    min:{enc.min}, max={enc.max}, delta={enc.delta}, offset={enc.offset}\n')
        else:
            stream.write('    no encoding\n')
        return stream.getvalue()

    def compute_scaling_offset(self, encoding_min, encoding_max):
        """(delta, offset) tensors for the given min / max tensors; (None, None) when they are None."""
        if encoding_min is None or encoding_max is None:
            return None, None
        scaling, offset, _ = grad_fn.get_computed_encodings(self.bitwidth, encoding_min, encoding_max,
                                                            self.use_symmetric_encodings, self.use_strict_symmetric,
                                                            self.is_unsigned_symmetric)
        return scaling, offset

    def quantize_dequantize(self, tensor: torch.Tensor, encoding_min: torch.nn.Parameter,
                            encoding_max: torch.nn.Parameter) -> torch.Tensor:
        if self.enabled:
            tensor = QuantizeDequantizeFunc.apply(tensor, encoding_min, encoding_max, self)
        return tensor

    @torch.no_grad()
    def _compute_updated_encoding(self):
        encoding_min, encoding_max = self._parameters_of_wrapper()
        if encoding_min is None or encoding_max is None:
            return None                       # not initialised yet
        emin, emax = encoding_min.detach().float(), encoding_max.detach().float()
        scale, offset = self.compute_scaling_offset(emin, emax)
        scale, offset = scale.expand_as(emin), offset.expand_as(emin)
        if not self.use_symmetric_encodings or self.is_unsigned_symmetric:
            # zero must be representable: min / max follow from delta and the rounded offset (reference :822-831)
            adjusted_min = scale * offset
            emax = emax - emin + adjusted_min
            emin = adjusted_min
        # one transfer for all channels
        table = torch.stack([emin, emax, scale, offset]).cpu().tolist()
        encodings = [libpymo.TfEncoding(mn, mx, d, o, self.bitwidth) for mn, mx, d, o in zip(*table)]
        return encodings[0] if len(encodings) == 1 else encodings

    def _set_encoding_min_max_parameters(self, encodings):
        if isinstance(encodings, list):
            assert isinstance(encodings[0], libpymo.TfEncoding), "Encodings should be a libpymo.TfEncoding() object"
            mins, maxs = [e.min for e in encodings], [e.max for e in encodings]
        else:
            assert isinstance(encodings, libpymo.TfEncoding), "Encodings should be a libpymo.TfEncoding() object"
            mins, maxs = [encodings.min], [encodings.max]
        params = self.wrapper_ref._parameters  # pylint: disable=protected-access
        device = self.wrapper_ref.device
        params[self.name + '_encoding_min'] = torch.nn.Parameter(torch.tensor(mins, dtype=torch.float32,
                                                                              device=device))
        params[self.name + '_encoding_max'] = torch.nn.Parameter(torch.tensor(maxs, dtype=torch.float32,
                                                                              device=device))

    def freeze_encoding(self):
        params = self.wrapper_ref._parameters  # pylint: disable=protected-access
        enc_min, enc_max = params[self.name + '_encoding_min'], params[self.name + '_encoding_max']
        if enc_min is None and enc_max is None:
            raise RuntimeError("Encoding can be frozen only when it is not None.")
        self._is_encoding_frozen = True
        enc_min.requires_grad = False
        enc_max.requires_grad = False


class QuantizeDequantizeFunc(torch.autograd.Function):
    """Quantize-dequantize with gradients w.r.t. the tensor and the learnable encoding min / max
    (reference :898-986).  Only the input tensor and the per-channel delta / offset are kept for backward."""

    @staticmethod
    def forward(ctx, tensor, encoding_min, encoding_max, tensor_quantizer):  # pylint: disable=arguments-differ
        ctx.tensor_quantizer = tensor_quantizer
        if tensor_quantizer.bitwidth == 32:
            return tensor
        if encoding_max is None or encoding_min is None:
            raise RuntimeError("Forward pass used for compute_encodings differs from forward pass used during "
                               "training")
        out, saved = grad_fn.learned_grid_forward(tensor, tensor_quantizer, encoding_min, encoding_max)
        ctx.is_symmetric = tensor_quantizer.use_symmetric_encodings
        # min / max are saved as copies: the wrapper clamps the parameters in place before every forward, also
        # between the forward and the backward of a module that is used twice (reference :942-955).  The library's
        # grid table holds such copies.
        if len(saved) == 4:
            ctx.saved_geometry = saved[1:]
            ctx.range_shapes = (encoding_min.shape, encoding_max.shape)
            ctx.save_for_backward(tensor, saved[0])
        else:
            ctx.saved_geometry = saved[2:]
            ctx.save_for_backward(tensor, saved[0], saved[1], encoding_min.detach().clone(),
                                  encoding_max.detach().clone())
        return out

    @staticmethod
    def backward(ctx, grad):  # pylint: disable=arguments-differ
        if ctx.tensor_quantizer.bitwidth == 32:
            return grad, None, None, None
        want_enc = ctx.needs_input_grad[1] or ctx.needs_input_grad[2]
        if len(ctx.saved_tensors) == 2:
            tensor, grid = ctx.saved_tensors
            saved, encoding_min, encoding_max = (grid,) + tuple(ctx.saved_geometry), grid[2], grid[3]
            shapes = ctx.range_shapes
        else:
            tensor, delta, offset, encoding_min, encoding_max = ctx.saved_tensors
            saved, shapes = (delta, offset) + tuple(ctx.saved_geometry), None
        tensor_grad, grad_min, grad_max = grad_fn.learned_grid_backward(
            tensor, grad, saved, encoding_min, encoding_max, ctx.is_symmetric, ctx.needs_input_grad[0], want_enc)
        if shapes is not None and grad_min is not None:
            grad_min, grad_max = grad_min.reshape(shapes[0]), grad_max.reshape(shapes[1])
        if not ctx.needs_input_grad[0]:
            tensor_grad = None
        return tensor_grad, grad_min if ctx.needs_input_grad[1] else None, \
            grad_max if ctx.needs_input_grad[2] else None, None


def initialize_learned_grid_quantizer_attributes(new_quantizer: LearnedGridTensorQuantizer,
                                                 old_quantizer: StaticGridTensorQuantizer):
    """Copies the user-settable attributes and the calibrated encoding of a static-grid quantizer into a learned-grid
    one (reference :1285-1345).  Signed symmetric encodings are made exactly symmetric (min = -max) first, and
    unsigned symmetric ones are turned into signed symmetric ones, because range learning keeps max == -min."""
    new_quantizer.enabled = old_quantizer.enabled
    new_quantizer.bitwidth = old_quantizer.bitwidth
    new_quantizer.data_type = old_quantizer.data_type
    new_quantizer.use_symmetric_encodings = old_quantizer.use_symmetric_encodings
    new_quantizer.use_strict_symmetric = old_quantizer.use_strict_symmetric
    new_quantizer.use_unsigned_symmetric = old_quantizer.use_unsigned_symmetric
    new_quantizer.is_unsigned_symmetric = False
    new_quantizer.encoding_min_max_fixed_vals = old_quantizer.encoding_min_max_fixed_vals
    new_quantizer.is_const = old_quantizer.is_const
    new_quantizer.is_singleton = old_quantizer.is_singleton
    if new_quantizer.data_type == QuantizationDataType.float or new_quantizer.bitwidth == 32:
        new_quantizer.encoding = None
        return
    old = old_quantizer.encoding
    encodings = old if isinstance(old, list) else ([old] if old is not None else [])
    if old_quantizer.enabled and old_quantizer.use_symmetric_encodings:
        half = (2 ** old_quantizer.bitwidth - 1) / 2
        for enc in encodings:
            enc.min = -enc.max
            if old_quantizer.is_unsigned_symmetric:
                enc.delta = enc.max / math.floor(half)
                enc.offset = -math.ceil(half)
    new_quantizer.encoding = old


def set_encoding_min_max_gating_threshold(encoding_min: torch.nn.Parameter, encoding_max: torch.nn.Parameter):
    """Learned min / max may drift out of order: min is kept <= 0, max >= 0 and max >= min + 1e-5
    (reference :1347-1359)."""
    with torch.no_grad():
        encoding_min.clamp_(max=0.0)
        encoding_max.clamp_(min=0.0)
        encoding_max.copy_(torch.maximum(encoding_max, encoding_min + 1e-5))
