"""Sequential MSE on the v2 quantized modules.

Mirrors TrainingExtensions/torch/src/python/aimet_torch/v2/seq_mse.py: SequentialMse with the v2 overrides
(apply_seq_mse :68-99, _get_grouped_convs_with_blockwise_quantization :101-118, _handle_grouped_block_quantizers
:120-137, compute_all_param_encodings :139-148, temporarily_disable_quantizers :150-196, compute_param_encodings
:198-216, get_min_and_max_for_candidate_selection :263-312, _get_candidate :314-323, _compute_loss :325-357,
optimize_module :359-395).  Candidates are tensors of the weight quantizer's shape (per tensor, per channel) or of the
weight's shape (blockwise: every element carries its block's extreme), the loss is kept per output channel and per
block of input channels, and the winner is chosen per block.  The walk over the model, the sampling of layer inputs and
the checkpointed flow are those of the v1 path.
"""
import contextlib
from typing import List, Optional, Tuple

import torch
from torch import nn

from .. import ops
from ..v1.seq_mse import SUPPORTED_MODULES, SeqMseParams, SequentialMse as V1SequentialMse, default_forward_fn  # noqa: F401
from .nn import BaseQuantizationMixin
from .quantization.affine import GroupedBlockQuantizeDequantize, QuantizeDequantize
from .quantsim import QuantizationSimModel
from .utils import reshape_tensor_for_blocks


def _reduced_to(tensor: torch.Tensor, shape, extreme) -> torch.Tensor:
    """`tensor` reduced by `extreme` (torch.amax / torch.amin) over every axis along which `shape`, aligned from the
    right, has one entry; the result has exactly `shape`."""
    shape = tuple(shape)
    aligned = (1,) * (tensor.dim() - len(shape)) + shape
    axes = [axis for axis, (have, want) in enumerate(zip(tensor.shape, aligned)) if want == 1 and have != 1]
    return (extreme(tensor, dim=axes, keepdim=True) if axes else tensor).reshape(shape)


class SequentialMse(V1SequentialMse):
    """Weight encodings of the v2 simulation model by minimizing each layer's output error, layer after layer."""

    @classmethod
    def apply_seq_mse(cls, model: nn.Module, sim: QuantizationSimModel, data_loader, params: SeqMseParams,
                      modules_to_exclude: Optional[List[nn.Module]] = None, checkpoints_config: Optional[str] = None):
        # pylint: disable=too-many-arguments
        # grouped convolutions whose blocks cut through a group's input channels cannot be searched block by block
        modules_to_exclude = list(modules_to_exclude or []) + cls._get_grouped_convs_with_blockwise_quantization(sim)
        with cls._handle_grouped_block_quantizers(sim):
            super().apply_seq_mse(model, sim, data_loader, params, modules_to_exclude, checkpoints_config)

    @staticmethod
    def _get_grouped_convs_with_blockwise_quantization(sim) -> List[nn.Module]:
        found = []
        for module in sim.model.modules():
            if isinstance(module, nn.Conv2d) and isinstance(module, BaseQuantizationMixin) and module.groups != 1:
                quantizer = module.param_quantizers['weight']
                block_size = getattr(quantizer, 'block_size', None)
                if block_size is not None and block_size[1] != module.weight.shape[1]:
                    found.append(module)
        return found

    @staticmethod
    @contextlib.contextmanager
    def _handle_grouped_block_quantizers(sim: QuantizationSimModel):
        """Inside the `with`, grouped blockwise quantizers behave as plain blockwise ones (every block its own group):
        the search picks a range per block."""
        grouped = [(q, q.block_grouping) for q in sim.model.modules() if isinstance(q, GroupedBlockQuantizeDequantize)]
        for quantizer, _ in grouped:
            quantizer.block_grouping = tuple(1 for _ in quantizer.shape)
        try:
            yield
        finally:
            for quantizer, grouping in grouped:
                quantizer.block_grouping = grouping

    @staticmethod
    def compute_all_param_encodings(sim: QuantizationSimModel):
        for _, qmodule in sim.named_qmodules():
            qmodule._compute_param_encodings(overwrite=True)       # pylint: disable=protected-access

    @staticmethod
    @contextlib.contextmanager
    def temporarily_disable_quantizers(model: nn.Module, sim: QuantizationSimModel, modules_to_exclude):
        """Inside the `with`, activation quantizers are out of every quantized module, and so are the parameter
        quantizers of unsupported module types and of the excluded modules (given as modules of `model`, or of the
        simulation model)."""
        # pylint: disable=protected-access, arguments-differ
        float_modules = dict(model.named_modules())
        excluded = modules_to_exclude or []
        put_back = []
        try:
            for name, qmodule in sim.named_qmodules():
                put_back.append(qmodule._remove_activation_quantizers())
                skipped = any(other is qmodule or other is float_modules.get(name) for other in excluded)
                if skipped or not isinstance(qmodule, SUPPORTED_MODULES):
                    put_back.append(qmodule._remove_param_quantizers())
            yield
        finally:
            for undo in reversed(put_back):
                undo._cleanup()

    @staticmethod
    def _weight_bitwidth(quant_module) -> int:
        quantizer = quant_module.param_quantizers['weight']
        return quantizer.bitwidth if quantizer is not None else 1 << 30    # not quantized: never searched

    _observers = {}

    @staticmethod
    def compute_param_encodings(quantizer, x_min: torch.Tensor, x_max: torch.Tensor):
        """min / max of `quantizer` as a fresh min-max quantizer of its geometry sets them on observing x_min, x_max."""
        # one observer per geometry serves every candidate of a search (and the next layer of the same geometry):
        # building a quantizer module costs more than observing a candidate
        block_size = None if quantizer.block_size is None else tuple(quantizer.block_size)
        key = (tuple(quantizer.shape), quantizer.bitwidth, quantizer.symmetric, block_size, x_min.device)
        observer = SequentialMse._observers.get(key)
        if observer is None:
            if len(SequentialMse._observers) >= 8:
                SequentialMse._observers.clear()
            observer = SequentialMse._observers[key] = QuantizeDequantize(
                quantizer.shape, quantizer.bitwidth, quantizer.symmetric,
                block_size=quantizer.block_size).to(x_min.device)
        with observer.compute_encodings():
            observer(torch.stack([x_min, x_max]))
        with torch.no_grad():
            quantizer.min.copy_(observer.min)
            quantizer.max.copy_(observer.max)

    @staticmethod
    def _is_symmetric_quantizer(quantizer) -> bool:
        return quantizer.symmetric

    @staticmethod
    def _freeze_quantizer_encoding(quantizer):
        quantizer.requires_grad_(False)
        quantizer.allow_overwrite(False)

    @staticmethod
    def _get_quantized_weight(quant_module: BaseQuantizationMixin) -> torch.Tensor:
        return quant_module.param_quantizers['weight'](quant_module.weight)

    @staticmethod
    def _get_original_module(quant_module: BaseQuantizationMixin) -> nn.Module:
        return quant_module                                          # a v2 quantized module is the module

    @staticmethod
    def _get_input_channel_block_size(quant_module) -> int:
        if not isinstance(quant_module, (nn.Linear, nn.Conv2d)):
            raise NotImplementedError('Unsupported module type: ', type(quant_module))
        quantizer = quant_module.param_quantizers['weight']
        if quantizer.block_size is None:
            return quant_module.weight.shape[1]
        return quant_module.weight.shape[1] // quantizer.shape[1]

    @classmethod
    def get_min_and_max_for_candidate_selection(cls, quant_module: BaseQuantizationMixin) \
            -> Tuple[torch.Tensor, torch.Tensor]:
        """The extremes the candidates are fractions of: of the quantizer's shape without blocks; with blocks, of the
        weight's shape, every element holding the extreme of its block."""
        if not isinstance(quant_module, (nn.Conv2d, nn.Linear)):
            raise ValueError('Unsupported module: ', quant_module)
        quantizer = quant_module.param_quantizers['weight']
        weight = quant_module.weight.detach()
        symmetric = cls._is_symmetric_quantizer(quantizer)
        if quantizer.block_size is None:
            if symmetric:
                top = _reduced_to(weight.abs(), quantizer.shape, torch.amax)
                return -top, top
            return _reduced_to(weight, quantizer.shape, torch.amin), _reduced_to(weight, quantizer.shape, torch.amax)
        in_blocks = reshape_tensor_for_blocks(weight, quantizer.shape, quantizer.block_size)
        # reshaped as (blocks, block size) pairs per axis: the block-size axes are every second one, from the last
        within = [in_blocks.dim() - 1 - 2 * k for k in range(len(quantizer.block_size))][::-1]
        if symmetric:
            top = torch.maximum(in_blocks, torch.amax(in_blocks.abs(), within, keepdim=True)).reshape(weight.shape)
            return -top, top
        top = torch.maximum(in_blocks, torch.amax(in_blocks, within, keepdim=True)).reshape(weight.shape)
        bottom = torch.minimum(in_blocks, torch.amin(in_blocks, within, keepdim=True)).reshape(weight.shape)
        return bottom, top

    @staticmethod
    def _get_candidate(candidate_idx, num_candidates: int, min_tensor: torch.Tensor, max_tensor: torch.Tensor):
        """Fraction (candidate_idx + 1) / num_candidates of the range; the index may be a tensor (one per block)."""
        return min_tensor / num_candidates * (candidate_idx + 1), max_tensor / num_candidates * (candidate_idx + 1)

    @classmethod
    def _compute_loss(cls, quant_module, x, xq, w, wq, params) -> torch.Tensor:
        """[output channels, blocks of input channels]: the loss of each block's partial product on its own."""
        # pylint: disable=too-many-arguments
        block = cls._get_input_channel_block_size(quant_module)
        channel_axis = -1 if isinstance(quant_module, nn.Linear) else -3
        losses = []
        for w_part, wq_part, x_part, xq_part in zip(torch.split(w, block, dim=1), torch.split(wq, block, dim=1),
                                                    torch.split(x, block, dim=channel_axis),
                                                    torch.split(xq, block, dim=channel_axis)):
            xqwq, xw = cls.compute_outputs(quant_module, x_part, xq_part, w_part, wq_part)
            losses.append(cls.compute_recon_loss(xqwq, xw, params))
        return torch.stack(losses, dim=-1)

    # ---- Linear layers: all blocks of input channels in one batched GEMM
    # The block-by-block loop above costs two small GEMMs per block, batch and candidate (5120 launches of each kind for
    # 32 blocks, 4 batches, 20 candidates).  For a Linear layer the partial products of all blocks are one batched GEMM,
    # [blocks, rows, block] x [blocks, block, out] -> [blocks, rows, out], and the float side does not depend on the
    # candidate: it is formed once per batch while it fits `_FLOAT_PRODUCTS_BYTES`.
    _FLOAT_PRODUCTS_BYTES = 16 << 30

    @staticmethod
    def _rows_in_blocks(inputs: torch.Tensor, block: int) -> torch.Tensor:
        """[..., in] -> [blocks, rows, block]"""
        rows = inputs.reshape(-1, inputs.shape[-1])
        return rows.reshape(rows.shape[0], -1, block).permute(1, 0, 2)

    @staticmethod
    def _weight_in_blocks(weight: torch.Tensor, block: int) -> torch.Tensor:
        """[out, in] -> [blocks, block, out]"""
        return weight.reshape(weight.shape[0], -1, block).permute(1, 2, 0)

    @staticmethod
    def _block_losses(products_q: torch.Tensor, products: torch.Tensor, loss_fn: str) -> torch.Tensor:
        """[blocks, rows, out] twice -> [out, blocks]: compute_recon_loss for every block at once, both tensors read
        once (as tensor operations: a subtraction, a square and a sum, six passes)."""
        rows = products.shape[1]
        if loss_fn == "mse":
            per_block = ops.column_error(products_q, products, ops.COLUMN_ERROR_SQUARED)
        elif loss_fn == "l1":
            per_block = ops.column_error(products_q, products, ops.COLUMN_ERROR_ABSOLUTE)
        elif loss_fn == "sqnr":
            noise, signal = ops.column_error(products_q, products, ops.COLUMN_ERROR_SQUARED_AND_SIGNAL)
            per_block = -10 * torch.log10((signal / rows) / (noise / rows + 1e-10))
        else:
            raise ValueError(f"Invalid loss function: {loss_fn}")
        return per_block.t()

    @classmethod
    def _linear_candidate_losses(cls, quant_module, x, xq, params, candidates):
        """For a Linear layer: yields nothing, drives `candidates` -- a generator that sets one candidate's encodings
        per step -- and returns the list of [out, blocks] losses, one per candidate."""
        block = cls._get_input_channel_block_size(quant_module)
        w = quant_module.weight.detach()
        batches = range(params.num_batches)
        same_inputs = xq is x
        rows = [cls._rows_in_blocks(x[b], block) for b in batches]
        rows_q = rows if same_inputs else [cls._rows_in_blocks(xq[b], block) for b in batches]
        w_blocks = cls._weight_in_blocks(w, block)
        kept_bytes = sum(r.shape[0] * r.shape[1] for r in rows) * w.shape[0] * w.element_size()
        keep = kept_bytes <= cls._FLOAT_PRODUCTS_BYTES
        products = [torch.bmm(r, w_blocks) for r in rows] if keep else None
        losses = []
        for _ in candidates:
            wq_blocks = cls._weight_in_blocks(cls._get_quantized_weight(quant_module), block)
            loss = None
            for b in batches:
                target = products[b] if keep else torch.bmm(rows[b], w_blocks)
                part = cls._block_losses(torch.bmm(rows_q[b], wq_blocks), target, params.loss_fn)
                loss = part if loss is None else loss.add_(part)
            losses.append(loss)
        return losses

    @classmethod
    def _conv_candidate_losses(cls, quant_module, x, xq, params, candidates):
        """For a convolution: `_compute_loss` per candidate and batch, with the float side -- the partial outputs of
        every block of input channels, which no candidate changes -- formed once per batch while it fits."""
        block = cls._get_input_channel_block_size(quant_module)
        w = quant_module.weight.detach()
        batches = range(params.num_batches)
        parts = lambda t: torch.split(t, block, dim=-3)
        w_parts = torch.split(w, block, dim=1)
        outputs = lambda inputs, weights: [cls._layer_output(quant_module, i, k) for i, k in zip(inputs, weights)]
        first = outputs(parts(x[0]), w_parts)
        kept_bytes = sum(o.numel() for o in first) * w.element_size() * params.num_batches
        keep = kept_bytes <= cls._FLOAT_PRODUCTS_BYTES
        kept = [first] + [outputs(parts(x[b]), w_parts) for b in batches[1:]] if keep else None
        del first
        losses = []
        for _ in candidates:
            wq_parts = torch.split(cls._get_quantized_weight(quant_module), block, dim=1)
            loss = None
            for b in batches:
                targets = kept[b] if keep else outputs(parts(x[b]), w_parts)
                part = torch.stack([cls.compute_recon_loss(got, want, params)
                                    for got, want in zip(outputs(parts(xq[b]), wq_parts), targets)], dim=-1)
                loss = part if loss is None else loss.add_(part)
            losses.append(loss)
        return losses

    @classmethod
    def optimize_module(cls, quant_module: BaseQuantizationMixin, x: torch.Tensor, xq: torch.Tensor,
                        params: SeqMseParams):
        quantizer = quant_module.param_quantizers['weight']
        min_tensor, max_tensor = cls.get_min_and_max_for_candidate_selection(quant_module)

        def candidates():
            for index in range(params.num_candidates):
                cand_min, cand_max = cls._get_candidate(index, params.num_candidates, min_tensor, max_tensor)
                cls.compute_param_encodings(quantizer, cand_min, cand_max)
                yield index

        if isinstance(quant_module, nn.Linear):
            with torch.no_grad():
                total_loss = cls._linear_candidate_losses(quant_module, x, xq, params, candidates())
        else:
            with torch.no_grad():
                total_loss = cls._conv_candidate_losses(quant_module, x, xq, params, candidates())
        best = torch.stack(total_loss).min(0)[1]                     # [output channels, blocks]
        block = cls._get_input_channel_block_size(quant_module)
        if block != quant_module.weight.shape[1]:
            best = best.repeat_interleave(block, dim=-1)             # one index per input channel
        while best.dim() < max_tensor.dim():
            best = best[..., None]
        best_min, best_max = cls._get_candidate(best, params.num_candidates, min_tensor, max_tensor)
        cls.compute_param_encodings(quantizer, best_min, best_max)
        cls._freeze_quantizer_encoding(quantizer)


# module-level names, as the reference offers them
apply_seq_mse = SequentialMse.apply_seq_mse
get_candidates = SequentialMse.get_candidates
optimize_module = SequentialMse.optimize_module
