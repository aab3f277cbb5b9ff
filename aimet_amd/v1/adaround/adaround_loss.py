"""Hyper-parameters and loss terms of AdaRound.

Mirrors TrainingExtensions/torch/src/python/aimet_torch/v1/adaround/adaround_loss.py: AdaroundHyperParameters
(:48-62), AdaroundLoss.compute_recon_loss (:70-80), compute_round_loss (:82-111), _compute_beta (:113-135).
The optimisation loop does not call compute_round_loss per iteration -- its gradient is fused into the backward
kernel -- but the function is kept for callers that want the value.
"""
from typing import Tuple

import numpy as np
import torch

from ...common.defs import AdaroundConstants


class AdaroundHyperParameters:
    """Hyper parameters of the per-layer optimisation."""

    def __init__(self, num_iterations: int, reg_param: float, beta_range: Tuple, warm_start: float):
        self.num_iterations = num_iterations
        self.reg_param = reg_param
        self.beta_range = beta_range
        self.warm_start = warm_start


class AdaroundLoss:
    """Reconstruction loss and rounding loss."""

    @staticmethod
    def compute_recon_loss(ada_quantized_output: torch.Tensor, orig_output: torch.Tensor) -> torch.Tensor:
        """Squared Frobenius norm over dim 1, averaged over the remaining dims."""
        return (torch.norm(ada_quantized_output - orig_output, p="fro", dim=1) ** 2).mean()

    @classmethod
    def in_warm_start(cls, opt_params: AdaroundHyperParameters, cur_iter: int) -> bool:
        return cur_iter < opt_params.num_iterations * opt_params.warm_start

    @classmethod
    def compute_round_loss(cls, alpha: torch.Tensor, opt_params: AdaroundHyperParameters, cur_iter: int):
        """reg_param * sum(1 - |2 h(alpha) - 1|^beta); 0 during the warm-start period."""
        if cls.in_warm_start(opt_params, cur_iter):
            return 0
        h_alpha = torch.clamp(torch.sigmoid(alpha) * (AdaroundConstants.ZETA - AdaroundConstants.GAMMA) +
                              AdaroundConstants.GAMMA, 0, 1)
        beta = cls._compute_beta(opt_params.num_iterations, cur_iter, opt_params.beta_range, opt_params.warm_start)
        reg_term = torch.add(1, -(torch.add(2 * h_alpha, -1).abs()).pow(beta)).sum()
        return opt_params.reg_param * reg_term

    @staticmethod
    def _compute_beta(max_iter: int, cur_iter: int, beta_range: Tuple, warm_start: float) -> float:
        """Cosine decay of beta from beta_range[0] to beta_range[1] after the warm-start period."""
        assert cur_iter < max_iter, 'Current iteration should be less than total maximum number of iterations.'
        start_beta, end_beta = beta_range
        warm_start_end_iter = warm_start * max_iter
        rel_iter = (cur_iter - warm_start_end_iter) / (max_iter - warm_start_end_iter)
        return end_beta + 0.5 * (start_beta - end_beta) * (1 + np.cos(rel_iter * np.pi))
