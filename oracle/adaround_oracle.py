"""CPU restatement of the reference's AdaRound arithmetic -- TEST INFRASTRUCTURE, never imported by the product.

Plain torch ops on CPU tensors with torch's own autograd and torch.optim.Adam, following, statement for statement
(paths relative to the reference root, ADA = TrainingExtensions/torch/src/python/aimet_torch/v1/adaround):

  generate_alpha        ADA/adaround_wrapper.py:211-224  (AdaroundWrapper._generate_alpha_parameter)
  apply_adaround        ADA/adaround_wrapper.py:124-149  (AdaroundWrapper.apply_adaround)
  compute_recon_loss    ADA/adaround_loss.py:70-80
  compute_round_loss    ADA/adaround_loss.py:82-111
  compute_beta          ADA/adaround_loss.py:113-135
  layer_output          ADA/adaround_optimizer.py:253-283 (_compute_output_with_adarounded_weights)
  optimize_rounding     ADA/adaround_optimizer.py:155-218 (the iteration loop of _optimize_rounding, with the batch
                        indices supplied by the caller so that both sides of a parity test see the same batches)

Pinned by the reference's own known answers (tests/golden/reference_vectors.json, section "adaround"): beta of the
cosine schedule, the rounding loss of a seeded alpha, the reconstruction losses and hard/soft reconstruction errors
of a seeded 1x1 convolution (TrainingExtensions/torch/test/python/test_adaround_loss.py:76-100,
test_adaround_optimizer.py:122-196), plus closed forms: h(generate_alpha(w)) equals the fractional part of w/delta,
hard rounding at alpha = generate_alpha(w) equals round-to-nearest, and finite-difference checks of the gradients.
"""
import math

import numpy as np
import torch
import torch.nn.functional as F

GAMMA = -0.1   # aimet_common/defs.py:305
ZETA = 1.1     # aimet_common/defs.py:306


def broadcast(vec, like, ch_axis):
    """quantsim_straight_through_grad.py:66-88 (broadcast_to_tensor)"""
    vec = torch.as_tensor(vec, dtype=torch.float32)
    if vec.numel() == 1:
        return vec.reshape(())
    shape = [1] * like.dim()
    shape[ch_axis] = like.shape[ch_axis]
    return vec.view(shape)


def generate_alpha(weight, delta):
    tensor_floor = torch.floor(weight / delta)
    tensor = (weight / delta) - tensor_floor
    alpha = -torch.log((ZETA - GAMMA) / (tensor - GAMMA) - 1)
    return alpha.float()


def rectified_sigmoid(alpha):
    return torch.clamp(torch.sigmoid(alpha) * (ZETA - GAMMA) + GAMMA, 0, 1)


def apply_adaround(weight, alpha, delta, offset, clip_min, clip_max, use_soft_rounding):
    tensor = torch.floor(weight / delta)
    if use_soft_rounding:
        h_alpha = rectified_sigmoid(alpha)
    else:
        h_alpha = (alpha >= 0).to(tensor.dtype)
    tensor = tensor + h_alpha
    tensor_quant = torch.clamp(tensor - offset, clip_min, clip_max)
    return (tensor_quant + offset) * delta


def compute_recon_loss(ada_quantized_output, orig_output):
    return (torch.norm(ada_quantized_output - orig_output, p="fro", dim=1) ** 2).mean()


def compute_beta(max_iter, cur_iter, beta_range, warm_start):
    start_beta, end_beta = beta_range
    warm_start_end_iter = warm_start * max_iter
    rel_iter = (cur_iter - warm_start_end_iter) / (max_iter - warm_start_end_iter)
    return end_beta + 0.5 * (start_beta - end_beta) * (1 + np.cos(rel_iter * np.pi))


def compute_round_loss(alpha, num_iterations, reg_param, beta_range, warm_start, cur_iter):
    if cur_iter < num_iterations * warm_start:
        return 0
    h_alpha = rectified_sigmoid(alpha)
    beta = compute_beta(num_iterations, cur_iter, beta_range, warm_start)
    reg_term = torch.add(1, -(torch.add(2 * h_alpha, -1).abs()).pow(beta)).sum()
    return reg_param * reg_term


def layer_output(kind, inp, weight, bias=None, **conv_args):
    if kind == "linear":
        return F.linear(inp, weight, bias=bias)
    if kind == "conv2d":
        return F.conv2d(inp, weight, bias=bias, **conv_args)
    if kind == "conv_transpose2d":
        return F.conv_transpose2d(inp, weight, bias=bias, **conv_args)
    raise ValueError(kind)


def optimize_rounding(kind, weight, alpha0, delta, offset, clip_min, clip_max, all_inp, all_out, batches,
                      num_iterations, reg_param, beta_range, warm_start, bias=None, act=None, ch_axis=0,
                      conv_args=None, first_iteration=0, trace=None):
    """Runs len(batches) iterations; returns (alpha, exp_avg, exp_avg_sq, last alpha.grad).

    `batches` is a list of index tensors (what torch.randperm(...)[:BATCH_SIZE] yields in the reference).
    `trace`, when a list, receives (recon_loss, round_loss) floats per iteration.
    """
    conv_args = conv_args or {}
    alpha = torch.nn.Parameter(alpha0.clone())
    d = broadcast(delta, weight, ch_axis)
    o = broadcast(offset, weight, ch_axis)
    optimizer = torch.optim.Adam([alpha])
    for k, idx in enumerate(batches):
        iteration = first_iteration + k
        inp, orig = all_inp[idx], all_out[idx]
        optimizer.zero_grad()
        w_ada = apply_adaround(weight, alpha, d, o, clip_min, clip_max, True)
        quant_out = layer_output(kind, inp, w_ada, bias, **conv_args)
        if act is not None:
            orig = act(orig)
            quant_out = act(quant_out)
        recon = compute_recon_loss(quant_out, orig)
        rnd = compute_round_loss(alpha, num_iterations, reg_param, beta_range, warm_start, iteration)
        (recon + rnd).backward()
        if trace is not None:
            trace.append((float(recon.detach()), float(rnd.detach()) if torch.is_tensor(rnd) else float(rnd)))
        optimizer.step()
    state = optimizer.state[alpha]
    return alpha.detach(), state["exp_avg"], state["exp_avg_sq"], alpha.grad
