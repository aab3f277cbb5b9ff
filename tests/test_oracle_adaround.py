"""Pins the AdaRound restatement (oracle/adaround_oracle.py) to the reference's known answers and to closed forms.

Known answers: TrainingExtensions/torch/test/python/test_adaround_loss.py:76-100 (beta, rounding loss) and
test_adaround_optimizer.py:122-196 (hard / soft reconstruction errors and reconstruction loss of a seeded 1x1
convolution whose encoding comes from the TF-Enhanced analyzer).
"""
import math

import numpy as np
import pytest
import torch

from oracle import adaround_oracle as ada


@pytest.fixture(scope="module")
def golden(vectors):
    return vectors["adaround"]


def test_beta_known_answer(golden):
    b = golden["beta"]
    assert ada.compute_beta(b["max_iter"], b["cur_iter"], tuple(b["beta_range"]), b["warm_start"]) == b["expected"]
    # closed forms of the cosine schedule: start of annealing, middle, (one past the) end
    assert ada.compute_beta(10000, 2000, (20, 2), 0.2) == 20
    assert ada.compute_beta(10000, 6000, (20, 2), 0.2) == pytest.approx(11.0, abs=1e-12)
    assert ada.compute_beta(10000, 10000, (20, 2), 0.2) == pytest.approx(2.0, abs=1e-12)


def test_round_loss_known_answer(golden):
    r = golden["round_loss"]
    np.random.seed(r["np_seed"])
    alpha = torch.from_numpy(np.random.rand(*r["alpha_shape"]))
    args = (r["num_iterations"], r["reg_param"], (20, 2), 0.2)
    assert ada.compute_round_loss(alpha, *args, 10) == 0
    assert ada.compute_round_loss(alpha, *args, r["warm_start_iter"]) == r["warm_start_expected"]
    loss = ada.compute_round_loss(alpha, *args, r["cur_iter"])
    assert loss.item() == pytest.approx(r["expected"], abs=10 ** -r["places"])


def test_recon_loss_equals_summed_mse():
    # test_adaround_loss.py:51-74
    np.random.seed(0)
    for shape in ((32, 3, 12, 12), (32, 10)):
        a, b = torch.from_numpy(np.random.rand(*shape)), torch.from_numpy(np.random.rand(*shape))
        expect = torch.nn.functional.mse_loss(a, b, reduction='none').sum(1).mean().item()
        assert ada.compute_recon_loss(a, b).item() == pytest.approx(expect, abs=1e-5)


def _seeded_conv_case(golden, oracle):
    g = golden["recons_metrics"]
    np.random.seed(g["np_seed"])
    weight = np.random.rand(*g["weight_shape"]).astype('float32')
    pdf = oracle.new_pdf()
    pdf.update(weight.reshape(-1))
    enc, _, _ = pdf.compute_encoding(g["weight_bw"], g["symmetric"])
    inp = np.random.rand(*g["inp_shape"]).astype('float32')
    out = np.random.rand(*g["out_shape"]).astype('float32')
    return g, torch.from_numpy(weight), enc, torch.from_numpy(inp), torch.from_numpy(out)


def test_recons_metrics_known_answer(golden, oracle):
    g, weight, enc, inp, out = _seeded_conv_case(golden, oracle)
    assert enc.delta == pytest.approx(g["scale"], abs=10 ** -g["scale_places"])
    delta = torch.tensor(enc.delta, dtype=torch.float32)
    offset = torch.tensor(enc.offset, dtype=torch.float32)
    alpha = ada.generate_alpha(weight, delta)
    clip_max = 2 ** g["weight_bw"] - 1
    errs = {}
    for soft in (False, True):
        w = ada.apply_adaround(weight, alpha, delta, offset, 0, clip_max, soft)
        y = ada.layer_output("conv2d", inp, w)
        errs[soft] = torch.nn.functional.mse_loss(y, out).item()
        if soft:
            assert ada.compute_recon_loss(y, out).item() == pytest.approx(g["recon_loss_soft"],
                                                                          abs=10 ** -g["cuda_places"])
    assert errs[False] == pytest.approx(g["recons_err_hard"], abs=10 ** -g["places"])
    assert errs[True] == pytest.approx(g["recons_err_soft"], abs=10 ** -g["places"])


def test_alpha_init_reproduces_fraction_and_nearest_rounding():
    """h(generate_alpha(w)) is the fractional part of w / delta, so soft rounding at the initial alpha gives back the
    weight itself (inside the grid) and hard rounding gives round-to-nearest."""
    torch.manual_seed(3)
    weight = torch.randn(8, 37) * 0.3
    delta = (torch.rand(8) * 0.02 + 0.01)
    offset = torch.full((8,), -128.0)
    d, o = ada.broadcast(delta, weight, 0), ada.broadcast(offset, weight, 0)
    alpha = ada.generate_alpha(weight, d)
    frac = weight / d - torch.floor(weight / d)
    assert torch.allclose(ada.rectified_sigmoid(alpha), frac, atol=2e-6)
    inside = (weight / d > -127.5) & (weight / d < 126.5)
    soft = ada.apply_adaround(weight, alpha, d, o, 0, 255, True)
    assert torch.allclose(soft[inside], weight[inside], atol=1e-6)
    hard = ada.apply_adaround(weight, alpha, d, o, 0, 255, False)
    nearest = torch.clamp(torch.floor(weight / d + 0.5) - o, 0, 255)
    decided = (frac - 0.5).abs() > 1e-4          # away from ties, where alpha's sign is numerically certain
    assert torch.equal(((hard / d) - o).round()[decided & inside], nearest[decided & inside])


def test_gradients_by_finite_differences():
    """Autograd of the restatement against central differences in float64 (catches a dropped factor or sign in any
    hand-derived gradient that is later compared with it)."""
    torch.manual_seed(5)
    weight = (torch.randn(4, 6) * 0.2).double()
    delta = torch.tensor(0.05).double()
    offset = torch.tensor(-8.0).double()
    alpha = torch.randn(4, 6).double().requires_grad_(True)
    inp, tgt = torch.randn(5, 6).double(), torch.randn(5, 4).double()

    def loss_fn(a):
        w = ada.apply_adaround(weight, a, delta, offset, 0, 15, True)
        y = torch.relu(ada.layer_output("linear", inp, w))
        return ada.compute_recon_loss(y, torch.relu(tgt)) + ada.compute_round_loss(a, 100, 0.01, (20, 2), 0.2, 60)

    assert torch.autograd.gradcheck(loss_fn, (alpha,), eps=1e-6, atol=1e-5)


def test_adam_trajectory_matches_hand_written_update():
    """torch.optim.Adam inside optimize_rounding against the textbook update written out in float64."""
    torch.manual_seed(7)
    weight = torch.randn(6, 10) * 0.1
    delta, offset = torch.full((6,), 0.02), torch.full((6,), -8.0)
    alpha0 = ada.generate_alpha(weight, ada.broadcast(delta, weight, 0))
    all_inp, all_out = torch.randn(64, 10), torch.randn(64, 6)
    batches = [torch.randperm(64)[:32] for _ in range(5)]
    alpha, m, v, grad = ada.optimize_rounding("linear", weight, alpha0, delta, offset, 0, 15, all_inp, all_out,
                                              batches, 5, 0.01, (20, 2), 0.2)
    # replay: gradients from autograd, update by hand
    a = alpha0.clone().double()
    m2, v2 = torch.zeros_like(a), torch.zeros_like(a)
    d, o = ada.broadcast(delta, weight, 0).double(), ada.broadcast(offset, weight, 0).double()
    for t, idx in enumerate(batches, start=1):
        p = a.clone().float().requires_grad_(True)
        w = ada.apply_adaround(weight, p, d.float(), o.float(), 0, 15, True)
        loss = ada.compute_recon_loss(ada.layer_output("linear", all_inp[idx], w), all_out[idx]) + \
            ada.compute_round_loss(p, 5, 0.01, (20, 2), 0.2, t - 1)
        g, = torch.autograd.grad(loss, p)
        g = g.double()
        m2 = 0.9 * m2 + 0.1 * g
        v2 = 0.999 * v2 + 0.001 * g * g
        a = a - 1e-3 / (1 - 0.9 ** t) * m2 / (v2.sqrt() / math.sqrt(1 - 0.999 ** t) + 1e-8)
    assert torch.allclose(alpha.double(), a, atol=5e-6)
    assert torch.allclose(m.double(), m2, rtol=1e-4, atol=1e-9)
