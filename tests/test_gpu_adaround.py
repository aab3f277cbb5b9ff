"""GPU parity of the AdaRound kernels and of the AdaRound flow against the CPU restatement of the reference
(oracle/adaround_oracle.py: torch CPU ops, torch autograd and torch.optim.Adam), through the C ABI.

Accuracy of the per-element terms is measured in ulp against float64 evaluated on the same float32 inputs
(test_term_accuracy_in_ulp), next to what torch's float32 CPU ops reach on the same inputs:
  h(alpha)             |error| <= 2 ulp(1)                      (torch CPU: 1.4)
  dh/dalpha            <= 8 ulp                                  (torch CPU: 11.4, from the cancellation in 1 - sigmoid)
  1 - |2h - 1|^beta    |error| <= 1.25 ulp(1)                    (torch CPU: 0.5)
  its derivative in h  <= 2.5 ulp                                (torch CPU: 1.3 ... 8.3)
The alpha gradient is the float32 combination of those terms, bit for bit (test_alpha_gradient).  Against the CPU
restatement's autograd it can only be compared up to the conditioning both sides share: a last-bit difference in h
moves |2h - 1|^(beta - 1) by (beta - 1) / |2h - 1| last bits, which is where the 2e-5 of the largest gradient comes from.
Adam: both moments equal torch.optim.Adam's on the CPU bit for bit given the same gradients; alpha in all but about one
element in a thousand per step, those by one ulp (test_adam_update_against_torch_cpu).
Trajectories over N iterations (GEMMs with different summation orders on the two sides):
  alpha after N Adam iterations  5e-5 absolute (lr = 1e-3, so this is 5 % of one step) for 99.9 % of the elements;
                       elements that crossed a clamp boundary may differ by a few steps (see _close_except_few)
"""
import json
import math
import os

import numpy as np
import pytest
import torch

from oracle import adaround_oracle as ada

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    from aimet_amd import ops as o
    return o


def _case(seed, shape, ch_axis, per_channel, bw=4):
    g = torch.Generator().manual_seed(seed)
    weight = torch.randn(*shape, generator=g) * 0.05
    num_channel = shape[ch_axis] if per_channel else 1
    if per_channel:
        red = [d for d in range(len(shape)) if d != ch_axis]
        absmax = weight.abs().amax(dim=red)
    else:
        absmax = weight.abs().max().reshape(1)
    # a grid a little narrower than the weight range, so that the clamp to [clip_min, clip_max] is exercised
    delta = (absmax * 1.7 / (2 ** bw - 1)).float()
    offset = torch.full((num_channel,), float(-2 ** (bw - 1)))
    n_per_channel = int(np.prod(shape[ch_axis + 1:])) if per_channel else int(np.prod(shape))
    return weight, delta, offset, num_channel, n_per_channel, 0.0, float(2 ** bw - 1)


CASES = [((64, 96), 0, True), ((7, 5, 3, 3), 0, True), ((6, 8, 3, 3), 1, True), ((33, 17), 0, False),
         ((1, 3), 0, True), ((512, 512), 0, True)]


@pytest.mark.parametrize("shape,ch_axis,per_channel", CASES)
def test_init_alpha_and_soft_round(ops, shape, ch_axis, per_channel):
    weight, delta, offset, C, npc, cmin, cmax = _case(11, shape, ch_axis, per_channel)
    d, o = ada.broadcast(delta, weight, ch_axis), ada.broadcast(offset, weight, ch_axis)
    alpha_ref = ada.generate_alpha(weight, d)
    wg, dg, og = weight.cuda(), delta.cuda(), offset.cuda()
    alpha = ops.adaround_init_alpha(wg, C, npc, dg)
    assert torch.allclose(alpha.cpu(), alpha_ref, atol=2e-6, rtol=0)
    # same alpha on both sides from here on; perturb it so that h leaves the initial fractional part
    torch.manual_seed(1)
    alpha_ref = alpha_ref + torch.randn_like(alpha_ref) * 2.0
    ag = alpha_ref.cuda()
    hard = ops.adaround_soft_round(wg, ag, C, npc, dg, og, cmin, cmax, False).cpu()
    assert torch.equal(hard, ada.apply_adaround(weight, alpha_ref, d, o, cmin, cmax, False))
    soft = ops.adaround_soft_round(wg, ag, C, npc, dg, og, cmin, cmax, True).cpu()
    soft_ref = ada.apply_adaround(weight, alpha_ref, d, o, cmin, cmax, True)
    # floor(w/delta) + h is rounded to float32 at magnitudes up to 2^bw: a one-ulp difference in sigmoid moves the sum
    # by one ulp of that magnitude, and the result by that times delta
    assert torch.allclose(soft, soft_ref, atol=float(4 * 2.0 ** -23 * 16 * delta.max()), rtol=0)


def _ulps(got, want64):
    """|got - want| in units of the float32 spacing at |want|."""
    want64 = np.asarray(want64, np.float64)
    spacing = np.maximum(np.spacing(np.abs(want64).astype(np.float32)).astype(np.float64), 2.0 ** -149)
    return np.abs(got.astype(np.float64) - want64) / spacing


def test_term_accuracy_in_ulp(ops):
    """The kernels' own sigmoid / h / dh and regulariser terms against float64 on the same float32 inputs, alpha over
    [-12, 12] and beta over the schedule's range; torch's float32 CPU ops on the same inputs for comparison."""
    g = torch.Generator().manual_seed(0)
    edge = math.log(11.0)                                # h leaves / reaches the clamp at sigmoid = 1/12 and 11/12
    alpha = torch.cat([torch.linspace(-12, 12, 2_000_001), torch.randn(1_000_000, generator=g) * 2.5,
                       edge + (torch.rand(200_000, generator=g) - 0.5) * 1e-3,
                       -edge + (torch.rand(200_000, generator=g) - 0.5) * 1e-3,
                       torch.tensor([0.0, -0.0, 30.0, -30.0, 88.0, -88.0, 100.0, -100.0, float("inf"), -float("inf")])])
    a64 = alpha.numpy().astype(np.float64)
    with np.errstate(over="ignore"):
        sig64 = 1.0 / (1.0 + np.exp(-a64))
    zeta_gamma, gamma = np.float64(np.float32(ada.ZETA - ada.GAMMA)), np.float64(np.float32(ada.GAMMA))
    inner64 = sig64 * zeta_gamma + gamma
    h64 = np.clip(inner64, 0, 1)
    dh64 = np.where((inner64 >= 0) & (inner64 <= 1), zeta_gamma * sig64 * (1 - sig64), 0.0)
    sig, h, dh = (t.cpu().numpy() for t in ops.adaround_eval_terms(alpha.cuda(), 0))
    at = alpha.clone().requires_grad_(True)
    ht = ada.rectified_sigmoid(at)
    ht.sum().backward()
    sig_t, h_t, dh_t = torch.sigmoid(alpha).numpy(), ht.detach().numpy(), at.grad.numpy()
    assert np.isfinite(sig).all() and np.isfinite(h).all() and np.isfinite(dh).all()
    assert np.array_equal(sig[-2:], [1.0, 0.0]) and np.array_equal(dh[-6:], np.zeros(6))
    open_range = np.abs(a64) <= 2.5                      # where the clamp is open and sigmoid's value matters
    inside = (inner64 > 1e-3) & (inner64 < 1 - 1e-3)
    decided = inside | (inner64 < -1e-6) | (inner64 > 1 + 1e-6)
    report = {
        "sigmoid, |alpha| <= 2.5 [ulp]": (_ulps(sig, sig64)[open_range].max(), _ulps(sig_t, sig64)[open_range].max(), 4.0),
        "sigmoid, |alpha| <= 12 [ulp]": (_ulps(sig, sig64)[np.abs(a64) <= 12].max(),
                                         _ulps(sig_t, sig64)[np.abs(a64) <= 12].max(), 16.0),
        "h [ulp(1)]": (np.abs(h - h64).max() / 2.0 ** -23, np.abs(h_t - h64).max() / 2.0 ** -23, 2.0),
        "dh/dalpha [ulp]": (_ulps(dh, dh64)[inside].max(), _ulps(dh_t, dh64)[inside].max(), 8.0),
    }
    assert np.array_equal((dh == 0)[decided], (dh64 == 0)[decided])
    # the regulariser's terms as functions of a float32 h
    hh = torch.cat([torch.rand(2_000_000, generator=g), 0.5 + (torch.rand(300_000, generator=g) - 0.5) * 1e-3,
                    torch.rand(200_000, generator=g) * 1e-3, 1 - torch.rand(200_000, generator=g) * 1e-3,
                    torch.tensor([0.0, 1.0, 0.5, 0.25, 0.75, 2.0 ** -25, 0.5 + 2.0 ** -25])])
    x32 = (2 * hh.numpy() - 1).astype(np.float32)       # the float32 2h - 1 every float32 implementation forms
    x64 = np.abs(x32).astype(np.float64)
    for beta in (2.0, 2.000492, 4.636038969321072, 11.0, 20.0):
        b32, bm1 = np.float64(np.float32(beta)), np.float64(np.float32(beta - 1.0))   # torch's pow takes float32
        reg64 = 1 - x64 ** b32
        dreg64 = -b32 * x64 ** bm1 * np.sign(x32) * 2
        reg, dreg = (t.cpu().numpy() for t in ops.adaround_eval_terms(hh.cuda(), 1, beta))
        hv = hh.clone().requires_grad_(True)
        rt = torch.add(1, -(torch.add(2 * hv, -1).abs()).pow(beta))
        rt.sum().backward()
        normal = np.abs(dreg64) > 1e-30
        report[f"1 - |2h-1|^beta, beta {beta:g} [ulp(1)]"] = (np.abs(reg - reg64).max() / 2.0 ** -23,
                                                             np.abs(rt.detach().numpy() - reg64).max() / 2.0 ** -23, 1.25)
        report[f"d/dh of it, beta {beta:g} [ulp]"] = (_ulps(dreg, dreg64)[normal].max(),
                                                      _ulps(hv.grad.numpy(), dreg64)[normal].max(), 2.5)
        assert reg[-7] == 0 and reg[-6] == 0 and abs(dreg[-7]) == abs(dreg[-6]) == np.float32(2 * beta)   # h = 0, 1: |2h - 1| = 1
    for name, (gpu, cpu, bound) in report.items():
        print(f"{name:42s} gpu {gpu:7.2f}   torch cpu {cpu:7.2f}   bound {bound}")
    for name, (gpu, cpu, bound) in report.items():
        assert gpu <= bound, name


def test_adam_update_against_torch_cpu(ops):
    """30 updates with the kernel's own gradient output replayed through torch.optim.Adam on the CPU."""
    torch.manual_seed(5)
    O, K = 64, 512
    w = torch.randn(O, K) * 0.05
    delta, offset = (w.abs().amax(dim=1) * 1.7 / 15).float(), torch.full((O,), -8.0)
    alpha = torch.randn(O, K) * 2
    ag, mg, vg = alpha.cuda(), torch.zeros(O, K).cuda(), torch.zeros(O, K).cuda()
    p = torch.nn.Parameter(alpha.clone())
    opt = torch.optim.Adam([p])
    for step in range(1, 31):
        gw = torch.randn(O, K) * 10 ** float(torch.randn(1))
        gout = torch.empty(O, K, device="cuda")
        ops.adaround_bwd_adam(w.cuda(), gw.cuda(), ag, mg, vg, O, K, delta.cuda(), offset.cuda(), 0.0, 15.0, 0.01,
                              20 - step * 0.5, 1e-3, 0.9, 0.999, 1e-8, step, grad_alpha=gout)
        p.grad = gout.cpu()
        opt.step()
    state = opt.state[p]
    assert torch.equal(mg.cpu(), state["exp_avg"]) and torch.equal(vg.cpu(), state["exp_avg_sq"])
    diff = (ag.cpu() - p.detach()).numpy().astype(np.float64)
    same = (diff == 0).mean()
    # a differing update moves alpha by one ulp of alpha, or (alpha near zero) by the few 1e-7 of the lr-sized step that
    # the one-ulp square root and reciprocal leave
    allowed = np.maximum(2 * np.spacing(np.abs(p.detach().numpy())), 30 * 1e-3 * 1e-6)
    print(f"alpha after 30 updates: identical {same:.5f}, largest difference {np.abs(diff).max():.3g}")
    assert same > 0.97 and (np.abs(diff) <= allowed).all()


@pytest.mark.parametrize("shape,ch_axis,per_channel", CASES[:4])
@pytest.mark.parametrize("beta", [-1.0, 20.0, 4.636038969321072, 2.0])
def test_alpha_gradient(ops, shape, ch_axis, per_channel, beta):
    weight, delta, offset, C, npc, cmin, cmax = _case(13, shape, ch_axis, per_channel)
    d, o = ada.broadcast(delta, weight, ch_axis), ada.broadcast(offset, weight, ch_axis)
    torch.manual_seed(2)
    alpha = (ada.generate_alpha(weight, d) + torch.randn_like(weight) * 2.5).requires_grad_(True)
    grad_w = torch.randn_like(weight)
    reg_param = 0.01
    loss = (ada.apply_adaround(weight, alpha, d, o, cmin, cmax, True) * grad_w).sum()
    reg_ref = None
    if beta >= 0:
        h = ada.rectified_sigmoid(alpha)
        reg_ref = torch.add(1, -(torch.add(2 * h, -1).abs()).pow(beta)).sum()
        loss = loss + reg_param * reg_ref
    loss.backward()
    partial = torch.zeros(ops.adaround_blocks(weight.numel()), device="cuda")
    got = ops.adaround_bwd(weight.cuda(), grad_w.cuda(), alpha.detach().cuda(), C, npc, delta.cuda(), offset.cuda(),
                           cmin, cmax, reg_param, beta, partial).cpu()
    # the gradient is the float32 combination of the terms whose accuracy test_term_accuracy_in_ulp bounds:
    #   (clip_min <= floor(w / delta) + h - offset <= clip_max ? grad_w delta dh : 0) + reg_param dreg dh
    f32 = np.float32
    _, h_g, dh_g = (t.cpu().numpy().reshape(weight.shape) for t in ops.adaround_eval_terms(alpha.detach().cuda(), 0))
    dn, on = np.broadcast_to(d.numpy(), weight.shape), np.broadcast_to(o.numpy(), weight.shape)
    t = np.floor(weight.numpy() / dn) + h_g - on
    want = np.where((t >= f32(cmin)) & (t <= f32(cmax)), grad_w.numpy() * dn * dh_g, f32(0))
    if beta >= 0:
        _, dreg_g = ops.adaround_eval_terms(torch.from_numpy(h_g).cuda(), 1, beta)
        want = want + f32(reg_param) * dreg_g.cpu().numpy().reshape(weight.shape) * dh_g
    assert np.array_equal(got.numpy().view(np.uint32), want.astype(f32).view(np.uint32))
    # against the restatement's autograd: up to the conditioning of |2h - 1|^(beta - 1) in h (see the module docstring)
    scale = alpha.grad.abs().max().item()
    assert torch.allclose(got, alpha.grad, atol=2e-5 * scale, rtol=2e-5)
    # same zero pattern: the clamp masks are decided identically
    assert torch.equal(got == 0, alpha.grad == 0)
    if beta >= 0:
        assert partial.sum().item() == pytest.approx(reg_ref.item(), rel=1e-5)


def _close_except_few(x, ref, atol, rtol=0.0, max_frac=1e-3):
    """allclose for all but a fraction `max_frac` of the elements.

    Over many iterations a few elements sit on a clamp boundary (sigmoid(alpha) * 1.2 - 0.1 within an ulp of 0 or 1,
    or floor(w/delta) + h - offset within an ulp of a grid limit), where a last-bit difference in sigmoid decides
    whether torch.clamp passes the gradient in that iteration; for those the GPU and the CPU legitimately take a
    different step."""
    bad = (x - ref).abs() > atol + rtol * ref.abs()
    return bad.float().mean().item() <= max_frac


class _Layer:
    """What AdaroundOptimizer reads from an AdaroundWrapper, without a QuantizationSimModel around it."""

    def __init__(self, module, alpha0, delta, offset, C, npc, cmin, cmax):
        self._module = module
        self.weight = module.weight
        self.alpha = torch.nn.Parameter(alpha0.clone().cuda())
        self.delta, self.offset = delta.cuda(), offset.cuda()
        self.num_channel, self.n_per_channel, self.clip_min, self.clip_max = C, npc, cmin, cmax
        self.use_soft_rounding = True

    def get_original_module(self):
        return self._module


def _run_product_loop(kind, weight, alpha0, delta, offset, C, npc, cmin, cmax, all_inp, all_out, batches, hyper, act,
                      conv_args):
    from aimet_amd.v1.adaround.adaround_loss import AdaroundHyperParameters
    from aimet_amd.v1.adaround.adaround_optimizer import AdaroundOptimizer
    if kind == "linear":
        module = torch.nn.Linear(weight.shape[1], weight.shape[0], bias=False)
    else:
        module = torch.nn.Conv2d(weight.shape[1], weight.shape[0], weight.shape[2], bias=False, **conv_args)
    module.weight.data = weight.clone()
    module.cuda()
    layer = _Layer(module, alpha0, delta, offset, C, npc, cmin, cmax)
    m, v = AdaroundOptimizer.optimize_rounding_on_cached_acts(layer, act, all_inp.cuda(), all_out.cuda(),
                                                              AdaroundHyperParameters(*hyper), batches=batches)
    return layer.alpha.detach().cpu(), m.cpu(), v.cpu(), layer.alpha.grad.cpu()


@pytest.mark.parametrize("kind,act", [("linear", None), ("linear", torch.relu), ("conv2d", torch.relu)])
def test_optimisation_trajectory(ops, kind, act):
    iters = 40
    hyper = (iters, 0.01, (20, 2), 0.2)
    if kind == "linear":
        shape, conv_args = (48, 64), {}
        torch.manual_seed(21)
        all_inp = torch.randn(128, 64)
    else:
        shape, conv_args = (8, 6, 3, 3), {"padding": 1}
        torch.manual_seed(22)
        all_inp = torch.randn(96, 6, 9, 9)
    weight, delta, offset, C, npc, cmin, cmax = _case(17, shape, 0, True)
    d = ada.broadcast(delta, weight, 0)
    alpha0 = ada.generate_alpha(weight, d)
    all_out = ada.layer_output(kind, all_inp, weight, **conv_args)          # the fp32 layer's output
    batches = [torch.randperm(all_inp.size(0))[:32] for _ in range(iters)]
    trace = []
    a_ref, m_ref, v_ref, g_ref = ada.optimize_rounding(kind, weight, alpha0, delta, offset, cmin, cmax, all_inp,
                                                       all_out, batches, *hyper, act=act, conv_args=conv_args,
                                                       trace=trace)
    a, m, v, g = _run_product_loop(kind, weight, alpha0, delta, offset, C, npc, cmin, cmax, all_inp, all_out, batches,
                                   hyper, act, conv_args)
    assert (a_ref - alpha0).abs().max() > 5e-3          # the loop did move alpha
    assert _close_except_few(a, a_ref, atol=5e-5)
    assert (a - a_ref).abs().max() < 5e-3
    assert _close_except_few(g, g_ref, atol=1e-4 * g_ref.abs().max().item(), rtol=1e-3)
    assert _close_except_few(m, m_ref, atol=1e-4 * m_ref.abs().max().item(), rtol=1e-3)
    assert _close_except_few(v, v_ref, atol=1e-4 * v_ref.abs().max().item(), rtol=1e-3)


@pytest.mark.parametrize("shape,per_channel,act,batch", [
    ((128, 512), True, 0, 32), ((64, 256), False, 1, 32), ((192, 768), True, 1, 32),
    # in_features that end in half a backward tile, and 2 / 4 / 8 blocks of 32 rows
    ((64, 128), True, 0, 32), ((96, 384), False, 1, 32), ((64, 384), True, 1, 64), ((96, 128), False, 0, 128),
    ((128, 640), True, 1, 256), ((64, 512), True, 0, 256), ((160, 256), False, 1, 128)])
def test_fused_linear_forward_and_backward(ops, shape, per_channel, act, batch):
    """The MFMA-fused Linear kernels against the elementwise kernels around torch's own GEMM on the GPU (same
    per-element arithmetic, different summation order in the GEMMs) and against the CPU restatement."""
    O, K = shape
    weight, delta, offset, C, npc, cmin, cmax = _case(31, shape, 0, per_channel)
    weight[1, 5] *= 6.0                                 # far outside the grid on both sides
    weight[2, 7] = -weight[2].abs().max() * 5.0
    weight[3, 9] = weight[3].abs().max() * 5.0
    torch.manual_seed(32)
    X, bias = torch.randn(300, K), torch.randn(O) * 0.1
    Y = torch.nn.functional.linear(X, weight, bias) + torch.randn(300, O) * 0.01
    idx = torch.randperm(300)[:batch]
    d, o = ada.broadcast(delta, weight, 0), ada.broadcast(offset, weight, 0)
    alpha = ada.generate_alpha(weight, d) + torch.randn_like(weight)
    wg, ag, dg, og, Xg, Yg, bg = (t.cuda() for t in (weight, alpha, delta, offset, X, Y, bias))
    ig = idx.to(torch.int32).cuda()
    ws = ops.adaround_linear_workspace(O, K, "cuda", batch)
    G = torch.empty(batch, O, device="cuda")
    out = torch.empty(batch, O, device="cuda")
    lp = torch.zeros((batch * O + 255) // 256, device="cuda")
    fg = ops.adaround_floor(wg, C, npc, dg)
    assert torch.equal(fg.cpu(), torch.floor(weight / d))
    ops.adaround_linear_fwd(fg, ag, Xg, ig, Yg, bg, C, dg, og, cmin, cmax, act, ws, G, out=out, loss_partial=lp)

    # CPU restatement
    a_ref = alpha.clone().requires_grad_(True)
    w_ref = ada.apply_adaround(weight, a_ref, d, o, cmin, cmax, True)
    out_ref = ada.layer_output("linear", X[idx], w_ref, bias)
    out_ref.retain_grad()
    f = torch.relu if act else (lambda t: t)
    loss_ref = ada.compute_recon_loss(f(out_ref), f(Y[idx]))
    loss_ref.backward()
    scale = out_ref.abs().max().item()
    assert torch.allclose(out.cpu(), out_ref.detach(), atol=2e-5 * scale, rtol=1e-5)
    gscale = out_ref.grad.abs().max().item()
    assert torch.allclose(G.cpu(), out_ref.grad, atol=1e-4 * gscale, rtol=1e-4)
    assert lp.sum().item() == pytest.approx(loss_ref.item(), rel=1e-4)

    # backward + Adam: fused against (torch GEMM + elementwise kernel) on the same G, and against the CPU gradient
    hyper = dict(reg_param=0.01, beta=7.5, lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8, step=3)
    m0, v0 = torch.rand_like(weight) * 1e-3, torch.rand_like(weight) * 1e-6
    a1, m1, v1 = ag.clone(), m0.cuda(), v0.cuda()
    g1 = torch.empty_like(a1)
    rp1 = torch.zeros(ops.adaround_linear_blocks(O, K), device="cuda")
    ops.adaround_linear_bwd_adam(fg, G, Xg, ig, a1, m1, v1, C, dg, og, cmin, cmax, reg_partial=rp1, grad_alpha=g1,
                                 **hyper)
    a2, m2, v2 = ag.clone(), m0.cuda(), v0.cuda()
    g2 = torch.empty_like(a2)
    rp2 = torch.zeros(ops.adaround_blocks(O * K), device="cuda")
    dW = (G.double().t() @ Xg[idx.cuda()].double()).float().contiguous()
    ops.adaround_bwd_adam(wg, dW, a2, m2, v2, C, npc, dg, og, cmin, cmax, reg_partial=rp2, grad_alpha=g2, **hyper)
    gs = g2.abs().max().item()
    assert torch.allclose(g1, g2, atol=2e-5 * gs, rtol=1e-4)
    assert torch.equal(g1 == 0, g2 == 0)
    assert torch.allclose(a1, a2, atol=2e-6, rtol=0)
    assert torch.allclose(m1, m2, atol=2e-5 * m2.abs().max().item(), rtol=1e-4)
    assert torch.allclose(v1, v2, atol=2e-5 * v2.abs().max().item(), rtol=1e-4)
    assert rp1.sum().item() == pytest.approx(rp2.sum().item(), rel=1e-5)
    # floor(W / delta) stored as int8: saturated to the window outside which its value cannot matter; everything the
    # two kernels produce from it is identical, bit for bit, to what they produce from the float32 form
    f8 = ops.adaround_floor_i8(wg, C, npc, dg, og, cmin, cmax)
    assert f8 is not None and f8.dtype == torch.int8
    lo, hi = o + cmin - 2, o + cmax + 1
    assert torch.equal(f8.cpu().float(), torch.minimum(torch.maximum(torch.floor(weight / d), lo), hi))
    assert (torch.floor(weight / d) < lo).any() and (torch.floor(weight / d) > hi).any()   # saturation happens
    G8, out8, lp8 = torch.empty_like(G), torch.empty_like(out), torch.zeros_like(lp)
    ops.adaround_linear_fwd(f8, ag, Xg, ig, Yg, bg, C, dg, og, cmin, cmax, act, ws, G8, out=out8, loss_partial=lp8)
    assert torch.equal(out8, out) and torch.equal(G8, G) and torch.equal(lp8, lp)
    a8, m8, v8 = ag.clone(), m0.cuda(), v0.cuda()
    g8, rp8 = torch.empty_like(a8), torch.zeros_like(rp1)
    ops.adaround_linear_bwd_adam(f8, G, Xg, ig, a8, m8, v8, C, dg, og, cmin, cmax, reg_partial=rp8, grad_alpha=g8,
                                 **hyper)
    assert torch.equal(a8, a1) and torch.equal(m8, m1) and torch.equal(v8, v1) and torch.equal(g8, g1)
    assert torch.equal(rp8, rp1)
    # a grid of 8 bits does not fit int8 (the window is 259 values wide) and goes to int16: same results again
    assert ops.adaround_floor_i8(wg, C, npc, dg, og, 0, 255) is None
    assert ops.adaround_floor_i8(wg, C, npc, dg, og + 200, cmin, cmax) is None
    assert ops.adaround_floor_packed(wg, C, npc, dg, og, cmin, cmax).dtype == torch.int8
    d8, o8 = dg / 16, og * 16                            # the 8-bit grid over the same range
    f16 = ops.adaround_floor_packed(wg, C, npc, d8, o8, 0, 255)
    assert f16.dtype == torch.int16
    f32 = ops.adaround_floor(wg, C, npc, d8)
    lo16 = ada.broadcast(o8.cpu(), weight, 0) - 2
    hi16 = ada.broadcast(o8.cpu(), weight, 0) + 256
    assert torch.equal(f16.cpu().float(), torch.minimum(torch.maximum(f32.cpu(), lo16), hi16))
    res = []
    for fl in (f32, f16):
        Gx, ax, mx_, vx, gx = torch.empty_like(G), ag.clone(), m0.cuda(), v0.cuda(), torch.empty_like(ag)
        ops.adaround_linear_fwd(fl, ag, Xg, ig, Yg, bg, C, d8, o8, 0, 255, act, ws, Gx)
        ops.adaround_linear_bwd_adam(fl, Gx, Xg, ig, ax, mx_, vx, C, d8, o8, 0, 255, grad_alpha=gx, **hyper)
        res.append((Gx, ax, mx_, vx, gx))
    for t32, t16 in zip(*res):
        assert torch.equal(t32, t16)
    assert ops.adaround_floor_int(wg, C, npc, dg / 4096, og * 4096, 0, 65535, torch.int16) is None   # 16-bit grid

    # CPU gradient of the full loss (reconstruction + regulariser) w.r.t. alpha
    h = ada.rectified_sigmoid(a_ref)
    reg = hyper["reg_param"] * torch.add(1, -(torch.add(2 * h, -1).abs()).pow(hyper["beta"])).sum()
    g_reg, = torch.autograd.grad(reg, a_ref)
    g_cpu = a_ref.grad + g_reg
    assert torch.allclose(g1.cpu(), g_cpu, atol=1e-4 * g_cpu.abs().max().item(), rtol=1e-3)


def test_fused_linear_rejects_other_shapes(ops):
    from aimet_amd._lib import MiqError
    w = torch.zeros(48, 256, device="cuda")
    with pytest.raises(MiqError):
        ops.adaround_linear_fwd(w, w, torch.zeros(32, 256, device="cuda"), None, torch.zeros(32, 48, device="cuda"),
                                None, 1, torch.ones(1, device="cuda"), torch.zeros(1, device="cuda"), 0, 15, 0,
                                torch.zeros(32 * 48, device="cuda"), torch.zeros(32, 48, device="cuda"))
    assert not ops.adaround_linear_supported(48, 256, 32)
    assert not ops.adaround_linear_supported(64, 192, 32) and ops.adaround_linear_supported(64, 128, 32)
    assert not ops.adaround_linear_supported(64, 256, 96) and ops.adaround_linear_supported(64, 256, 256)
    w = torch.zeros(64, 256, device="cuda")
    with pytest.raises(MiqError, match="32, 64, 128 or 256"):
        ops.adaround_linear_fwd(w, w, torch.zeros(96, 256, device="cuda"), None, torch.zeros(96, 64, device="cuda"),
                                None, 1, torch.ones(1, device="cuda"), torch.zeros(1, device="cuda"), 0, 15, 0,
                                torch.zeros(96 * 64 * 8, device="cuda"), torch.zeros(96, 64, device="cuda"))
    # fewer than 32 cached rows and no row index: refused before any launch
    w = torch.zeros(64, 256, device="cuda")
    with pytest.raises(MiqError, match="num_rows"):
        ops.adaround_linear_fwd(w, w, torch.zeros(16, 256, device="cuda"), None, torch.zeros(16, 64, device="cuda"),
                                None, 1, torch.ones(1, device="cuda"), torch.zeros(1, device="cuda"), 0, 15, 0,
                                ops.adaround_linear_workspace(64, 256, "cuda"), torch.zeros(32, 64, device="cuda"))


def test_fused_linear_row_index_out_of_range(ops):
    """A batch index beyond the cached rows: IndexError from the optimizer before anything is launched (as the
    reference's tensor indexing raises); through the C ABI the read stays inside the buffers and that row's results
    are NaN."""
    from aimet_amd.v1.adaround.adaround_loss import AdaroundHyperParameters
    from aimet_amd.v1.adaround.adaround_optimizer import AdaroundOptimizer
    weight, delta, offset, C, npc, cmin, cmax = _case(51, (64, 256), 0, True)
    alpha0 = ada.generate_alpha(weight, ada.broadcast(delta, weight, 0))
    torch.manual_seed(52)
    X, Y = torch.randn(40, 256), torch.randn(40, 64)
    module = torch.nn.Linear(256, 64, bias=False)
    module.weight.data = weight.clone()
    layer = _Layer(module.cuda(), alpha0, delta, offset, C, npc, cmin, cmax)
    good = torch.randperm(40)[:32]
    for bad_value in (40, -41):
        bad = good.clone()
        bad[7] = bad_value
        with pytest.raises(IndexError):
            AdaroundOptimizer.optimize_rounding_on_cached_acts(layer, None, X.cuda(), Y.cuda(),
                                                               AdaroundHyperParameters(2, 0.01, (20, 2), 0.2),
                                                               batches=[good, bad])
    assert torch.equal(layer.alpha.detach().cpu(), alpha0)          # nothing ran
    wg, dg, og = weight.cuda(), delta.cuda(), offset.cuda()
    fl = ops.adaround_floor(wg, C, npc, dg)
    ws = ops.adaround_linear_workspace(64, 256, "cuda")
    G, out = torch.empty(32, 64, device="cuda"), torch.empty(32, 64, device="cuda")
    bad = good.clone()
    bad[7], bad[20] = 1 << 30, -5
    ops.adaround_linear_fwd(fl, alpha0.cuda(), X.cuda(), bad.to(torch.int32).cuda(), Y.cuda(), None, C, dg, og, cmin,
                            cmax, 0, ws, G, out=out)
    rows_nan = torch.isnan(G).all(dim=1).cpu()
    assert rows_nan.tolist() == [i in (7, 20) for i in range(32)]
    assert torch.isnan(out[7]).all() and torch.isfinite(out[6]).all()
    assert not ops.adaround_linear_supported(64, 256, 16)
    assert ops.adaround_linear_supported(4096, 4096, 32)


@pytest.mark.parametrize("act", [None, torch.relu])
@pytest.mark.parametrize("per_channel", [True, False])
def test_fused_optimisation_trajectory(ops, act, per_channel, monkeypatch):
    """40 iterations through AdaroundOptimizer on a Linear layer whose shape takes the fused kernels, against the CPU
    restatement on the same batches."""
    iters = 40
    hyper = (iters, 0.01, (20, 2), 0.2)
    shape = (64, 256)
    torch.manual_seed(41)
    all_inp = torch.randn(160, 256)
    weight, delta, offset, C, npc, cmin, cmax = _case(43, shape, 0, per_channel)
    alpha0 = ada.generate_alpha(weight, ada.broadcast(delta, weight, 0))
    # the target is not exactly reproducible by the layer: with an exactly reproducible one the gradient of every
    # output channel without a clipped weight is rounding noise, which Adam normalises into full-size random steps
    all_out = ada.layer_output("linear", all_inp, weight) + 0.02 * torch.randn(160, 64)
    batches = [torch.randperm(all_inp.size(0))[:32] for _ in range(iters)]
    a_ref, m_ref, v_ref, g_ref = ada.optimize_rounding("linear", weight, alpha0, delta, offset, cmin, cmax, all_inp,
                                                       all_out, batches, *hyper, act=act)
    calls = []
    real = ops.adaround_linear_fwd
    monkeypatch.setattr(ops, "adaround_linear_fwd", lambda *a, **k: (calls.append(1), real(*a, **k))[1])
    a, m, v, g = _run_product_loop("linear", weight, alpha0, delta, offset, C, npc, cmin, cmax, all_inp, all_out,
                                   batches, hyper, act, {})
    assert len(calls) == iters                          # the fused path ran
    from aimet_amd.v1.adaround.adaround_optimizer import AdaroundOptimizer
    assert AdaroundOptimizer.use_int8_floor
    monkeypatch.setattr(AdaroundOptimizer, "use_int8_floor", False)
    a32, m32, v32, g32 = _run_product_loop("linear", weight, alpha0, delta, offset, C, npc, cmin, cmax, all_inp,
                                           all_out, batches, hyper, act, {})
    for got, want in ((a, a32), (m, m32), (v, v32), (g, g32)):
        assert torch.equal(got, want)                   # int8 and float32 storage of floor(W / delta): same trajectory
    assert (a_ref - alpha0).abs().max() > 5e-3
    assert _close_except_few(a, a_ref, atol=5e-5)
    assert (a - a_ref).abs().max() < 5e-3               # and nowhere by more than a few steps of lr = 1e-3
    assert _close_except_few(g, g_ref, atol=1e-4 * g_ref.abs().max().item(), rtol=1e-3)
    assert _close_except_few(m, m_ref, atol=1e-4 * m_ref.abs().max().item(), rtol=1e-3)
    assert _close_except_few(v, v_ref, atol=1e-4 * v_ref.abs().max().item(), rtol=1e-3)


@pytest.mark.parametrize("kind,shape,pixels,batch,per_channel", [
    ("conv2d", (64, 128, 1, 1), (1, 1), 32, True),      # a 1x1 convolution on pooled features: 32 rows
    ("conv2d", (32, 256, 1, 1), (2, 2), 32, True),      # 4 pixels: 128 rows
    ("conv2d", (64, 384, 1, 1), (2, 4), 32, False),     # 8 pixels: 256 rows, half a backward tile at the end
    ("conv2d", (32, 128, 1, 1), (1, 2), 32, True),      # 64 rows
    ("linear", (64, 384), None, 64, True),
    ("linear", (96, 256), None, 128, False)])
def test_fused_path_for_more_rows_and_1x1_convolutions(ops, kind, shape, pixels, batch, per_channel, monkeypatch):
    """30 iterations through AdaroundOptimizer on layers the widened fused path takes -- batches of 64 and 128 rows,
    in_features that are a multiple of 128 only, 1x1 convolutions whose rows are the pixels of the 32 images -- against
    the CPU restatement (functional.conv2d / functional.linear under autograd and torch.optim.Adam) on the same
    batches, and against the unfused product path (soft-rounding kernel, torch's layer, fused backward kernel)."""
    from aimet_amd.v1.adaround.adaround_optimizer import AdaroundOptimizer
    iters = 30
    hyper = (iters, 0.01, (20, 2), 0.2)
    act = torch.relu
    torch.manual_seed(61)
    samples = 3 * batch
    all_inp = torch.randn(samples, shape[1], *pixels) if kind == "conv2d" else torch.randn(samples, shape[1])
    weight, delta, offset, C, npc, cmin, cmax = _case(63, shape, 0, per_channel)
    alpha0 = ada.generate_alpha(weight, ada.broadcast(delta, weight, 0))
    all_out = ada.layer_output(kind, all_inp, weight)
    all_out = all_out + 0.02 * torch.randn_like(all_out)      # see test_fused_optimisation_trajectory
    batches = [torch.randperm(samples)[:batch] for _ in range(iters)]
    a_ref, m_ref, v_ref, g_ref = ada.optimize_rounding(kind, weight, alpha0, delta, offset, cmin, cmax, all_inp,
                                                       all_out, batches, *hyper, act=act)
    calls = []
    real = ops.adaround_linear_fwd
    monkeypatch.setattr(ops, "adaround_linear_fwd", lambda *a, **k: (calls.append(a[13].shape), real(*a, **k))[1])
    rows = batch * (pixels[0] * pixels[1] if pixels else 1)
    if rows > AdaroundOptimizer.fused_rows_limit:
        # 256 rows go through the general path by default (it is the faster one there); the kernels take them
        a, _, _, _ = _run_product_loop(kind, weight, alpha0, delta, offset, C, npc, cmin, cmax, all_inp, all_out,
                                       batches[:2], hyper, act, {})
        assert calls == []
        monkeypatch.setattr(AdaroundOptimizer, "fused_rows_limit", 256)
    a, m, v, g = _run_product_loop(kind, weight, alpha0, delta, offset, C, npc, cmin, cmax, all_inp, all_out,
                                   batches, hyper, act, {})
    assert calls == [(rows, shape[0])] * iters            # the fused path ran, on that many rows
    monkeypatch.setattr(AdaroundOptimizer, "use_fused_linear", False)
    a_u, m_u, v_u, g_u = _run_product_loop(kind, weight, alpha0, delta, offset, C, npc, cmin, cmax, all_inp, all_out,
                                           batches, hyper, act, {})
    assert len(calls) == iters
    assert a.shape == weight.shape and (a_ref - alpha0).abs().max() > 5e-3
    for got, want, scale in ((a, a_ref, None), (a, a_u, None), (g, g_ref, g_ref), (g, g_u, g_ref), (m, m_ref, m_ref),
                             (m, m_u, m_ref), (v, v_ref, v_ref), (v, v_u, v_ref)):
        if scale is None:
            assert _close_except_few(got, want, atol=5e-5) and (got - want).abs().max() < 5e-3
        else:
            assert _close_except_few(got, want, atol=1e-4 * scale.abs().max().item(), rtol=1e-3)


@pytest.mark.parametrize("kind,shape,conv_args,act", [
    ("conv2d", (8, 6, 3, 3), {"padding": 1}, torch.relu), ("conv2d", (8, 6, 3, 3), {"padding": 1, "stride": 2}, None),
    ("conv2d", (8, 4, 3, 3), {"padding": 2, "dilation": 2, "groups": 2}, torch.relu), ("linear", (48, 64), {}, torch.relu),
    ("linear", (48, 64), {}, None)])
def test_written_out_gradient_equals_autograd(ops, kind, shape, conv_args, act, monkeypatch):
    """The general path forms dLoss/dW' of the reconstruction loss by hand for Conv2d / Linear with no activation or
    ReLU.  Same trajectory as with autograd's recording of the same operations (to the summation order of the
    convolution's weight-gradient kernel), and both against the CPU restatement."""
    from aimet_amd.v1.adaround.adaround_optimizer import AdaroundOptimizer
    iters = 25
    hyper = (iters, 0.01, (20, 2), 0.2)
    torch.manual_seed(71)
    cin = shape[1] * conv_args.get("groups", 1)
    all_inp = torch.randn(96, cin, 9, 9) if kind == "conv2d" else torch.randn(96, shape[1])
    weight, delta, offset, C, npc, cmin, cmax = _case(73, shape, 0, True)
    alpha0 = ada.generate_alpha(weight, ada.broadcast(delta, weight, 0))
    all_out = ada.layer_output(kind, all_inp, weight, **conv_args)
    all_out = all_out + 0.02 * torch.randn_like(all_out)
    batches = [torch.randperm(96)[:32] for _ in range(iters)]
    monkeypatch.setattr(AdaroundOptimizer, "use_fused_linear", False)
    calls = []
    real = AdaroundOptimizer._recon_loss_weight_gradient.__func__
    monkeypatch.setattr(AdaroundOptimizer, "_recon_loss_weight_gradient",
                        classmethod(lambda cls, *a: (calls.append(1), real(cls, *a))[1]))
    run = lambda: _run_product_loop(kind, weight, alpha0, delta, offset, C, npc, cmin, cmax, all_inp, all_out, batches,
                                    hyper, act, conv_args)
    a, m, v, g = run()
    assert len(calls) == iters
    monkeypatch.setattr(AdaroundOptimizer, "use_explicit_gradient", False)
    a2, m2, v2, g2 = run()
    assert len(calls) == iters
    assert _close_except_few(a, a2, atol=5e-5) and (a - a2).abs().max() < 5e-3
    assert _close_except_few(g, g2, atol=1e-5 * g2.abs().max().item(), rtol=1e-4)
    assert _close_except_few(m, m2, atol=1e-5 * m2.abs().max().item(), rtol=1e-4)
    a_ref, m_ref, v_ref, g_ref = ada.optimize_rounding(kind, weight, alpha0, delta, offset, cmin, cmax, all_inp,
                                                       all_out, batches, *hyper, act=act, conv_args=conv_args)
    assert _close_except_few(a, a_ref, atol=5e-5) and (a - a_ref).abs().max() < 5e-3
    assert _close_except_few(g, g_ref, atol=1e-4 * g_ref.abs().max().item(), rtol=1e-3)


@pytest.mark.parametrize("shape", [(32, 8, 7, 7), (32, 64, 28, 28), (5, 10), (16, 7, 3), (32, 33)])
@pytest.mark.parametrize("activation", (0, 1))
def test_reconstruction_gradient_in_one_pass(ops, shape, activation):
    """dLoss/dout of the written-out gradient by one kernel: the five tensor operations it stands for, to the bit (the
    sign of zeros included), target rows gathered from the cache by sample number as torch's indexing gathers them."""
    torch.manual_seed(sum(shape) + activation)
    cached = 80
    out = torch.randn(shape).cuda()
    target_all = torch.randn(cached, *shape[1:]).cuda()
    index = torch.randperm(cached)[:shape[0]].cuda()
    index[0] = -1                                                       # counts from the end
    out.view(-1)[3] = float("nan")
    out.view(-1)[5] = 0.0
    target_all[index[1]].view(-1)[0] = float("nan")

    def by_tensor_operations(o, t):
        qa, ta = (torch.relu(o), torch.relu(t)) if activation else (o, t)
        g = (qa - ta) * (2.0 / (o.numel() // o.shape[1]))
        return g * (qa > 0) if activation else g

    def same(a, b):
        nan = torch.isnan(b)
        zero = torch.zeros_like(a)
        return torch.equal(torch.isnan(a), nan) and \
            torch.equal(torch.where(nan, zero, a).view(torch.int32), torch.where(nan, zero, b).view(torch.int32))

    got = ops.adaround_recon_grad(out, target_all, index, activation)
    assert got.shape == out.shape and same(got, by_tensor_operations(out, target_all[index]))
    got = ops.adaround_recon_grad(out, target_all, None, activation)    # the first rows of the cache
    assert same(got, by_tensor_operations(out, target_all[:shape[0]]))
    # a sample number the cache does not have: that row is NaN, the others are as before
    bad = index.clone()
    bad[2] = cached
    got = ops.adaround_recon_grad(out, target_all, bad, activation)
    assert torch.isnan(got[2]).all()
    keep = [i for i in range(shape[0]) if i != 2]
    assert same(got[keep], by_tensor_operations(out, target_all[index])[keep])
    with pytest.raises(ValueError):
        ops.adaround_recon_grad(out, target_all[:, :1], index, activation)
    with pytest.raises(ValueError):
        ops.adaround_recon_grad(out, target_all, index[:2], activation)


def test_fused_path_leaves_other_convolutions_alone(ops, monkeypatch):
    """A 3x3 kernel, a stride, a padding, groups, a row count that is not 32 / 64 / 128 / 256: the unfused path."""
    from aimet_amd.v1.adaround.adaround_optimizer import AdaroundOptimizer
    weight, delta, offset, C, npc, cmin, cmax = _case(65, (32, 128, 1, 1), 0, True)
    qm = type("Q", (), dict(num_channel=C, n_per_channel=npc))()
    batches = [torch.arange(32)]
    x = torch.randn(64, 128, 2, 2).cuda()
    y = torch.randn(64, 32, 2, 2).cuda()
    ok = torch.nn.Conv2d(128, 32, 1)
    assert AdaroundOptimizer._fused_rows(ok, weight.cuda(), qm, x, y, batches) is not None
    for conv in (torch.nn.Conv2d(128, 32, 1, stride=2), torch.nn.Conv2d(128, 32, 1, padding=1),
                 torch.nn.Conv2d(128, 32, 1, stride=(1, 2)), torch.nn.Conv2d(128, 32, 1, padding=(0, 1))):
        assert AdaroundOptimizer._fused_rows(conv, weight.cuda(), qm, x, y, batches) is None
    w3 = torch.randn(32, 128, 3, 3).cuda()
    assert AdaroundOptimizer._fused_rows(torch.nn.Conv2d(128, 32, 3), w3, qm, x, y, batches) is None
    x3 = torch.randn(64, 128, 1, 3).cuda()                 # 96 rows
    assert AdaroundOptimizer._fused_rows(ok, weight.cuda(), qm, x3, torch.randn(64, 32, 1, 3).cuda(), batches) is None
    assert AdaroundOptimizer._fused_rows(ok, weight.cuda(), qm, x, y, [torch.arange(16)]) is not None     # 64 rows
    assert AdaroundOptimizer._fused_rows(ok, weight.cuda(), qm, x, y, [torch.arange(24)]) is None
    assert AdaroundOptimizer._fused_rows(torch.nn.ConvTranspose2d(128, 32, 1), weight.cuda(), qm, x, y, batches) is None


def test_cfg5_fused_linear_at_configured_size(ops):
    """The AdaRound configuration at its size: Linear [4096,4096], weights N(0, 0.02), 2048 cached rows N(0,1),
    4-bit per-output-channel symmetric min/max encodings, seed 1005.  24 iterations of the 1000-iteration schedule
    that straddle the end of the warm start (190 .. 213, so both the reconstruction-only and the regularised
    iterations run), from an alpha moved off its initial value: at alpha0 with a target the layer reproduces exactly
    the gradient is the summation-order noise of the GEMM, which Adam turns into full-size random steps on either side.
    Compared with the CPU restatement: alpha, both moments, the last gradient, the per-iteration reconstruction and
    rounding losses and the hard-rounding decisions; int8 and float32 storage of floor(W / delta) must agree bit
    for bit through the 16 K-tiles per output block this shape has."""
    O = K = 4096
    rows, iters, first = 2048, 24, 190
    hyper = (1000, 0.01, (20, 2), 0.2)
    g = torch.Generator().manual_seed(1005)
    weight = torch.randn(O, K, generator=g) * 0.02
    X = torch.randn(rows, K, generator=g)
    Y = torch.nn.functional.linear(X, weight)
    absmax = weight.abs().amax(dim=1)
    delta = (absmax / 7.0).float()                       # symmetric 4-bit: max(|min|, |max|) / floor(15 / 2)
    offset = torch.full((O,), -8.0)
    cmin, cmax = 0.0, 15.0
    d = ada.broadcast(delta, weight, 0)
    alpha0 = ada.generate_alpha(weight, d) + 0.7 * torch.randn(O, K, generator=g)
    batches = [torch.randperm(rows, generator=g)[:32] for _ in range(iters)]
    trace = []
    a_ref, m_ref, v_ref, g_ref = ada.optimize_rounding("linear", weight, alpha0, delta, offset, cmin, cmax, X, Y,
                                                       batches, *hyper, first_iteration=first, trace=trace)

    wg, dg, og, Xg, Yg = (t.cuda() for t in (weight, delta, offset, X, Y))
    index = torch.stack(batches).to(torch.int32).cuda()
    ws = ops.adaround_linear_workspace(O, K, "cuda")
    f32 = ops.adaround_floor(wg, O, K, dg)
    f8 = ops.adaround_floor_i8(wg, O, K, dg, og, cmin, cmax)
    assert f8 is not None and f8.dtype == torch.int8
    results = {}
    for name, fl in (("int8", f8), ("float32", f32)):
        alpha, m, v = alpha0.cuda(), torch.zeros(O, K, device="cuda"), torch.zeros(O, K, device="cuda")
        grad = torch.empty_like(alpha)
        gout = torch.empty(32, O, device="cuda")
        recon = torch.zeros(iters, (32 * O + 255) // 256, device="cuda")
        reg = torch.zeros(iters, ops.adaround_linear_blocks(O, K), device="cuda")
        for k in range(iters):
            it = first + k
            beta = -1.0 if it < hyper[3] * hyper[0] else ada.compute_beta(hyper[0], it, hyper[2], hyper[3])
            ops.adaround_linear_fwd(fl, alpha, Xg, index[k], Yg, None, O, dg, og, cmin, cmax, 0, ws, gout,
                                    loss_partial=recon[k])
            ops.adaround_linear_bwd_adam(fl, gout, Xg, index[k], alpha, m, v, O, dg, og, cmin, cmax, hyper[1], beta,
                                         1e-3, 0.9, 0.999, 1e-8, k + 1, reg_partial=reg[k], grad_alpha=grad)
        results[name] = (alpha, m, v, grad, recon.double().sum(dim=1).cpu(), reg.double().sum(dim=1).cpu())
    for a, b in zip(results["int8"], results["float32"]):
        assert torch.equal(a, b)                          # identical trajectory from either storage
    a, m, v, gr, recon, reg = results["int8"]
    a, m, v, gr = a.cpu(), m.cpu(), v.cpu(), gr.cpu()
    assert (a_ref - alpha0).abs().max() > 5e-3
    for k, (rc, rn) in enumerate(trace):
        assert recon[k].item() == pytest.approx(rc, rel=2e-4), k
        if first + k < 200:
            assert rn == 0 and reg[k].item() == 0
        else:
            # the kernel returns sum(1 - |2h - 1|^beta); the loss term is reg_param times that
            assert hyper[1] * reg[k].item() == pytest.approx(rn, rel=1e-4), k
    assert _close_except_few(a, a_ref, atol=5e-5)
    assert (a - a_ref).abs().max() < 5e-3
    assert _close_except_few(gr, g_ref, atol=1e-4 * g_ref.abs().max().item(), rtol=1e-3)
    assert _close_except_few(m, m_ref, atol=1e-4 * m_ref.abs().max().item(), rtol=1e-3)
    assert _close_except_few(v, v_ref, atol=1e-4 * v_ref.abs().max().item(), rtol=1e-3)
    same = ((a >= 0) == (a_ref >= 0)).double().mean().item()
    print(f"cfg5: identical hard-rounding decisions {same:.7f}")
    assert same > 0.9999
    # hard-rounded weights from the optimised alpha: identical wherever the decision is
    hard = ops.adaround_soft_round(wg, a.cuda(), O, K, dg, og, cmin, cmax, False).cpu()
    hard_ref = ada.apply_adaround(weight, a_ref, d, ada.broadcast(offset, weight, 0), cmin, cmax, False)
    assert ((hard == hard_ref).double().mean().item()) >= same - 1e-12


@pytest.mark.parametrize("target_noise", [0.02, 0.0])
def test_cfg5_whole_schedule(ops, target_noise, monkeypatch):
    """All 1000 iterations of the AdaRound configuration (Linear [4096,4096], 2048 cached rows, 4-bit per-channel
    symmetric min/max encodings, seed 1005, warm start 0.2, beta 20 -> 2) through the fused kernels, from the initial
    alpha, against the restatement's torch ops, autograd and torch.optim.Adam on the same GPU and the same batches:
    loss curves and the fraction of identical hard-rounding decisions at the end.

    target_noise = 0.02: the target is the layer's output plus noise, so every iteration has a gradient that means
    something: curves agree to 1e-5 and the decisions to 0.9999.
    target_noise = 0: the configuration as written, the target is exactly what alpha's initial value reproduces (the
    symmetric grid clips no weight), so for the 200 warm-start iterations the reconstruction gradient is the summation
    noise of the GEMMs, which Adam normalises into full-size steps of random sign.  Any two summation orders then walk
    apart: the yardstick is the restatement against itself with the layer's GEMM accumulated in float64 (the same sums,
    rounded once instead of at every step)."""
    O = K = 4096
    rows, iters = 2048, 1000
    hyper = (iters, 0.01, (20, 2), 0.2)
    g = torch.Generator().manual_seed(1005)
    weight = torch.randn(O, K, generator=g) * 0.02
    X = torch.randn(rows, K, generator=g)
    Y = torch.nn.functional.linear(X, weight)
    if target_noise:
        Y = Y + target_noise * torch.randn(rows, O, generator=g)
    delta, offset = (weight.abs().amax(dim=1) / 7.0).float(), torch.full((O,), -8.0)
    cmin, cmax = 0.0, 15.0
    alpha0 = ada.generate_alpha(weight, ada.broadcast(delta, weight, 0))
    batches = [torch.randperm(rows, generator=g)[:32] for _ in range(iters)]
    wg, dg, og, Xg, Yg, a0g = (t.cuda() for t in (weight, delta, offset, X, Y, alpha0))

    def restatement(batch_list):
        trace = []
        a, _, _, _ = ada.optimize_rounding("linear", wg, a0g, dg, og, cmin, cmax, Xg, Yg, batch_list, *hyper,
                                           trace=trace)
        return a, np.array(trace)

    a_ref, curve_ref = restatement([b.cuda() for b in batches])
    index = torch.stack(batches).to(torch.int32).cuda()
    ws = ops.adaround_linear_workspace(O, K, "cuda")
    f8 = ops.adaround_floor_i8(wg, O, K, dg, og, cmin, cmax)
    alpha, m, v = a0g.clone(), torch.zeros(O, K, device="cuda"), torch.zeros(O, K, device="cuda")
    gout = torch.empty(32, O, device="cuda")
    recon = torch.zeros(iters, (32 * O + 255) // 256, device="cuda")
    reg = torch.zeros(iters, ops.adaround_linear_blocks(O, K), device="cuda")
    for k in range(iters):
        beta = -1.0 if k < hyper[3] * iters else ada.compute_beta(iters, k, hyper[2], hyper[3])
        ops.adaround_linear_fwd(f8, alpha, Xg, index[k], Yg, None, O, dg, og, cmin, cmax, 0, ws, gout,
                                loss_partial=recon[k])
        ops.adaround_linear_bwd_adam(f8, gout, Xg, index[k], alpha, m, v, O, dg, og, cmin, cmax, hyper[1], beta, 1e-3,
                                     0.9, 0.999, 1e-8, k + 1, reg_partial=reg[k])
    curve = np.stack([recon.double().sum(dim=1).cpu().numpy(), hyper[1] * reg.double().sum(dim=1).cpu().numpy()], 1)
    same = ((alpha >= 0) == (a_ref >= 0)).double().mean().item()
    late = slice(200, iters)
    dev_recon = (np.abs(curve[late, 0] - curve_ref[late, 0]) / curve_ref[late, 0]).max()
    dev_round = (np.abs(curve[late, 1] - curve_ref[late, 1]) / curve_ref[late, 1]).max()
    print(f"cfg5 x 1000, target noise {target_noise}: identical hard-rounding decisions {same:.8f}; largest relative "
          f"deviation of the loss curves after the warm start: reconstruction {dev_recon:.3g}, rounding {dev_round:.3g}; "
          f"final losses {curve[-1, 0]:.6g} / {curve[-1, 1]:.6g} against {curve_ref[-1, 0]:.6g} / {curve_ref[-1, 1]:.6g}")
    assert (a_ref - a0g).abs().mean() > 0.5              # the schedule did its work
    assert curve[:200, 1].max() == 0 and curve_ref[:200, 1].max() == 0
    if target_noise:
        assert same >= 0.9999
        assert dev_recon < 1e-5 and dev_round < 1e-5
        assert np.abs(curve[:200, 0] - curve_ref[:200, 0]).max() < 1e-5 * curve_ref[:200, 0].max()
    else:
        monkeypatch.setattr(ada, "layer_output",
                            lambda kind, inp, w, bias=None: (inp.double() @ w.double().t()).float())
        a_f64, curve_f64 = restatement([b.cuda() for b in batches])
        yardstick = ((a_f64 >= 0) == (a_ref >= 0)).double().mean().item()
        dev_f64 = (np.abs(curve_f64[late, 0] - curve_ref[late, 0]) / curve_ref[late, 0]).max()
        dev_round_f64 = (np.abs(curve_f64[late, 1] - curve_ref[late, 1]) / curve_ref[late, 1]).max()
        print(f"   the restatement against itself with the GEMM accumulated in float64: {yardstick:.8f}, curves "
              f"{dev_f64:.3g} / {dev_round_f64:.3g}")
        assert same > 0.999 and same >= yardstick - 3e-4
        assert dev_recon < max(2 * dev_f64, 5e-3) and dev_round < max(2 * dev_round_f64, 1e-4)


class _TinyNet(torch.nn.Module):
    def __init__(self):
        super().__init__()
        self.conv1 = torch.nn.Conv2d(3, 8, 3, padding=1)
        self.relu1 = torch.nn.ReLU(inplace=True)
        self.pool = torch.nn.AdaptiveAvgPool2d(4)
        self.flatten = torch.nn.Flatten()
        self.fc = torch.nn.Linear(8 * 16, 10)

    def forward(self, x):
        return self.fc(self.flatten(self.pool(self.relu1(self.conv1(x)))))


def _loader(n_batches, batch, seed):
    g = torch.Generator().manual_seed(seed)
    return [(torch.randn(batch, 3, 8, 8, generator=g).cuda(), torch.zeros(batch)) for _ in range(n_batches)]


def _forward_fn(model, inputs):
    x, _ = inputs
    return model(x)


def test_reference_style_layer_optimisation(tmp_path):
    """Shaped after TestAdaroundOptimizer._optimize_layer_rounding (test_adaround_optimizer.py:65-109): alpha changes,
    alpha.grad is populated, and afterwards the layer uses hard rounding."""
    from aimet_amd.v1.adaround.adaround_loss import AdaroundHyperParameters
    from aimet_amd.v1.adaround.adaround_optimizer import AdaroundOptimizer
    from aimet_amd.v1.adaround.adaround_weight import Adaround
    from aimet_amd.v1.quantsim import QuantizationSimModel
    from aimet_amd import utils
    for warm_start in (1.0, 0.2):
        torch.manual_seed(0)
        model = _TinyNet().eval().cuda()
        dummy = torch.randn(1, 3, 8, 8).cuda()
        sim = QuantizationSimModel(model, dummy_input=dummy, quant_scheme='tf_enhanced', default_param_bw=4)
        Adaround._compute_param_encodings(sim)
        with Adaround._replace_quantization_layer(sim.model, "conv1") as wrapper:
            wrapper.alpha = torch.nn.Parameter(torch.randn(wrapper.weight.shape).cuda())
            before = wrapper.alpha.detach().clone()
            cached = utils.CachedDataset(_loader(5, 10, 1), 5)
            opt = AdaroundHyperParameters(num_iterations=10, reg_param=0.01, beta_range=(20, 2),
                                          warm_start=warm_start)
            AdaroundOptimizer.adaround_module(model.conv1, wrapper, model, sim.model, None, cached, _forward_fn, opt)
            assert not torch.equal(before, wrapper.alpha.detach())
            assert wrapper.alpha.grad is not None
            assert wrapper.use_soft_rounding is False


def test_recons_metrics_known_answer(vectors, ops):
    """test_adaround_optimizer.py:122-196 on the GPU: TF-Enhanced encoding of a seeded weight, hard / soft
    reconstruction errors and the reconstruction loss."""
    from aimet_amd.v1.adaround.adaround_loss import AdaroundLoss
    from aimet_amd.v1.adaround.adaround_optimizer import AdaroundOptimizer
    from aimet_amd.v1.adaround.adaround_wrapper import AdaroundWrapper
    from aimet_amd.v1.qc_quantize_op import StaticGridQuantWrapper
    from aimet_amd.common.defs import QuantScheme
    g = vectors["adaround"]["recons_metrics"]
    np.random.seed(g["np_seed"])
    weight = np.random.rand(*g["weight_shape"]).astype('float32')
    conv = torch.nn.Conv2d(4, 4, 1, bias=False).cuda()
    conv.weight.data = torch.from_numpy(weight).cuda()
    qw = StaticGridQuantWrapper(conv, g["weight_bw"], 8, round_mode='nearest',
                                quant_scheme=QuantScheme.post_training_tf_enhanced)
    qw.param_quantizers['weight'].update_encoding_stats(conv.weight.data)
    qw.param_quantizers['weight'].compute_encoding()
    assert qw.param_quantizers['weight'].encoding.delta == pytest.approx(g["scale"], abs=10 ** -g["scale_places"])
    inp = torch.from_numpy(np.random.rand(*g["inp_shape"]).astype('float32')).cuda()
    out = torch.from_numpy(np.random.rand(*g["out_shape"]).astype('float32')).cuda()
    wrapper = AdaroundWrapper(qw)
    hard, soft = AdaroundOptimizer._compute_recons_metrics(wrapper, None, inp, out)
    assert hard == pytest.approx(g["recons_err_hard"], abs=10 ** -g["places"])
    assert soft == pytest.approx(g["recons_err_soft"], abs=10 ** -g["places"])
    y = AdaroundOptimizer._compute_output_with_adarounded_weights(wrapper, inp)
    assert AdaroundLoss.compute_recon_loss(y, out).item() == pytest.approx(g["recon_loss_soft"],
                                                                           abs=10 ** -g["cuda_places"])


def test_apply_adaround_end_to_end(tmp_path, oracle):
    """Adaround.apply_adaround on a small conv + linear model against the same flow replayed with the CPU restatement:
    same encodings file, same seeded batches, adarounded weights equal on the quantization grid."""
    from aimet_amd.v1.adaround.adaround_weight import Adaround, AdaroundParameters
    torch.manual_seed(0)
    model = _TinyNet().eval().cuda()
    dummy = torch.randn(1, 3, 8, 8).cuda()
    loader = _loader(4, 16, 5)
    iters = 30
    params = AdaroundParameters(loader, num_batches=4, default_num_iterations=iters, forward_fn=_forward_fn)
    torch.manual_seed(1234)
    ada_model = Adaround.apply_adaround(model, dummy, params, str(tmp_path), "tiny", default_param_bw=4)
    with open(os.path.join(str(tmp_path), "tiny.encodings")) as f:
        enc = json.load(f)["param_encodings"]
    assert set(enc) == {"conv1.weight", "fc.weight"}

    # replay on the CPU
    cpu = _TinyNet().eval()
    cpu.load_state_dict({k: v.cpu() for k, v in model.state_dict().items()})
    quant = _TinyNet().eval()
    quant.load_state_dict(cpu.state_dict())
    torch.manual_seed(1234)                     # the product drew its batches from the host generator seeded so
    xs = torch.cat([b[0].cpu() for b in loader])
    for name, kind, act, conv_args in (("conv1", "conv2d", torch.relu, {"padding": 1}), ("fc", "linear", None, {})):
        e = enc[name + ".weight"][0]
        assert e["bitwidth"] == 4
        delta = torch.tensor([e["scale"]], dtype=torch.float32)
        offset = torch.tensor([float(e["offset"])], dtype=torch.float32)
        layer_fp, layer_q = getattr(cpu, name), getattr(quant, name)
        with torch.no_grad():
            if name == "conv1":
                inp, out = xs, layer_fp(xs)
            else:
                inp = quant.flatten(quant.pool(torch.relu(quant.conv1(xs))))
                out = layer_fp(cpu.flatten(cpu.pool(torch.relu(cpu.conv1(xs)))))
        weight = layer_fp.weight.detach()
        alpha0 = ada.generate_alpha(weight, delta.reshape(()))
        batches = [torch.randperm(inp.size(0))[:32] for _ in range(iters)]
        alpha, _, _, _ = ada.optimize_rounding(kind, weight, alpha0, delta, offset, 0, 15, inp, out, batches, iters,
                                               0.01, (20, 2), 0.2, bias=layer_fp.bias.detach(), act=act,
                                               conv_args=conv_args)
        w_ref = ada.apply_adaround(weight, alpha, delta.reshape(()), offset.reshape(()), 0, 15, True)
        got = getattr(ada_model, name).weight.detach().cpu()
        assert torch.allclose(got, w_ref, atol=float(delta) * 2e-3, rtol=0), name
        # later layers see this layer through its weight quantizer (same encoding, round to nearest)
        w_seen = oracle.qdq_per_tensor(w_ref.numpy().reshape(-1), e["min"], e["max"], 4).reshape(w_ref.shape)
        with torch.no_grad():
            layer_q.weight.copy_(torch.from_numpy(w_seen))
    assert not any(isinstance(m, torch.nn.Module) and type(m).__name__.endswith("Wrapper")
                   for m in ada_model.modules())


def test_v2_quantized_modules_and_sim():
    """v2 quantized modules: parameters and activations are quantize-dequantized around the base forward."""
    from aimet_amd.v2.nn import QuantizationMixin, QuantizedLinear
    from aimet_amd.v2.quantization.affine import QuantizeDequantize
    from aimet_amd.v2.quantsim import QuantizationSimModel
    torch.manual_seed(0)
    lin = torch.nn.Linear(16, 8).cuda()
    q = QuantizationMixin.from_module(lin)
    assert isinstance(q, QuantizedLinear) and isinstance(q, torch.nn.Linear) and q.weight is lin.weight
    x = torch.randn(4, 16).cuda()
    assert torch.equal(q(x), lin(x))                         # no quantizers yet
    q.param_quantizers['weight'] = QuantizeDequantize((), bitwidth=4, symmetric=True).cuda()
    q.output_quantizers[0] = QuantizeDequantize((), bitwidth=8, symmetric=False).cuda()
    with q.compute_encodings():
        q(x)
    wq = q.param_quantizers['weight']
    assert wq.is_initialized() and q.output_quantizers[0].is_initialized()
    want = q.output_quantizers[0](torch.nn.functional.linear(x, wq(lin.weight), lin.bias))
    assert torch.equal(q(x), want)
    assert q.weight is lin.weight                            # the patch is gone after the call
    with pytest.raises(RuntimeError):
        QuantizationMixin.from_module(torch.nn.Bilinear(2, 2, 2))
    model = _TinyNet().eval().cuda()
    sim = QuantizationSimModel(model, torch.randn(1, 3, 8, 8).cuda(), quant_scheme='tf', default_param_bw=8)
    names = [n for n, _ in sim.named_qmodules()]
    assert names == ["conv1", "relu1", "pool", "flatten", "fc"]
    sim.compute_encodings(lambda m, a: m(a), torch.randn(8, 3, 8, 8).cuda())
    y = sim.model(torch.randn(2, 3, 8, 8).cuda())
    assert y.shape == (2, 10) and torch.isfinite(y).all()


def test_v2_apply_adaround_end_to_end(tmp_path, oracle):
    """aimet_amd.v2.adaround.Adaround.apply_adaround (signed grid of the symmetric v2 weight quantizers) against the
    same flow replayed with the CPU restatement."""
    from aimet_amd.v2.adaround import Adaround, AdaroundParameters, AdaroundWrapper
    from aimet_amd.v2.nn import BaseQuantizationMixin
    from aimet_amd.common.defs import QuantScheme
    torch.manual_seed(0)
    model = _TinyNet().eval().cuda()
    dummy = torch.randn(1, 3, 8, 8).cuda()
    loader = _loader(4, 16, 7)
    iters = 30
    params = AdaroundParameters(loader, num_batches=4, default_num_iterations=iters, forward_fn=_forward_fn)
    torch.manual_seed(4321)
    ada_model = Adaround.apply_adaround(model, dummy, params, str(tmp_path), "tiny2", default_param_bw=4,
                                        default_quant_scheme=QuantScheme.post_training_tf)
    assert not any(isinstance(m, (BaseQuantizationMixin, AdaroundWrapper)) for m in ada_model.modules())
    with open(os.path.join(str(tmp_path), "tiny2.encodings")) as f:
        enc = json.load(f)["param_encodings"]
    assert set(enc) == {"conv1.weight", "fc.weight"}
    cpu = _TinyNet().eval()
    cpu.load_state_dict({k: v.cpu() for k, v in model.state_dict().items()})
    quant = _TinyNet().eval()
    quant.load_state_dict(cpu.state_dict())
    torch.manual_seed(4321)
    xs = torch.cat([b[0].cpu() for b in loader])
    for name, kind, act, conv_args in (("conv1", "conv2d", torch.relu, {"padding": 1}), ("fc", "linear", None, {})):
        e = enc[name + ".weight"][0]
        assert e["bitwidth"] == 4 and e["is_symmetric"] == "True" and e["offset"] == 0
        delta = torch.tensor([e["scale"]], dtype=torch.float32)
        offset = torch.tensor([0.0])
        layer_fp, layer_q = getattr(cpu, name), getattr(quant, name)
        with torch.no_grad():
            if name == "conv1":
                inp, out = xs, layer_fp(xs)
            else:
                inp = quant.flatten(quant.pool(torch.relu(quant.conv1(xs))))
                out = layer_fp(cpu.flatten(cpu.pool(torch.relu(cpu.conv1(xs)))))
        weight = layer_fp.weight.detach()
        alpha0 = ada.generate_alpha(weight, delta.reshape(()))
        batches = [torch.randperm(inp.size(0))[:32] for _ in range(iters)]
        alpha, _, _, _ = ada.optimize_rounding(kind, weight, alpha0, delta, offset, -8, 7, inp, out, batches, iters,
                                               0.01, (20, 2), 0.2, bias=layer_fp.bias.detach(), act=act,
                                               conv_args=conv_args)
        w_ref = ada.apply_adaround(weight, alpha, delta.reshape(()), offset.reshape(()), -8, 7, True)
        got = getattr(ada_model, name).weight.detach().cpu()
        assert torch.allclose(got, w_ref, atol=float(delta) * 2e-3, rtol=0), name
        w_seen, _, _ = oracle.v2_qdq(w_ref.numpy().reshape(-1), 1, w_ref.numel(), delta.numpy(), offset.numpy(), -8, 7)
        with torch.no_grad():
            layer_q.weight.copy_(torch.from_numpy(w_seen.reshape(w_ref.shape)))
