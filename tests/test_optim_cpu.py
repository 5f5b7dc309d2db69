"""RangerLite: the CPU restatement of the fused update (oracle) against closed forms and against the
torch-op path; the optimizer class on CPU tensors against torch.optim.Adam where the two coincide."""
import math

import numpy as np
import pytest
import torch

from nnueft.optim import RangerLite

F = np.float32


def _arrays(n, seed):
    rng = np.random.default_rng(seed)
    return (rng.standard_normal(n).astype(F), rng.standard_normal(n).astype(F) * F(0.1))


def test_first_step_closed_forms(oracle_cpu):
    # zero state, step 1: vm / bias_correction2 = g*g exactly when computed in this order, so the
    # denominator is |g| + eps and the step has a closed form
    p0, g = _arrays(257, 1)
    beta1, beta2, lr, eps = 0.9, 0.999, 1e-2, 1e-7
    # Adam flavour
    p = p0.copy(); gm = np.zeros_like(p); vm = np.zeros_like(p)
    oracle_cpu.ranger_lite_update(p, g, gm, None, vm, None, beta2=beta2, bias_correction2=1 - beta2, beta1=beta1,
                                  one_minus_beta1=1 - beta1, lr_div_bc1=lr / (1 - beta1), eps=eps, step=1)
    assert np.allclose(vm, (g * g) * F(1 - beta2), rtol=1e-6)
    assert np.allclose(gm, g * F(1 - beta1), rtol=1e-6)
    expect = p0 - lr * g / (np.abs(g) + eps)
    assert np.allclose(p, expect, rtol=0, atol=2e-7)
    # positive-negative pair, step 1 (odd: grad_ma is the positive buffer, the negative one is still zero);
    # bias correction uses 2 effective steps: lr / (1 - beta1^2) * g (1 - beta1^2) (1 + pnm) / noise / (|g| + eps)
    pnm = 1.0
    noise = math.sqrt((1 + pnm) ** 2 + pnm ** 2)
    p = p0.copy(); gm = np.zeros_like(p); ngm = np.zeros_like(p); vm = np.zeros_like(p)
    oracle_cpu.ranger_lite_update(p, g, gm, ngm, vm, None, beta2=beta2, bias_correction2=1 - beta2, beta1=beta1 ** 2,
                                  one_minus_beta1=1 - beta1 ** 2, one_plus_pnm=1 + pnm, pnm_factor=pnm,
                                  noise_norm=noise, lr_div_bc1=lr / (1 - beta1 ** 2), eps=eps, step=1)
    assert not ngm.any() and np.allclose(gm, g * F(1 - beta1 ** 2), rtol=1e-6)
    expect = p0 - lr * (2 / math.sqrt(5)) * g / (np.abs(g) + eps)
    assert np.allclose(p, expect, rtol=0, atol=2e-7)
    # step 2 (even): the other buffer takes the new gradient, the first one enters with -pnm_factor
    g2 = _arrays(257, 2)[0]
    gm_before = gm.copy()
    oracle_cpu.ranger_lite_update(p, g2, gm, ngm, vm, None, beta2=beta2, bias_correction2=1 - beta2 ** 2,
                                  beta1=beta1 ** 2, one_minus_beta1=1 - beta1 ** 2, one_plus_pnm=1 + pnm,
                                  pnm_factor=pnm, noise_norm=noise, lr_div_bc1=lr / (1 - beta1 ** 2), eps=eps, step=2)
    assert np.array_equal(gm, gm_before) and np.allclose(ngm, g2 * F(1 - beta1 ** 2), rtol=1e-6)


def test_decay_phase2_and_lookahead_closed_forms(oracle_cpu):
    p0, g = _arrays(64, 3)
    # zero gradient and zero moments: the step is decay only, then the blend with the slow weights
    zero = np.zeros_like(p0)
    vm = np.full_like(p0, 0.25)
    slow = np.ones_like(p0)
    p = p0.copy(); gm = zero.copy()
    oracle_cpu.ranger_lite_update(p, zero, gm, None, vm, slow, beta2=0.999, bias_correction2=0.5, beta1=0.9,
                                  one_minus_beta1=0.1, lr_div_bc1=1.0, eps=1e-7, wd_factor=0.25,
                                  update_variance=False, alpha=0.5)
    assert np.array_equal(vm, np.full_like(p0, 0.25))            # phase 2 leaves the variance alone
    assert np.array_equal(p, (p0 * F(0.75)) * F(0.5) + F(0.5))   # every factor a power of two: exact
    assert np.array_equal(slow, p)
    # variance kernel alone
    vm = np.full_like(p0, 2.0)
    oracle_cpu.ranger_lite_update_variance(g, vm, 0.5)
    assert np.array_equal(vm, F(1.0) + (g * g) * F(0.5))


@pytest.mark.parametrize("pnm", [True, False])
def test_oracle_follows_the_torch_op_path_over_several_steps(oracle_cpu, pnm):
    # the same quantities computed with the torch ops of the reference's Python path
    # (ranger_lite.py:689-735); grouping differs (sqrt(v)/sqrt(bc) against sqrt(v/bc)), so to rounding
    n, beta1, beta2, lr, eps, pf = 1000, 0.9, 0.999, 3e-3, 1e-7, 1.0
    p0, _ = _arrays(n, 4)
    p = p0.copy(); gm = np.zeros_like(p); ngm = np.zeros_like(p); vm = np.zeros_like(p)
    tp = torch.from_numpy(p0.copy()); tgm = torch.zeros(n); tngm = torch.zeros(n); tvm = torch.zeros(n)
    noise = math.sqrt((1 + pf) ** 2 + pf ** 2)
    for step in range(1, 8):
        g = _arrays(n, 10 + step)[0]
        tg = torch.from_numpy(g)
        tvm.mul_(beta2).addcmul_(tg, tg, value=1 - beta2)
        denom = (tvm.sqrt() / math.sqrt(1 - beta2 ** step)).add_(eps)
        if pnm:
            pos, neg = (tgm, tngm) if step % 2 == 1 else (tngm, tgm)
            pos.mul_(beta1 ** 2).add_(tg, alpha=1 - beta1 ** 2)
            bc1 = 1 - beta1 ** (((step + 1) // 2) * 2)
            tp.addcdiv_(pos.mul(1 + pf).add(neg, alpha=-pf).mul(1 / noise), denom, value=-lr / bc1)
            oracle_cpu.ranger_lite_update(p, g, gm, ngm, vm, None, beta2=beta2, bias_correction2=1 - beta2 ** step,
                                          beta1=beta1 ** 2, one_minus_beta1=1 - beta1 ** 2, one_plus_pnm=1 + pf,
                                          pnm_factor=pf, noise_norm=noise, lr_div_bc1=lr / bc1, eps=eps, step=step)
        else:
            tgm.mul_(beta1).add_(tg, alpha=1 - beta1)
            bc1 = 1 - beta1 ** step
            tp.addcdiv_(tgm, denom, value=-lr / bc1)
            oracle_cpu.ranger_lite_update(p, g, gm, None, vm, None, beta2=beta2, bias_correction2=1 - beta2 ** step,
                                          beta1=beta1, one_minus_beta1=1 - beta1, lr_div_bc1=lr / bc1, eps=eps, step=step)
    assert np.allclose(p, tp.numpy(), rtol=1e-5, atol=1e-6)
    assert np.allclose(vm, tvm.numpy(), rtol=1e-5) and np.allclose(gm, tgm.numpy(), rtol=1e-5, atol=1e-7)


def _params(seed, shapes=((7, 5), (11,), (3, 4, 2))):
    g = torch.Generator().manual_seed(seed)
    return [torch.nn.Parameter(torch.randn(*s, generator=g)) for s in shapes]


def _grads(params, seed):
    g = torch.Generator().manual_seed(seed)
    for p in params:
        p.grad = torch.randn(p.shape, generator=g)


def test_class_equals_torch_adam_when_reduced_to_it():
    a, b = _params(1), _params(1)
    ours = RangerLite(a, lr=1e-2, betas=(0.9, 0.999), eps=1e-8, pnm_activate=False, lookahead_active=False,
                      normloss_active=False)
    ref = torch.optim.Adam(b, lr=1e-2, betas=(0.9, 0.999), eps=1e-8)
    for s in range(6):
        _grads(a, 20 + s)
        _grads(b, 20 + s)
        ours.step()
        ref.step()
    for x, y in zip(a, b):
        torch.testing.assert_close(x, y, rtol=1e-5, atol=1e-6)


def test_class_lookahead_merge_and_eval_swap():
    a, b = _params(2), _params(2)
    start = [p.detach().clone() for p in a]
    with_la = RangerLite(a, lr=1e-2, normloss_active=False, lookahead_mergetime=5, lookahead_blending_alpha=0.5)
    without = RangerLite(b, lr=1e-2, normloss_active=False, lookahead_active=False)
    for s in range(5):
        _grads(a, 30 + s)
        _grads(b, 30 + s)
        with_la.step()
        without.step()
        if s < 4:
            for x, y in zip(a, b):
                assert torch.equal(x, y)
    # the fifth step merged: fast * alpha + slow * (1 - alpha), slow = the start weights
    for x, y, s0 in zip(a, b, start):
        torch.testing.assert_close(x, y * 0.5 + s0 * 0.5, rtol=1e-6, atol=1e-7)
        assert torch.equal(with_la.state[x]["lookahead_params"], x)
    _grads(a, 40)
    with_la.step()
    fast = [p.detach().clone() for p in a]
    slow = [with_la.state[p]["lookahead_params"].clone() for p in a]
    with_la.eval()
    with_la.eval()                                   # idempotent
    for p, s in zip(a, slow):
        assert torch.equal(p, s)
    with_la.train()
    with_la.train()
    for p, f in zip(a, fast):
        assert torch.equal(p, f)


def test_class_weight_decay_and_param_groups():
    a = _params(3)
    opt = RangerLite([{"params": a[:1], "lr": 1e-2, "weight_decay": 0.1}, {"params": a[1:], "lr": 5e-3}],
                     normloss_active=False, lookahead_active=False)
    before = [p.detach().clone() for p in a]
    _grads(a, 50)
    opt.step()
    assert opt.param_size == sum(p.numel() for p in a)
    # step 1: the debiased variance is g*g, its mean over all parameters the norm; decay shrinks group 0 only
    norm = math.sqrt(sum(float((p.grad * p.grad).sum()) for p in a) / opt.param_size)
    upd = lambda p, lr: lr * (2 / math.sqrt(5)) * p.grad / (p.grad.abs() + 1e-7)
    torch.testing.assert_close(a[0], before[0] * (1 - 0.1 * 1e-2 / norm) - upd(a[0], 1e-2), rtol=1e-5, atol=1e-6)
    torch.testing.assert_close(a[1], before[1] - upd(a[1], 5e-3), rtol=1e-5, atol=1e-6)
    sd = opt.state_dict()
    assert set(sd["state"][0]) == {"step", "grad_ma", "variance_ma", "neg_grad_ma"}
