"""RangerLite update kernels (through the C ABI) against the CPU oracle: bit-exact; the optimizer
class on the GPU against its torch-op path on the CPU."""
import math

import numpy as np
import pytest
import torch

from nnueft.optim import RangerLite

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")
F = np.float32


def _native():
    from nnueft import _native

    return _native, _native.load()


def _stream():
    return torch.cuda.current_stream().cuda_stream


def _state(n, seed, offset=0):
    """p, grad, grad_ma, neg_grad_ma, variance_ma, slow as numpy; `offset` floats of slack in front so the
    device copies can start at an address that is not 16-byte aligned."""
    rng = np.random.default_rng(seed)
    mk = lambda s: (rng.standard_normal(n + offset) * s).astype(F)
    return [mk(1.0), mk(0.3), mk(0.1), mk(0.1), np.abs(mk(0.05)), mk(1.0)]


@pytest.mark.parametrize("n,offset", [(1, 0), (3, 0), (5, 1), (1027, 0), (4096, 0), (70001, 3), (1 << 20, 0)])
@pytest.mark.parametrize("flavour", ["pnm_odd", "pnm_even", "adam"])
@pytest.mark.parametrize("phase2,merge", [(False, False), (True, False), (False, True), (True, True)])
def test_update_kernels_bit_exact(oracle_cpu, n, offset, flavour, phase2, merge):
    nat, lib = _native()
    host = _state(n, 7 * n + offset, offset)
    dev = [torch.from_numpy(a).to(DEV)[offset:] for a in host]
    host = [a[offset:].copy() for a in host]
    p, g, gm, ngm, vm, slow = host
    dp, dg, dgm, dngm, dvm, dslow = dev
    beta1, beta2, lr, eps, pf = 0.9, 0.999, 8.75e-4, 1e-7, 1.0
    step = {"pnm_odd": 7, "pnm_even": 8, "adam": 5}[flavour]
    bc2 = 1 - beta2 ** step
    wd = 0.0125 if phase2 else 0.0
    if flavour == "adam":
        bc1 = 1 - beta1 ** step
        oracle_cpu.ranger_lite_update(p, g, gm, None, vm, slow if merge else None, beta2=beta2, bias_correction2=bc2,
                                      beta1=beta1, one_minus_beta1=1 - beta1, lr_div_bc1=lr / bc1, eps=eps, step=step,
                                      wd_factor=wd, update_variance=not phase2, alpha=0.5)
        nat.check(lib.nnueft_ranger_lite_update_adam(dp.data_ptr(), dg.data_ptr(), dgm.data_ptr(), dvm.data_ptr(), n,
                                                     beta2, 1 - beta2, bc2, beta1, 1 - beta1, lr / bc1, eps, wd,
                                                     0 if phase2 else 1, dslow.data_ptr() if merge else None, 0.5,
                                                     _stream()), "adam")
    else:
        bc1 = 1 - beta1 ** (((step + 1) // 2) * 2)
        noise = math.sqrt((1 + pf) ** 2 + pf ** 2)
        oracle_cpu.ranger_lite_update(p, g, gm, ngm, vm, slow if merge else None, beta2=beta2, bias_correction2=bc2,
                                      beta1=beta1 ** 2, one_minus_beta1=1 - beta1 ** 2, one_plus_pnm=1 + pf,
                                      pnm_factor=pf, noise_norm=noise, lr_div_bc1=lr / bc1, eps=eps, step=step,
                                      wd_factor=wd, update_variance=not phase2, alpha=0.5)
        nat.check(lib.nnueft_ranger_lite_update_pnm(dp.data_ptr(), dg.data_ptr(), dgm.data_ptr(), dngm.data_ptr(),
                                                    dvm.data_ptr(), n, beta2, 1 - beta2, bc2, beta1 ** 2,
                                                    1 - beta1 ** 2, 1 + pf, pf, noise, lr / bc1, eps, step, wd,
                                                    0 if phase2 else 1, dslow.data_ptr() if merge else None, 0.5,
                                                    _stream()), "pnm")
    for name, h, d in zip("p grad grad_ma neg_grad_ma variance_ma slow".split(), host, dev):
        assert np.array_equal(d.cpu().numpy(), h), name


@pytest.mark.parametrize("n", [2, 1025, 300000])
def test_variance_and_merge_kernels_bit_exact(oracle_cpu, n):
    nat, lib = _native()
    p, g, _, _, vm, slow = _state(n, n)
    dp, dg, dvm, dslow = [torch.from_numpy(a).to(DEV) for a in (p, g, vm, slow)]
    oracle_cpu.ranger_lite_update_variance(g, vm, 0.999)
    nat.check(lib.nnueft_ranger_lite_update_variance(dg.data_ptr(), dvm.data_ptr(), n, 0.999, 1 - 0.999, _stream()),
              "variance")
    assert np.array_equal(dvm.cpu().numpy(), vm)
    nat.check(lib.nnueft_ranger_lite_lookahead_merge(dp.data_ptr(), dslow.data_ptr(), n, 0.25, _stream()), "merge")
    expect = p * F(0.25) + slow * F(0.75)
    assert np.array_equal(dp.cpu().numpy(), expect) and np.array_equal(dslow.cpu().numpy(), expect)


@pytest.mark.parametrize("kw", [dict(), dict(pnm_activate=False), dict(lookahead_active=False),
                                dict(weight_decay=0.05), dict(weight_decay=0.05, pnm_activate=False)],
                         ids=["default", "adam", "no_lookahead", "decay", "decay_adam"])
def test_class_on_gpu_follows_its_cpu_path(kw):
    shapes = ((300, 40), (40,), (8, 16, 3), (1,))
    g0 = torch.Generator().manual_seed(3)
    cpu = [torch.nn.Parameter(torch.randn(*s, generator=g0)) for s in shapes]
    gpu = [torch.nn.Parameter(p.detach().clone().to(DEV)) for p in cpu]
    wd = kw.pop("weight_decay", 0.0)
    groups = lambda ps: [{"params": ps[:2], "lr": 1e-2, "weight_decay": wd}, {"params": ps[2:], "lr": 3e-3}]
    oc = RangerLite(groups(cpu), normloss_active=False, **kw)
    og = RangerLite(groups(gpu), normloss_active=False, **kw)
    for s in range(11):            # two lookahead merges
        gen = torch.Generator().manual_seed(100 + s)
        for a, b in zip(cpu, gpu):
            a.grad = torch.randn(a.shape, generator=gen)
            b.grad = a.grad.to(DEV)
        oc.step()
        og.step()
        for a, b in zip(cpu, gpu):
            torch.testing.assert_close(b.detach().cpu(), a.detach(), rtol=2e-5, atol=2e-6)
    for a, b in zip(cpu, gpu):
        for key in oc.state[a]:
            x, y = oc.state[a][key], og.state[b][key]
            if torch.is_tensor(x):
                torch.testing.assert_close(y.cpu(), x, rtol=2e-5, atol=2e-6)
            else:
                assert x == y
    og.eval()
    for a, b in zip(cpu, gpu):
        if "lookahead_params" in oc.state[a]:
            torch.testing.assert_close(b.detach().cpu(), oc.state[a]["lookahead_params"], rtol=2e-5, atol=2e-6)
    og.train()


@pytest.mark.parametrize("kw", [dict(), dict(pnm_activate=False), dict(weight_decay=0.05)], ids=["default", "adam", "decay"])
def test_multi_tensor_launch_gives_the_bits_of_single_launches(kw):
    """Small tensors are updated several per launch; the arithmetic per element is the same, so two
    optimizers that differ only in that threshold stay equal bit for bit (20 tensors: two launches)."""
    g0 = torch.Generator().manual_seed(5)
    shapes = [(257,), (3, 70), (1,), (64, 33)] * 5
    one = [torch.nn.Parameter(torch.randn(*s, generator=g0).to(DEV)) for s in shapes]
    many = [torch.nn.Parameter(p.detach().clone()) for p in one]
    wd = kw.pop("weight_decay", 0.0)
    groups = lambda ps: [{"params": ps[:7], "lr": 1e-2, "weight_decay": wd}, {"params": ps[7:], "lr": 3e-3, "betas": (0.8, 0.99)}]
    o1 = RangerLite(groups(one), normloss_active=False, **kw)
    o1.MULTI_TENSOR_BELOW = 0
    o2 = RangerLite(groups(many), normloss_active=False, **kw)
    for s in range(7):
        gen = torch.Generator().manual_seed(200 + s)
        for a, b in zip(one, many):
            a.grad = torch.randn(a.shape, generator=gen).to(DEV)
            b.grad = a.grad.clone()
        o1.step()
        o2.step()
    for a, b in zip(one, many):
        assert torch.equal(a, b)
        for key, x in o1.state[a].items():
            if torch.is_tensor(x):
                assert torch.equal(x, o2.state[b][key])
