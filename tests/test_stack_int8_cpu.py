"""Pins the integer layer-stack oracle: brute force in Python integers, and the fake-quantized float
module (nnueft.model.LayerStacks, i.e. model/modules/layer_stacks.py:33-84) evaluated in float64 on
weights that are exactly representable -- there every float step is exact and must equal its integer
image."""
import numpy as np
import torch

from nnueft import model as M
from nnueft import quantized


def _random_stack(rng, L1, L2, L3, count):
    W1 = rng.integers(-20, 21, size=(count * L2, L1)).astype(np.int8)
    b1 = rng.integers(-200000, 200000, size=count * L2).astype(np.int32)
    W2 = rng.integers(-127, 128, size=(count * L3, 2 * L2)).astype(np.int8)
    b2 = rng.integers(-20000, 20000, size=count * L3).astype(np.int32)
    Wo = rng.integers(-127, 128, size=(count, 2 * L2 + 2 * L3)).astype(np.int8)
    bo = rng.integers(-50000, 50000, size=count).astype(np.int32)
    return W1, b1, W2, b2, Wo, bo


def _brute(x, bucket, W1, b1, W2, b2, Wo, bo, L2, L3):
    out = []
    clip = lambda v: max(0, min(127, v))
    for p in range(x.shape[0]):
        k = int(bucket[p])
        a1 = [int(b1[k * L2 + o]) + sum(int(w) * int(v) for w, v in zip(W1[k * L2 + o], x[p])) for o in range(L2)]
        y1 = [clip((a * a) >> 21) for a in a1] + [clip(a >> 7) for a in a1]
        a2 = [int(b2[k * L3 + j]) + sum(int(w) * v for w, v in zip(W2[k * L3 + j], y1)) for j in range(L3)]
        y2 = [clip((a * a) >> 19) for a in a2] + [clip(a >> 6) for a in a2]
        a3 = int(bo[k]) + sum(int(w) * v for w, v in zip(Wo[k], y1 + y2))
        num = 2 * (a3 + a1[L2 - 2] - a1[L2 - 1]) * 9600
        out.append(int(num / 32768) if abs(num) < 2 ** 52 else None)   # truncation toward zero
    return np.array(out, np.int64)


def test_stack_oracle_brute_force(oracle_cpu):
    rng = np.random.default_rng(0)
    B, L1, L2, L3, count = 24, 40, 6, 5, 3
    x = rng.integers(0, 128, size=(B, L1)).astype(np.uint8)
    bucket = rng.integers(0, count, size=B).astype(np.int64)
    t = _random_stack(rng, L1, L2, L3, count)
    got = oracle_cpu.stack_int8_fwd(x, bucket, *t, L2, L3, count)
    want = _brute(x, bucket, *t, L2, L3)
    assert np.array_equal(got.astype(np.int64), want)
    assert (got != 0).any() and (got < 0).any() and (got > 0).any()


def test_stack_oracle_equals_fake_quantized_float_module(oracle_cpu):
    torch.manual_seed(1)
    L1, L2, L3, count, B = 64, 16, 32, 8, 400
    cfg = M.ModelConfig(L1=L1, L2=L2, L3=L3)
    q = M.QuantizationManager(cfg.quantize_config)
    ls = M.LayerStacks(count, cfg, q).double()
    with torch.no_grad():   # weights on the quantization grid, different per bucket
        ls.l1.linear.weight.copy_(torch.randint(-40, 41, ls.l1.linear.weight.shape) / 128.0)
        ls.l1.linear.bias.copy_(torch.randint(-9000, 9000, ls.l1.linear.bias.shape) / 16384.0)
        ls.l1.factorized_linear.weight.copy_(torch.randint(-10, 11, ls.l1.factorized_linear.weight.shape) / 128.0)
        ls.l2.linear.weight.copy_(torch.randint(-127, 128, ls.l2.linear.weight.shape) / 64.0)
        ls.l2.linear.bias.copy_(torch.randint(-4000, 4000, ls.l2.linear.bias.shape) / 8192.0)
        ls.output.linear.weight.copy_(torch.randint(-127, 128, ls.output.linear.weight.shape) / 128.0)
        ls.output.linear.bias.copy_(torch.randint(-9000, 9000, ls.output.linear.bias.shape) / 16384.0)
    w1, b1, w2, b2, wo, bo = quantized.quantize_layer_stacks(ls)
    assert w1.dtype == torch.int8 and b1.dtype == torch.int32 and w1.shape == (count * L2, L1)
    xq = torch.randint(0, 128, (B, L1), dtype=torch.uint8)
    bucket = torch.randint(0, count, (B,))
    with torch.no_grad():
        fl = ls(xq.double() / 128.0, bucket, True, True)          # fake quantization of acts and weights on
    want = torch.round(fl[:, 0] * 9600.0).to(torch.int64).numpy()
    got = oracle_cpu.stack_int8_fwd(xq.numpy(), bucket.numpy(), w1.numpy(), b1.numpy(), w2.numpy(), b2.numpy(),
                                    wo.numpy(), bo.numpy(), L2, L3, count)
    assert np.array_equal(got.astype(np.int64), want)
    assert len(np.unique(got)) > B // 4
