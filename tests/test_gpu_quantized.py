"""Quantized inference on the GPU (BASELINE config 5): int16 feature transformer, then the int8 layer
stacks, bit-exact against the integer oracle; and the whole chain against the float model it was
quantized from."""
import numpy as np
import pytest
import torch

from nnueft import halfka_v2_hm as hk
from nnueft import model as M
from nnueft import quantized

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.mark.parametrize("B,L1,L2,L3,count", [(50, 64, 16, 32, 8), (33, 3072, 32, 32, 8), (7, 40, 6, 5, 3),
                                              (4096, 1024, 16, 32, 8)])
def test_stack_int8_against_oracle(oracle_cpu, B, L1, L2, L3, count):
    rng = np.random.default_rng(B + L1)
    x = rng.integers(0, 128, size=(B, L1)).astype(np.uint8)
    bucket = rng.integers(0, count, size=B).astype(np.int64)
    W1 = rng.integers(-30, 31, size=(count * L2, L1)).astype(np.int8)
    b1 = rng.integers(-200000, 200000, size=count * L2).astype(np.int32)
    W2 = rng.integers(-127, 128, size=(count * L3, 2 * L2)).astype(np.int8)
    b2 = rng.integers(-20000, 20000, size=count * L3).astype(np.int32)
    Wo = rng.integers(-127, 128, size=(count, 2 * L2 + 2 * L3)).astype(np.int8)
    bo = rng.integers(-50000, 50000, size=count).astype(np.int32)
    t = lambda a: torch.from_numpy(a).to(DEV)
    got = quantized.stack_int8_forward(t(x), t(bucket), t(W1), t(b1), t(W2), t(b2), t(Wo), t(bo))
    want = oracle_cpu.stack_int8_fwd(x, bucket, W1, b1, W2, b2, Wo, bo, L2, L3, count)
    assert np.array_equal(got.cpu().numpy(), want)
    assert len(np.unique(want)) > min(B, 20) // 2


def test_config_5_end_to_end_at_full_size(oracle_cpu):
    """BASELINE.json config 5 as a whole at its real size: L1=3072, B=65536, exported numbering (22528 rows); the
    int16 feature transformer, then the int8 layer stacks of a quantized model (L2=32 and the literal 15+1), every
    output bit-equal to the CPU integer evaluation of the same quantized tensors."""
    L1, B, R = 3072, 65536, hk.NUM_INPUTS_EXPORT
    us, them, white, black, pc = hk.synthetic_batch(B, 1239, fold_kings=True)
    g = torch.Generator().manual_seed(5)
    W = torch.randn(R, L1 + 8, generator=g) * 0.02
    W[:, L1:] = torch.randn(R, 8, generator=g) * 0.5
    bias = torch.randn(L1 + 8, generator=g) * 0.1
    w16, b16, p32 = quantized.quantize_feature_transformer(W, bias, L1)
    stm = (1 - us[:, 0]).astype(np.uint8)
    bucket = ((pc - 1) // 4).astype(np.int64)
    t = lambda a: torch.from_numpy(a).to(DEV)
    x_u8, psqt = quantized.ft_int16_forward(t(white), t(black), t(stm), w16.to(DEV), b16.to(DEV), p32.to(DEV), t(bucket))
    r_x, r_ps = oracle_cpu.ft_int16_fwd(white, black, stm, w16.numpy(), b16.numpy(), p32.numpy(), bucket)
    assert np.array_equal(x_u8.cpu().numpy(), r_x) and np.array_equal(psqt.cpu().numpy(), r_ps)
    for L2 in (32, 16):
        torch.manual_seed(5 + L2)
        stacks = M.LayerStacks(8, M.ModelConfig(L1=L1, L2=L2, L3=32), M.QuantizationManager(M.QuantizationConfig()))
        with torch.no_grad():
            stacks.l1.linear.weight.mul_(0.5)
            stacks.l1.factorized_linear.weight.normal_(0, 0.004)
        stack = quantized.quantize_layer_stacks(stacks)
        out = quantized.stack_int8_forward(x_u8, t(bucket), *[s.to(DEV) for s in stack])
        want = oracle_cpu.stack_int8_fwd(r_x, bucket, *[s.numpy() for s in stack], L2, 32, 8)
        assert np.array_equal(out.cpu().numpy(), want)
        total = out.cpu().numpy().astype(np.int64) + r_ps
        assert len(np.unique(total)) > 1000 and np.abs(out.cpu().numpy()).max() > 0


def test_quantized_chain_tracks_the_float_model(oracle_cpu):
    """Export a float model (weights on the quantization grid so that nothing is lost in the export),
    evaluate it with the integer kernels, compare with its own fake-quantized float forward."""
    torch.manual_seed(2)
    L1, B = 256, 512
    model = M.NNUEModel("HalfKAv2_hm^", M.ModelConfig(L1=L1, L2=16, L3=32)).double()
    f = model.input.features[0]
    with torch.no_grad():
        f.weight[:, :L1] = torch.randint(-12, 13, (hk.NUM_INPUTS, L1)) / 256.0
        model.input.bias[:L1] = torch.randint(0, 60, (L1,)) / 256.0
        ls = model.layer_stacks
        ls.l1.linear.weight.copy_(torch.randint(-20, 21, ls.l1.linear.weight.shape) / 128.0)
        ls.l1.linear.bias.copy_(torch.randint(-9000, 9000, ls.l1.linear.bias.shape) / 16384.0)
        ls.l2.linear.weight.copy_(torch.randint(-127, 128, ls.l2.linear.weight.shape) / 64.0)
        ls.l2.linear.bias.copy_(torch.randint(-4000, 4000, ls.l2.linear.bias.shape) / 8192.0)
        ls.output.linear.weight.copy_(torch.randint(-127, 128, ls.output.linear.weight.shape) / 128.0)
    us, them, white, black, pc = hk.synthetic_batch(B, 21)
    with torch.no_grad():
        fl = model(torch.from_numpy(us).double(), torch.from_numpy(them).double(), torch.from_numpy(white),
                   torch.from_numpy(black), torch.from_numpy(pc), True, True)[:, 0]
    # exported tensors: 22528-row table, int16 / int32 / int8
    export = model.input.get_export_weights().float()
    w16, b16, p32 = quantized.quantize_feature_transformer(export, model.input.bias.detach().float(), L1)
    stack = quantized.quantize_layer_stacks(model.layer_stacks)
    _, _, wf, bf, _ = hk.synthetic_batch(B, 21, fold_kings=True)
    t = lambda a: torch.from_numpy(a).to(DEV)
    stm = t((1 - us[:, 0]).astype(np.uint8))
    bucket = t((pc - 1) // 4)
    x_u8, psqt = quantized.ft_int16_forward(t(wf), t(bf), stm, w16.to(DEV), b16.to(DEV), p32.to(DEV), bucket)
    out = quantized.stack_int8_forward(x_u8, bucket, *[s.to(DEV) for s in stack])
    total = (out + psqt).cpu().numpy().astype(np.float64) / 9600.0        # net units
    want = fl.numpy()
    # the integer chain rounds the psqt term and the final division once each: within 2/9600
    assert np.abs(total - want).max() <= 2.5 / 9600.0
    # and it is exactly the integer oracle
    r_x, r_ps = oracle_cpu.ft_int16_fwd(wf, bf, stm.cpu().numpy(), w16.numpy(), b16.numpy(), p32.numpy(),
                                        ((pc - 1) // 4))
    assert np.array_equal(x_u8.cpu().numpy(), r_x) and np.array_equal(psqt.cpu().numpy(), r_ps)
    r_out = oracle_cpu.stack_int8_fwd(r_x, (pc - 1) // 4, *[s.numpy() for s in stack], 16, 32, 8)
    assert np.array_equal(out.cpu().numpy(), r_out)


@pytest.mark.parametrize("compression", ["none", "leb128"])
def test_net_read_back_from_a_nnue_file_evaluates_the_same(compression):
    """model -> .nnue bytes -> model: the integer kernels give the same outputs for both."""
    import io

    from nnueft import serialize as S

    torch.manual_seed(5)
    L1, B = 128, 300
    cfg = dict(L1=L1, L2=15, L3=32)
    model = M.NNUEModel("HalfKAv2_hm^", M.ModelConfig(**cfg))
    with torch.no_grad():
        model.input.features[0].virtual_weight.normal_(0, 0.01)
        model.layer_stacks.l1.factorized_linear.weight.normal_(0, 0.01)
    buf = bytes(S.NNUEWriter(model, "round trip", compression).buf)
    back = S.NNUEReader(io.BytesIO(buf), "HalfKAv2_hm^", M.ModelConfig(**cfg)).model
    us, _, _, _, pc = hk.synthetic_batch(B, 31)
    _, _, wf, bf, _ = hk.synthetic_batch(B, 31, fold_kings=True)
    t = lambda a: torch.from_numpy(a).to(DEV)
    stm, bucket = t((1 - us[:, 0]).astype(np.uint8)), t((pc - 1) // 4)
    outs = []
    for m in (model, back):
        w16, b16, p32 = quantized.quantize_feature_transformer(m.input.get_export_weights().float(),
                                                               m.input.bias.detach().float(), L1)
        x_u8, psqt = quantized.ft_int16_forward(t(wf), t(bf), stm, w16.to(DEV), b16.to(DEV), p32.to(DEV), bucket)
        out = quantized.stack_int8_forward(x_u8, bucket, *[s.to(DEV) for s in quantized.quantize_layer_stacks(m.layer_stacks)])
        outs.append((x_u8.cpu(), psqt.cpu(), out.cpu()))
    for a, b in zip(*outs):
        assert torch.equal(a, b)
