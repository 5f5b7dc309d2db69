"""The callers of the operator (quantization constants, feature block, FT module, layer stacks, loss)
on the CPU: closed forms, known answers and round trips."""
import math

import numpy as np
import pytest
import torch

from nnueft import halfka_v2_hm as hk
from nnueft import model as M


def test_quantization_constants():
    # literals of model/quantize.py:58-113
    q = M.QuantizationManager(M.QuantizationConfig())
    assert q.l0_correction_factor == 1.0                       # 256^2 / 512 / 128
    assert q.sqr_crelu_correction_factor == 1.0
    assert q.max_ft_activation == 255 / 256 and q.max_hidden_activation == 127 / 128
    assert q.weight_scales_dict["ft_weight"] == 256 and q.weight_scales_dict["ft_psqt_weight"] == 9600
    assert q.weight_scales_dict["ls_l1_bias"] == 128 * 128 and q.weight_scales_dict["ls_l2_weight"] == 64
    assert q.max_hidden_weight == [127 / 128, 127 / 64, 127 / 128]
    assert (255 * 255) >> 9 == 127


def test_fake_quantization_known_answers():
    q = M.QuantizationManager(M.QuantizationConfig())
    x = torch.tensor([0.0, 1 / 512, 3 / 512, 0.30, -0.30, 1.0], requires_grad=True)
    w = q.fake_quantize_weights(x, "ft_weight")
    # round half to even on x*256: 0.5 -> 0, 1.5 -> 2, 76.8 -> 77
    assert w.tolist() == [0.0, 0.0, 2 / 256, 77 / 256, -77 / 256, 1.0]
    w.sum().backward()
    assert x.grad.tolist() == [1.0] * 6                        # straight-through
    a = q.fake_quantize_ft_act(torch.tensor([0.0, 0.999, 0.5, 127.9 / 128]))
    assert a.tolist() == [0.0, 127 / 128, 0.5, 127 / 128]      # floor(x*128 + 1e-5) / 128
    o = q.fake_quantize_output(torch.tensor([[0.1234], [-0.1234]]))
    den, mult = 128 * 128 * 2, 9600
    want = math.trunc(round(0.1234 * den) * mult / den) / mult
    assert o[:, 0].tolist() == [float(np.float32(want)), -float(np.float32(want))]


def test_export_remap_closed_form_and_round_trip():
    torch.manual_seed(0)
    f = M.HalfKav2Hm(4)
    with torch.no_grad():
        f.weight.copy_(torch.arange(hk.NUM_INPUTS * 4, dtype=torch.float32).reshape(-1, 4))
    exp = f.get_export_weights()
    assert exp.shape == (hk.NUM_INPUTS_EXPORT, 4)
    inv = {int(b): sq for sq, b in enumerate(hk.KING_BUCKETS) if b >= 0}
    for b in (0, 7, 31):
        s0, d0, ksq = b * 768, b * 704, inv[b]
        assert torch.equal(exp[d0:d0 + 640], f.weight[s0:s0 + 640])
        for sq in range(64):
            src = s0 + 640 + sq if sq == ksq else s0 + 704 + sq      # own king only on its own square
            assert torch.equal(exp[d0 + 640 + sq], f.weight[src])
    g = M.HalfKav2Hm(4)
    g.load_export_weights(exp)
    assert torch.equal(g.get_export_weights(), exp)                 # identity on the exported rows
    # rows the export drops are zero after the round trip
    assert not g.weight[640:704][[s for s in range(64) if s != inv[0]]].any()
    assert not g.weight[704 + inv[0]].any()
    # virtual weights are folded in
    with torch.no_grad():
        f.virtual_weight.fill_(1.0)
    assert torch.equal(f.get_export_weights(), exp + 1.0)


def test_psqt_initial_values():
    vals = M.HalfKav2Hm.halfka_psqts()
    assert len(vals) == hk.NUM_INPUTS
    assert vals[hk.feature_index(hk.WHITE, 4, 12, hk.PAWN, hk.WHITE)] == 126
    assert vals[hk.feature_index(hk.WHITE, 4, 12, hk.QUEEN, hk.BLACK)] == -2538
    assert vals[hk.feature_index(hk.WHITE, 4, 4, hk.KING, hk.WHITE)] == 0
    v = np.array(vals).reshape(32, 12, 64)
    assert np.array_equal(v[:, 0::2], -v[:, 1::2])                  # own / opposing piece blocks mirror
    assert set(np.unique(np.abs(v))) == {0, 126, 781, 825, 1276, 2538}


def test_composed_ft_cpu_matches_explicit_formula():
    torch.manual_seed(1)
    q = M.QuantizationManager(M.QuantizationConfig())
    ft = M.ComposedFeatureTransformer([M.HalfKav2Hm], 32, 8, q)
    ft.init_weights()
    with torch.no_grad():
        ft.features[0].virtual_weight.normal_(0, 0.01)
    assert ft.NUM_INPUTS == 24576 and ft.MAX_ACTIVE_FEATURES == 32 and ft.HASH == 0x7F234CB8
    us, them, white, black, pc = [torch.from_numpy(a) for a in hk.synthetic_batch(16, 3)]
    psqt = (pc - 1) // 4
    l0, wp, bp = ft(us, them, white, black, psqt, True, True)
    f = ft.features[0]
    merged = f.weight + f.virtual_weight.repeat(32, 1)
    merged = torch.cat([(merged[:, :32] * 256).round() / 256, (merged[:, 32:] * 9600).round() / 9600], 1)
    bias = torch.cat([(ft.bias[:32] * 256).round() / 256, torch.zeros(8)])
    from oracle import ref_torch

    r_l0, r_wp, r_bp = ref_torch.double_feature_transform(us, them, white, black, psqt, merged, bias, 255 / 256, 32)
    assert torch.equal(l0, torch.floor(r_l0 * 128 + 1e-5) / 128)
    assert torch.equal(wp, r_wp) and torch.equal(bp, r_bp)
    (l0.sum() + wp.sum()).backward()
    assert f.weight.grad is not None and f.virtual_weight.grad is not None and ft.bias.grad is not None
    # the virtual gradient is the block sum of the real one
    assert torch.allclose(f.virtual_weight.grad, f.weight.grad.view(32, 768, -1).sum(0), atol=1e-5)


def test_stacked_linear_equals_per_bucket_layers():
    torch.manual_seed(2)
    q = M.QuantizationManager(M.QuantizationConfig())
    sl = M.FactorizedStackedLinear(16, 4, 8, q, "ls_l1")
    with torch.no_grad():
        sl.linear.weight.normal_()
        sl.factorized_linear.weight.normal_()
        sl.factorized_linear.bias.normal_()
    x = torch.randn(10, 16)
    idx = torch.randint(0, 8, (10,))
    out = sl(x, idx)
    for i in range(10):
        layer = sl.at_index(int(idx[i]))
        w = sl.linear.weight[int(idx[i]) * 4:int(idx[i]) * 4 + 4] + sl.factorized_linear.weight
        assert torch.allclose(layer.weight, w)
        assert torch.allclose(out[i], layer(x[i]), atol=1e-5)


def test_loss_closed_forms():
    p = M.LossParams()
    # prediction and target on the same win-rate curve: loss 0
    same = M.LossParams(in_scaling=380, out_scaling=380)
    s = torch.tensor([[-300.0], [0.0], [150.0]])
    assert float(M.sf_loss(s, s, torch.zeros(3, 1), same, 1.0)) == 0.0
    # one sample, lambda = 0: |outcome - qf|^2.5
    sc = torch.tensor([[100.0]])
    qf = 0.5 * (1 + torch.sigmoid((sc - 270) / 340) - torch.sigmoid((-sc - 270) / 340))
    got = M.sf_loss(sc, torch.tensor([[0.0]]), torch.tensor([[1.0]]), p, 0.0)
    assert float(got) == pytest.approx(float((1.0 - qf).abs() ** 2.5), rel=1e-6)
    # antisymmetry of the win-rate model: qf(0) = 0.5
    assert float(M.sf_loss(torch.zeros(1, 1), torch.zeros(1, 1), torch.full((1, 1), 0.5), p, 0.3)) == 0.0
    # tablebase scores are remapped, ordinary scores are not
    r = M.remap_tablebase_score(torch.tensor([100.0, 31990.0, -31990.0]), 4000.0, 4000.0, 0.85)
    assert r[0] == 100.0 and r[1] == pytest.approx(4000 + 0.85 ** 10 * 4000) and r[2] == -r[1]


def test_full_model_forward_backward_cpu():
    torch.manual_seed(3)
    model = M.NNUEModel("HalfKAv2_hm^", M.ModelConfig(L1=64, L2=16, L3=32))
    us, them, white, black, pc = [torch.from_numpy(a) for a in hk.synthetic_batch(32, 4)]
    out = model(us, them, white, black, pc)
    assert out.shape == (32, 1) and torch.isfinite(out).all()
    loss = M.sf_loss(out * 600.0, torch.randn(32, 1) * 400, torch.full((32, 1), 0.5), M.LossParams(), 1.0)
    loss.backward()
    for name, prm in model.named_parameters():
        assert prm.grad is not None and torch.isfinite(prm.grad).all(), name
    # material only: the PSQT initialisation makes the side with more material score higher
    assert float(model.input.features[0].weight[:, 64:].detach().abs().max()) == pytest.approx(2538 / 600)


def test_oracle_table_functions(oracle_cpu):
    rng = np.random.default_rng(0)
    W = rng.standard_normal((48, 12)).astype(np.float32)
    V = rng.standard_normal((16, 12)).astype(np.float32)
    m = oracle_cpu.table_merge(W, V, 8)
    t = torch.from_numpy(W) + torch.from_numpy(V).repeat(3, 1)
    t = torch.cat([(t[:, :8] * 256).round() / 256, (t[:, 8:] * 9600).round() / 9600], 1)
    assert np.array_equal(m, t.numpy())
    assert np.array_equal(oracle_cpu.table_merge(W, V, 8, fake_quantize=False),
                          (torch.from_numpy(W) + torch.from_numpy(V).repeat(3, 1)).numpy())
    g = rng.integers(-9, 9, size=(48, 12)).astype(np.float32)
    assert np.array_equal(oracle_cpu.table_virtual_grad(g, 16), g.reshape(3, 16, 12).sum(0))


# The reference trains under torch.compile (train.py:296) and saves whole modules with torch.save;
# both must keep working with the operators of this build in the graph.
def _tiny_model_and_batch():
    from nnueft import halfka_v2_hm as hk

    torch.manual_seed(0)
    m = M.NNUEModel("HalfKAv2_hm^", M.ModelConfig(L1=64, L2=8, L3=16))
    batch = [torch.from_numpy(a) for a in hk.synthetic_batch(32, 3)]
    return m, batch


def test_module_survives_torch_save_and_load():
    import io

    m, batch = _tiny_model_and_batch()
    out = m(*batch)
    buf = io.BytesIO()
    torch.save(m, buf)            # a file this test wrote itself
    buf.seek(0)
    m2 = torch.load(buf, weights_only=False)
    assert torch.equal(m2(*batch), out)
    buf = io.BytesIO()
    torch.save(m.state_dict(), buf)
    buf.seek(0)
    m3 = M.NNUEModel("HalfKAv2_hm^", M.ModelConfig(L1=64, L2=8, L3=16))
    m3.load_state_dict(torch.load(buf, weights_only=True))
    assert torch.equal(m3(*batch), out)


@pytest.mark.parametrize("backend", ["eager", "aot_eager"])
def test_model_under_torch_compile_on_cpu(backend):
    m, batch = _tiny_model_and_batch()
    out = m(*batch)
    out.sum().backward()
    ref = {n: p.grad.clone() for n, p in m.named_parameters()}
    m.zero_grad()
    torch._dynamo.reset()
    cm = torch.compile(m, backend=backend)
    o = cm(*batch)
    o.sum().backward()
    assert torch.allclose(o, out, atol=1e-6)
    for n, p in m.named_parameters():
        assert torch.allclose(p.grad, ref[n], atol=1e-5), n


@pytest.mark.parametrize("post_mul", [1.0, 0.75, 1.3])
def test_act_fake_quantize_oracle_equals_the_torch_ops(oracle_cpu, post_mul):
    g = torch.Generator().manual_seed(21)
    x = torch.cat([torch.rand(5000, generator=g), torch.randn(3000, generator=g) * 3,
                   torch.arange(0, 129).float() / 128, torch.tensor([0.0, -0.0, 127 / 128, 1.0, 1e-6, -1e-6])])
    q = M.QuantizationManager(M.QuantizationConfig())
    ref = q.fake_quantize_ft_act(x) * post_mul           # mul, add, floor, div, then the correction factor
    got = oracle_cpu.act_fake_quantize(x.numpy(), scale=q.hidden_quantized_one, eps=M.FAKE_QUANTIZE_EPS,
                                       post_mul=post_mul)
    assert np.array_equal(got, ref.numpy())
    # the grid: multiples of 1/128, never above x by more than the epsilon's worth
    if post_mul == 1.0:
        assert np.array_equal(got * 128, np.floor(got * 128))
        assert (got <= x.numpy() + 1e-5 / 128 + 1e-7).all()


@pytest.mark.parametrize("B,n_in,out,count", [(50, 64, 5, 3), (300, 96, 16, 8), (64, 32, 32, 1)])
def test_bucket_linear_oracle_equals_wide_layer_and_selection(oracle_cpu, B, n_in, out, count):
    # the reference's formula (stacked_linear.py:38-66): F.linear over all blocks, reshape, pick one block per position
    import torch.nn.functional as F

    rng = np.random.default_rng(B)
    x = rng.standard_normal((B, n_in)).astype(np.float32)
    W = rng.standard_normal((count * out, n_in)).astype(np.float32)
    b = rng.standard_normal(count * out).astype(np.float32)
    k = rng.integers(0, count, size=B)
    gy = rng.standard_normal((B, out)).astype(np.float32)
    tx, tW, tb = [torch.from_numpy(a).requires_grad_() for a in (x, W, b)]
    wide = F.linear(tx, tW, tb).reshape(-1, out)
    y = wide[torch.from_numpy(k) + torch.arange(0, B * count, count)]
    y.backward(torch.from_numpy(gy))
    assert np.allclose(oracle_cpu.bucket_linear_fwd(x, k, W, b, out, count), y.detach().numpy(), rtol=1e-5, atol=1e-5)
    gx, gW, gb = oracle_cpu.bucket_linear_bwd(x, k, W, gy, out, count)
    assert np.allclose(gx, tx.grad.numpy(), rtol=1e-5, atol=1e-5)
    assert np.allclose(gW, tW.grad.numpy(), rtol=1e-5, atol=1e-5)
    assert np.allclose(gb, tb.grad.numpy(), rtol=1e-5, atol=1e-5)


def test_synthetic_training_loop_on_cpu():
    """The thin loop (host batches -> prefetcher -> model -> loss -> RangerLite) on the CPU path."""
    from nnueft import train_synthetic

    losses, rate = train_synthetic.run(steps=14, batch_size=256, l1=64, device="cpu", lr=2e-3)
    assert len(losses) == 14 and all(np.isfinite(losses)) and losses[-1] < losses[0] and rate > 0


def test_loss_with_a_per_sample_lambda_tensor():
    """The reference's jittered lambda schedule hands sf_loss one lambda per sample (model/lambda_utils.py:69-83);
    the loss must take it (through the torch formula) and agree with per-sample evaluation."""
    p = M.LossParams()
    g = torch.Generator().manual_seed(1)
    net = torch.randn(6, 1, generator=g) * 300
    score = torch.randn(6, 1, generator=g) * 400
    outcome = torch.tensor([[0.0], [0.5], [1.0], [1.0], [0.0], [0.5]])
    lam = torch.tensor([[1.0], [0.75], [0.5], [0.0], [0.9], [0.3]])
    got = M.sf_loss(net, score, outcome, p, lam)
    each = torch.stack([M.sf_loss(net[i:i + 1], score[i:i + 1], outcome[i:i + 1], p, float(lam[i])) for i in range(6)])
    assert float(got) == pytest.approx(float(each.mean()), rel=1e-6)     # weights are 1 at w1 = 0
    assert float(M.sf_loss(net, score, outcome, p, torch.tensor(0.75))) == \
        pytest.approx(float(M.sf_loss(net, score, outcome, p, 0.75)), rel=1e-6)


def test_clip_weights_bounds_what_gets_exported():
    """NNUEModel.clip_weights (model/model.py:42-72): the layer-stack weights end inside the range of their int8
    image; for the first layer the bound applies to real + shared weight, which is what the export sums."""
    torch.manual_seed(5)
    m = M.NNUEModel("HalfKAv2_hm^", M.ModelConfig(L1=64, L2=16, L3=32))
    ls, q = m.layer_stacks, m.quantization
    with torch.no_grad():
        ls.l1.linear.weight.normal_(0, 3.0)
        ls.l1.factorized_linear.weight.normal_(0, 0.5)
        ls.l2.linear.weight.normal_(0, 5.0)
        ls.output.linear.weight.normal_(0, 5.0)
    before_input = m.input.features[0].weight.clone()
    m.clip_weights(include_input=True)
    assert torch.equal(m.input.features[0].weight, before_input)          # HalfKAv2_hm clips nothing
    v = ls.l1.factorized_linear.weight
    total = ls.l1.linear.weight + v.repeat(ls.l1.linear.weight.shape[0] // v.shape[0], 1)
    total = total.detach()
    assert float(total.abs().max()) <= q.max_hidden_weight[0] * (1 + 1e-6)
    assert float((total.abs() - q.max_hidden_weight[0]).abs().min()) < 1e-6      # and the bound is reached
    assert float(ls.l2.linear.weight.detach().abs().max()) == pytest.approx(q.max_hidden_weight[1])
    assert float(ls.output.linear.weight.detach().abs().max()) == pytest.approx(q.max_hidden_weight[2])
    assert q.max_hidden_weight == pytest.approx([127 / 128, 127 / 64, 127 / 128])   # weights x128 / x64 / x128


def test_train_clip_write_read_round_trip():
    """A few optimizer steps with a large learning rate push layer-stack weights past the int8 range; without the
    clip the writer refuses the net, with it the file reads back to the model's quantized tensors."""
    import io

    from nnueft import serialize as S
    from nnueft.optim import RangerLite

    torch.manual_seed(9)
    m = M.NNUEModel("HalfKAv2_hm^", M.ModelConfig(L1=64, L2=15, L3=32))
    opt = RangerLite(M.optimizer_param_groups(m, lr=0.8), normloss_active=False)
    us, them, white, black, pc = [torch.from_numpy(a) for a in hk.synthetic_batch(64, 8)]
    g = torch.Generator().manual_seed(2)
    score, outcome = torch.randn(64, 1, generator=g) * 400, torch.full((64, 1), 0.5)
    for _ in range(4):
        opt.zero_grad()
        loss = M.sf_loss(m(us, them, white, black, pc) * 600.0, score, outcome, M.LossParams(), 1.0)
        loss.backward()
        opt.step()
    assert float(m.layer_stacks.l2.linear.weight.detach().abs().max()) > m.quantization.max_hidden_weight[1]
    with pytest.raises(RuntimeError, match="out of bounds"):
        S.NNUEWriter(m, "unclipped")
    m.clip_weights(include_input=True)
    buf = bytes(S.NNUEWriter(m, "clipped").buf)
    back = S.NNUEReader(io.BytesIO(buf), "HalfKAv2_hm^", M.ModelConfig(L1=64, L2=15, L3=32)).model
    assert bytes(S.NNUEWriter(back, "clipped").buf) == buf
