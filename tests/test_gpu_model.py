"""The module layer above the operator on the GPU: fused table passes against the oracle and the
torch ops, the FT module against the CPU path, and a short training run of the full model."""
import numpy as np
import pytest
import torch

import nnueft
from nnueft import _native
from nnueft import halfka_v2_hm as hk
from nnueft import model as M

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.mark.parametrize("R,cols,L1,vrows", [(3072, 40, 32, 768), (24576, 136, 128, 768), (300, 11, 6, 100)])
@pytest.mark.parametrize("quantize", [True, False])
def test_table_merge_and_virtual_grad(oracle_cpu, R, cols, L1, vrows, quantize):
    rng = np.random.default_rng(R + cols)
    W = (rng.standard_normal((R, cols)) * 0.1).astype(np.float32)
    V = (rng.standard_normal((vrows, cols)) * 0.1).astype(np.float32)
    g = rng.standard_normal((R, cols)).astype(np.float32)
    w = torch.from_numpy(W).to(DEV).requires_grad_()
    v = torch.from_numpy(V).to(DEV).requires_grad_()
    merged = M._table_merge(w, v, L1, 256.0, 9600.0, quantize)
    assert np.array_equal(merged.detach().cpu().numpy(), oracle_cpu.table_merge(W, V, L1, fake_quantize=quantize))
    merged.backward(torch.from_numpy(g).to(DEV))
    assert np.array_equal(w.grad.cpu().numpy(), g)                                   # straight-through
    assert np.array_equal(v.grad.cpu().numpy(), oracle_cpu.table_virtual_grad(g, vrows))
    # the torch ops of the reference give the same table
    t = torch.from_numpy(W) + torch.from_numpy(V).repeat(R // vrows, 1)
    if quantize:
        t = torch.cat([(t[:, :L1] * 256).round() / 256, (t[:, L1:] * 9600).round() / 9600], 1)
    assert torch.equal(merged.detach().cpu(), t)


@pytest.mark.parametrize("quantize", [True, False])
@pytest.mark.parametrize("act_on", [True, False])
@pytest.mark.parametrize("B,L1,lists", [(700, 512, "halfka"), (3000, 1024, "halfka"), (600, 544, "any")])
def test_forward_over_the_virtual_table_equals_merge_then_forward(B, L1, lists, quantize, act_on):
    """nnueft_double_fwd_virtual (real + virtual weights merged where the tile goes into LDS) against
    nnueft_table_merge followed by nnueft_double_fwd / nnueft_double_fwd_act, through the C ABI: the same
    bits in l0, the psqt outputs and the saved row sums.  "any": index lists that leave their table block
    (those lists are summed from global memory, merged there too)."""
    lib = _native.load()
    K, R, n_psqt, vrows = 32, hk.NUM_INPUTS, 8, 768
    oc = L1 + n_psqt
    rng = np.random.default_rng(B + L1)
    us, them, white, black, pc = hk.synthetic_batch(B, B + 1)
    if lists == "any":
        n = rng.integers(0, K + 1, size=(2, B))
        idx = rng.integers(0, R, size=(2, B, K)).astype(np.int32)
        idx[np.arange(K)[None, None, :] >= n[:, :, None]] = -1
        white, black = idx[0].copy(), idx[1].copy()
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(DEV)
    d_us, d_them, d_w, d_b, d_psqt = t(us), t(them), t(white), t(black), t(((pc - 1) // 4).astype(np.int64))
    W = t((rng.standard_normal((R, oc)) * 0.05).astype(np.float32))
    V = t((rng.standard_normal((vrows, oc)) * 0.05).astype(np.float32))
    bias = t((rng.standard_normal(oc) * 0.05).astype(np.float32))
    st = torch.cuda.current_stream().cuda_stream
    assert lib.nnueft_double_fwd_virtual_fits(B, K, R, L1, n_psqt, vrows) == 1
    assert lib.nnueft_double_fwd_virtual_fits(B, K, R, L1, n_psqt, 512) == 0
    assert lib.nnueft_double_fwd_virtual_fits(B, K, R, 128, n_psqt, vrows) == 0
    nbytes = lib.nnueft_fwd_workspace_bytes(B, K, R, L1, n_psqt)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=DEV)
    scale_ft, scale_psqt, act = 256.0, 9600.0, (127.0, 1e-5, 0.75)

    def outs():
        return [torch.full(s, float("nan"), device=DEV) for s in ((B, L1), (B, 1), (B, 1), (2, B, L1))]

    got = outs()
    _native.check(lib.nnueft_double_fwd_virtual(
        d_us.data_ptr(), d_them.data_ptr(), d_w.data_ptr(), d_b.data_ptr(), d_psqt.data_ptr(), W.data_ptr(),
        V.data_ptr(), bias.data_ptr(), 255.0 / 256.0, *[x.data_ptr() for x in got], B, K, R, L1, n_psqt, vrows,
        scale_ft, scale_psqt, int(quantize), ws.data_ptr(), nbytes, int(act_on), *act, st), "double_fwd_virtual")
    merged = torch.empty_like(W)
    _native.check(lib.nnueft_table_merge(W.data_ptr(), V.data_ptr(), merged.data_ptr(), R, oc, L1, vrows, scale_ft,
                                         scale_psqt, int(quantize), st), "table_merge")
    want = outs()
    head = (d_us.data_ptr(), d_them.data_ptr(), d_w.data_ptr(), d_b.data_ptr(), d_psqt.data_ptr(), merged.data_ptr(),
            bias.data_ptr(), 255.0 / 256.0, *[x.data_ptr() for x in want], B, K, R, L1, n_psqt, ws.data_ptr(), nbytes)
    if act_on:
        _native.check(lib.nnueft_double_fwd_act(*head, *act, st), "double_fwd_act")
    else:
        _native.check(lib.nnueft_double_fwd(*head, st), "double_fwd")
    torch.cuda.synchronize()
    for a, b in zip(got, want):
        assert not torch.isnan(a).any()
        assert torch.equal(a, b)
    # sizes the LDS-tiled gather does not take are refused, not run some other way
    rc = lib.nnueft_double_fwd_virtual(
        d_us.data_ptr(), d_them.data_ptr(), d_w.data_ptr(), d_b.data_ptr(), d_psqt.data_ptr(), W.data_ptr(),
        V.data_ptr(), bias.data_ptr(), 255.0 / 256.0, *[x.data_ptr() for x in got], B, K, R, L1, n_psqt, 512,
        scale_ft, scale_psqt, int(quantize), ws.data_ptr(), nbytes, int(act_on), *act, st)
    assert rc != 0


@pytest.mark.parametrize("fq_acts,fq_weights", [(True, True), (False, False)])
def test_ft_module_with_the_merge_folded_into_the_forward(fq_acts, fq_weights):
    """ComposedFeatureTransformer with the table merge inside the forward kernel against the same module with
    the separate merge pass: outputs and every gradient (weight, virtual weight, bias) bit for bit."""
    results = []
    B, L1 = 2048, 512
    batch = [torch.from_numpy(a).to(DEV) for a in hk.synthetic_batch(B, 16)]
    us, them, white, black, pc = batch
    psqt = (pc - 1) // 4
    gl = None
    old = M.FOLD_TABLE_MERGE
    try:
        for fold in (True, False):
            M.FOLD_TABLE_MERGE = fold
            model = _make_model(L1, 9).to(DEV)
            out = model.input(us, them, white, black, psqt, fq_acts, fq_weights)
            if gl is None:
                gl = [torch.randn_like(o) for o in out]
            torch.autograd.backward(list(out), gl)
            f = model.input.features[0]
            results.append([o.detach() for o in out] + [f.weight.grad, f.virtual_weight.grad, model.input.bias.grad])
    finally:
        M.FOLD_TABLE_MERGE = old
    for a, b in zip(*results):
        assert torch.equal(a, b)
    assert results[0][4].abs().sum() > 0


def _make_model(L1, seed):
    torch.manual_seed(seed)
    model = M.NNUEModel("HalfKAv2_hm^", M.ModelConfig(L1=L1, L2=16, L3=32))
    with torch.no_grad():
        model.input.features[0].virtual_weight.normal_(0, 0.005)
    return model


@pytest.mark.parametrize("mode", ["deterministic", "atomic"])
def test_ft_module_gpu_equals_cpu_path(mode):
    old = nnueft.get_backward_mode()
    nnueft.set_backward_mode(mode)
    try:
        cpu_model = _make_model(128, 5)
        gpu_model = _make_model(128, 5).to(DEV)
        B = 1024       # 32768 slots per list: the CPU backward then has the deterministic order
        batch = [torch.from_numpy(a) for a in hk.synthetic_batch(B, 6)]
        us, them, white, black, pc = batch
        psqt = (pc - 1) // 4
        out_c = cpu_model.input(us, them, white, black, psqt, True, True)
        out_g = gpu_model.input(*[t.to(DEV) for t in (us, them, white, black, psqt)], True, True)
        for a, b in zip(out_g, out_c):
            assert torch.equal(a.cpu(), b)
        gl = [torch.randn_like(t) for t in out_c]
        torch.autograd.backward(list(out_c), gl)
        torch.autograd.backward(list(out_g), [t.to(DEV) for t in gl])
        fc, fg = cpu_model.input.features[0], gpu_model.input.features[0]
        if mode == "deterministic":
            assert torch.equal(fg.weight.grad.cpu(), fc.weight.grad)
        else:
            torch.testing.assert_close(fg.weight.grad.cpu(), fc.weight.grad, atol=1e-4, rtol=1e-3)
        torch.testing.assert_close(fg.virtual_weight.grad.cpu(), fc.virtual_weight.grad, atol=1e-3, rtol=1e-3)
        torch.testing.assert_close(gpu_model.input.bias.grad.cpu(), cpu_model.input.bias.grad, atol=1e-3, rtol=1e-3)
    finally:
        nnueft.set_backward_mode(old)


def test_full_model_trains_on_gpu():
    """Config 4 in small: FT + layer stacks + loss + optimizer; the loss falls on a fixed batch and the
    GPU model agrees with the same weights evaluated through the CPU path."""
    model = _make_model(256, 7).to(DEV)
    B = 2048
    us, them, white, black, pc = [torch.from_numpy(a).to(DEV) for a in hk.synthetic_batch(B, 8)]
    g = torch.Generator().manual_seed(9)
    score = (torch.randn(B, 1, generator=g) * 400).clamp(-3000, 3000).to(DEV)
    outcome = (torch.randint(0, 3, (B, 1), generator=g).float() / 2).to(DEV)
    opt = torch.optim.Adam(model.parameters(), lr=1e-3)
    p = M.LossParams()
    losses = []
    for _ in range(12):
        opt.zero_grad(set_to_none=True)
        out = model(us, them, white, black, pc)
        loss = M.sf_loss(out * model.quantization.nnue2score, score, outcome, p, 0.75)
        loss.backward()
        for prm in model.parameters():
            assert prm.grad is not None and torch.isfinite(prm.grad).all()
        opt.step()
        losses.append(float(loss))
    assert all(np.isfinite(losses)) and losses[-1] < losses[0]
    cpu_model = _make_model(256, 7)
    cpu_model.load_state_dict({k: v.cpu() for k, v in model.state_dict().items()})
    with torch.no_grad():
        a = model(us, them, white, black, pc, False, False).cpu()
        b = cpu_model(us.cpu(), them.cpu(), white.cpu(), black.cpu(), pc.cpu(), False, False)
    torch.testing.assert_close(a, b, atol=2e-4, rtol=1e-3)


@pytest.mark.parametrize("backend", ["aot_eager", "cudagraphs"])
@pytest.mark.parametrize("L1,fq", [(1024, True), (1024, False), (128, True)])
def test_feature_transformer_module_compiles_as_one_graph(backend, L1, fq):
    """ComposedFeatureTransformer under torch.compile(fullgraph=True): everything it launches is a torch custom op
    with a shape function (the forward that merges real and virtual weights at L1 = 1024, the table merge pass and
    the plain operator at L1 = 128, the virtual-weight gradient, the bias grid), so dynamo finds no graph break, and
    with "cudagraphs" the HIP kernels sit inside the captured graph (no empty-graph warning).  Bits equal the
    eager run's on every call."""
    import warnings

    old = nnueft.get_backward_mode()
    nnueft.set_backward_mode("deterministic")
    try:
        model = _make_model(L1, 21).to(DEV)
        ft = model.input
        us, them, white, black, pc = [torch.from_numpy(a).to(DEV) for a in hk.synthetic_batch(700, 22)]
        psqt = (pc - 1) // 4
        up = [torch.randn(700, L1, device=DEV), torch.randn(700, 1, device=DEV), torch.randn(700, 1, device=DEV)]

        def run(fn):
            for p in ft.parameters():
                p.grad = None
            out = fn(us, them, white, black, psqt, fq, fq)
            torch.autograd.backward(list(out), up)
            return [o.detach().clone() for o in out], {n: p.grad.clone() for n, p in ft.named_parameters()}

        ref_out, ref_grad = run(ft)
        assert all(g.abs().max() > 0 for g in ref_grad.values())
        torch._dynamo.reset()
        cm = torch.compile(ft, backend=backend, fullgraph=True)
        with warnings.catch_warnings(record=True) as seen:
            warnings.simplefilter("always")
            for _ in range(4):
                out, grad = run(cm)
                for a, b in zip(out, ref_out):
                    assert torch.equal(a, b)
                for n in ref_grad:
                    assert torch.equal(grad[n], ref_grad[n]), n
        assert not [w for w in seen if "CUDA Graph is empty" in str(w.message)]
    finally:
        nnueft.set_backward_mode(old)
        torch._dynamo.reset()


@pytest.mark.parametrize("whole_model", [True, False], ids=["model", "modules"])
@pytest.mark.parametrize("backend", ["aot_eager", "inductor"])
def test_model_under_torch_compile_on_gpu(backend, whole_model):
    """The reference compiles the model (train.py:296).  whole_model: torch.compile(model) leaves
    NNUEModel.forward as it is (it is marked not to be traced).  Otherwise a function over the feature
    transformer and the layer stacks is compiled: the feature transformer's launches are custom ops and stay in
    the graph, the layer stacks' launchers are opaque to dynamo (torch.compiler.disable) and break the graph
    around them.  Either way the results are the eager ones, deterministic backward included.  ("cudagraphs" is
    exercised where something is captured: on the operator and on the feature transformer module, see
    test_feature_transformer_module_compiles_as_one_graph; over the layer stacks it would capture the empty
    stretches between their launchers.)"""
    old = nnueft.get_backward_mode()
    nnueft.set_backward_mode("deterministic")
    try:
        model = _make_model(128, 11).to(DEV)
        batch = [torch.from_numpy(a).to(DEV) for a in hk.synthetic_batch(512, 12)]
        out = model(*batch)
        out.sum().backward()
        ref = {n: p.grad.clone() for n, p in model.named_parameters()}
        model.zero_grad()
        torch._dynamo.reset()

        def modules(us, them, white, black, piece_count):
            psqt, ls = model.calculate_buckets(piece_count)
            l0, wp, bp = model.input(us, them, white, black, psqt, True, True)
            return model.layer_stacks(l0, ls, True, True) + (wp - bp) * (us - 0.5)

        cm = torch.compile(model if whole_model else modules, backend=backend)
        for _ in range(2):      # the second call runs the cached graph
            model.zero_grad()
            o = cm(*batch)
            o.sum().backward()
            torch.testing.assert_close(o, out, atol=1e-5, rtol=1e-5)
            if whole_model or backend == "aot_eager":   # same kernels upstream, so the same bits
                assert torch.equal(model.input.features[0].weight.grad, ref["input.features.0.weight"])
            for n, p in model.named_parameters():
                torch.testing.assert_close(p.grad, ref[n], atol=1e-4, rtol=1e-4)
    finally:
        nnueft.set_backward_mode(old)
        torch._dynamo.reset()


@pytest.mark.parametrize("n,post_mul", [(1, 1.0), (7, 0.5), (4096 * 33 + 3, 1.0), (16384 * 3072 // 8, 1.3)])
def test_act_fake_quantize_kernel(oracle_cpu, n, post_mul):
    from nnueft.model import _ActFakeQuantize

    g = torch.Generator().manual_seed(n)
    x = (torch.rand(n, generator=g) * 1.2 - 0.1).to(DEV).requires_grad_()
    out = _ActFakeQuantize.apply(x, 128.0, post_mul)
    ref = oracle_cpu.act_fake_quantize(x.detach().cpu().numpy(), 128.0, M.FAKE_QUANTIZE_EPS, post_mul)
    assert np.array_equal(out.detach().cpu().numpy(), ref)
    up = torch.randn(n, generator=g).to(DEV)
    out.backward(up)
    assert torch.equal(x.grad, up * post_mul)


@pytest.mark.parametrize("B,n_in,out,count", [(1, 32, 1, 1), (37, 64, 16, 8), (300, 128, 32, 8), (1000, 3072, 32, 8),
                                              (4097, 1024, 16, 8), (513, 96, 7, 3), (64, 256, 32, 64),
                                              (20000, 32, 4, 8), (5000, 32, 2, 40), (16384, 64, 3, 32)])
def test_bucket_linear_kernels(oracle_cpu, B, n_in, out, count):
    from nnueft import _native

    lib = _native.load()
    rng = np.random.default_rng(B + n_in)
    x = rng.standard_normal((B, n_in)).astype(np.float32)
    W = (rng.standard_normal((count * out, n_in)) / np.sqrt(n_in)).astype(np.float32)
    bias = rng.standard_normal(count * out).astype(np.float32)
    bucket = rng.integers(0, count, size=B).astype(np.int64)
    if count > 2:
        bucket[bucket == 1] = 0          # one bucket nobody uses: its gradient blocks must come out zero
    gy = rng.standard_normal((B, out)).astype(np.float32)
    t = lambda a: torch.from_numpy(a).to(DEV)
    dx, dW, db, dk, dgy = t(x), t(W), t(bias), t(bucket), t(gy)
    nbytes = lib.nnueft_bucket_linear_workspace_bytes(B, count)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=DEV)
    stream = torch.cuda.current_stream().cuda_stream
    y = torch.full((B, out), float("nan"), device=DEV)
    _native.check(lib.nnueft_bucket_linear_fwd(dx.data_ptr(), dk.data_ptr(), dW.data_ptr(), db.data_ptr(), y.data_ptr(),
                                               B, n_in, out, count, ws.data_ptr(), nbytes, 0, stream), "fwd")
    ref = oracle_cpu.bucket_linear_fwd(x, bucket, W, bias, out, count)
    tol = lambda r: 1e-5 * max(float(np.abs(r).max()), 1e-30)
    assert np.abs(y.cpu().numpy() - ref).max() <= tol(ref)
    gx = torch.full((B, n_in), float("nan"), device=DEV)
    gW = torch.full((count * out, n_in), float("nan"), device=DEV)
    gb = torch.full((count * out,), float("nan"), device=DEV)
    _native.check(lib.nnueft_bucket_linear_bwd(dx.data_ptr(), dk.data_ptr(), dW.data_ptr(), dgy.data_ptr(),
                                               gx.data_ptr(), gW.data_ptr(), gb.data_ptr(), B, n_in, out, count,
                                               ws.data_ptr(), nbytes, 1, stream), "bwd")   # grouping left by the forward call
    rx, rW, rb = oracle_cpu.bucket_linear_bwd(x, bucket, W, gy, out, count)
    assert np.abs(gx.cpu().numpy() - rx).max() <= tol(rx)
    assert np.abs(gW.cpu().numpy() - rW).max() <= tol(rW)
    assert np.abs(gb.cpu().numpy() - rb).max() <= tol(rb)
    if count > 2:
        assert not gW.cpu().numpy()[out:2 * out].any() and not gb.cpu().numpy()[out:2 * out].any()
    # twice the same bits
    gW2 = torch.empty_like(gW)
    ws.zero_()
    _native.check(lib.nnueft_bucket_linear_group(dk.data_ptr(), B, count, ws.data_ptr(), nbytes, stream), "group")
    y2 = torch.empty_like(y)
    _native.check(lib.nnueft_bucket_linear_fwd(dx.data_ptr(), dk.data_ptr(), dW.data_ptr(), db.data_ptr(), y2.data_ptr(),
                                               B, n_in, out, count, ws.data_ptr(), nbytes, 1, stream), "fwd")
    assert torch.equal(y, y2)
    ws.zero_()                                   # regrouped inside the next call
    _native.check(lib.nnueft_bucket_linear_bwd(dx.data_ptr(), dk.data_ptr(), dW.data_ptr(), dgy.data_ptr(), None,
                                               gW2.data_ptr(), gb.data_ptr(), B, n_in, out, count, ws.data_ptr(),
                                               nbytes, 0, stream), "bwd")
    assert torch.equal(gW, gW2)


def test_stacked_linear_on_gpu_equals_the_wide_layer():
    torch.manual_seed(3)
    q = M.QuantizationManager(M.QuantizationConfig())
    layer = M.FactorizedStackedLinear(512, 16, 8, q, "ls_l1")
    with torch.no_grad():
        layer.factorized_linear.weight.normal_(0, 0.02)
    gpu = M.FactorizedStackedLinear(512, 16, 8, q, "ls_l1").to(DEV)
    gpu.load_state_dict(layer.state_dict())
    x = torch.rand(700, 512)
    idx = torch.randint(0, 8, (700,))
    for fq in (False, True):
        layer.zero_grad()
        gpu.zero_grad()
        xc = x.clone().requires_grad_()
        xg = x.to(DEV).requires_grad_()
        yc = layer(xc, idx, fq)
        yg = gpu(xg, idx.to(DEV), fq)
        torch.testing.assert_close(yg.cpu(), yc, rtol=1e-4, atol=1e-5)
        up = torch.randn_like(yc)
        yc.backward(up)
        yg.backward(up.to(DEV))
        torch.testing.assert_close(xg.grad.cpu(), xc.grad, rtol=1e-4, atol=1e-5)
        for (n, a), (_, b) in zip(layer.named_parameters(), gpu.named_parameters()):
            torch.testing.assert_close(b.grad.cpu(), a.grad, rtol=1e-4, atol=2e-5, msg=n)
    # the one-pass weight preparation gives the bits of the torch ops it replaces
    for fq in (False, True):
        w1, b1 = gpu._params_one_pass(fq)
        w0, b0 = gpu._params()
        if fq:
            w0, b0 = q.fake_quantize_weights(w0, "ls_l1_weight"), q.fake_quantize_weights(b0, "ls_l1_bias")
        assert torch.equal(w1, w0) and torch.equal(b1, b0)
    plain = M.StackedLinear(64, 32, 8, q, "ls_l2").to(DEV)
    w1, b1 = plain._params_one_pass(True)
    assert torch.equal(w1, q.fake_quantize_weights(plain.linear.weight, "ls_l2_weight"))
    assert torch.equal(b1, q.fake_quantize_weights(plain.linear.bias, "ls_l2_bias"))
    w1, b1 = plain._params_one_pass(False)
    assert w1 is plain.linear.weight and b1 is plain.linear.bias


def _tail_inputs(B, n, seed):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(B, n, generator=g) * 0.7
    # values on and next to the quantization grid and the clamp bounds
    edge = torch.tensor([0.0, 1.0, -1.0, 1.0 / 127, 126.5 / 127, 127.0 / 127, 2.0, -0.0039])[: B * n]
    x.view(-1)[: edge.numel()] = edge
    return x


@pytest.mark.parametrize("B,n", [(1, 2), (33, 16), (4097, 32)])
@pytest.mark.parametrize("fq", [True, False])
def test_sqr_crelu_kernel_equals_the_torch_ops(B, n, fq):
    """One kernel against the chain of torch ops it replaces (LayerStacks._sqr_and_linear on the CPU,
    autograd for the gradient): same bits forward; the gradient to one rounding."""
    q = M.QuantizationManager(M.QuantizationConfig())
    ls = M.LayerStacks(8, M.ModelConfig(L1=64, L2=n, L3=32), q)
    x = _tail_inputs(B, n, 5 + B)
    xc = x.clone().requires_grad_()
    yc, sc = ls._sqr_crelu(xc, fq, want_skip=True)
    xg = x.to(DEV).requires_grad_()
    yg, sg = ls._sqr_crelu(xg, fq, want_skip=True)
    assert torch.equal(yg.cpu(), yc) and torch.equal(sg.cpu(), sc)
    g = torch.Generator().manual_seed(9)
    gy, gs = torch.randn(B, 2 * n, generator=g), torch.randn(B, 1, generator=g)
    torch.autograd.backward([yc, sc], [gy, gs])
    torch.autograd.backward([yg, sg], [gy.to(DEV), gs.to(DEV)])
    torch.testing.assert_close(xg.grad.cpu(), xc.grad, rtol=1e-6, atol=1e-7)
    # without the skip value
    xg2 = x.to(DEV).requires_grad_()
    y2, none = ls._sqr_crelu(xg2, fq)
    assert none is None and torch.equal(y2, yg)
    y2.backward(gy.to(DEV))
    xc2 = x.clone().requires_grad_()
    ls._sqr_and_linear(xc2, fq).backward(gy)
    torch.testing.assert_close(xg2.grad.cpu(), xc2.grad, rtol=1e-6, atol=1e-7)


@pytest.mark.parametrize("fq", [True, False])
def test_stack_output_kernel_equals_the_torch_ops(fq):
    q = M.QuantizationManager(M.QuantizationConfig())
    B = 5000
    g = torch.Generator().manual_seed(4)
    lin, skip = torch.randn(B, 1, generator=g) * 0.5, torch.randn(B, 1, generator=g) * 0.2
    wp, bp = torch.randn(B, 1, generator=g) * 0.3, torch.randn(B, 1, generator=g) * 0.3
    us = torch.randint(0, 2, (B, 1), generator=g).float()
    cpu = [t.clone().requires_grad_() for t in (lin, skip, wp, bp)]
    v = cpu[0] + cpu[1]
    if fq:
        v = q.fake_quantize_output(v)
    want = v + (cpu[2] - cpu[3]) * (us - 0.5)
    gpu = [t.to(DEV).requires_grad_() for t in (lin, skip, wp, bp)]
    den, mult = q.output_quantization()
    got = M._StackOutput.apply(*gpu, us.to(DEV), den, mult, fq)
    assert torch.equal(got.cpu(), want)
    up = torch.randn(B, 1, generator=g)
    want.backward(up)
    got.backward(up.to(DEV))
    for a, b in zip(gpu, cpu):
        assert torch.equal(a.grad.cpu(), b.grad)


@pytest.mark.parametrize("params,lam", [(M.LossParams(), 0.75), (M.LossParams(qp_asymmetry=0.3, w1=1.0), 1.0),
                                         (M.LossParams(pow_exp=2.0, w1=0.5, w2=0.25), 0.3)])
@pytest.mark.parametrize("B", [1, 1000, 16384])
def test_sf_loss_kernels_against_the_torch_formula(params, lam, B):
    """The fused loss against sf_loss written in torch ops, evaluated in float64 on the CPU with autograd
    for the gradient.  Tolerance: 1e-5 relative for the loss; for the gradient 1e-4 of the largest entry,
    2e-3 with position weights (w1 != 0): they depend on 1 - pf, which float32 holds to about 1e-2
    relative for a tablebase score, whoever evaluates it."""
    g = torch.Generator().manual_seed(B)
    net = (torch.randn(B, 1, generator=g) * 400)
    score = (torch.randn(B, 1, generator=g) * 600).clamp(-3000, 3000)
    score.view(-1)[: min(B, 4)] = torch.tensor([31990.0, -31800.0, 31755.0, -32000.0])[: min(B, 4)]   # tablebase scores
    outcome = torch.randint(0, 3, (B, 1), generator=g).float() / 2
    x64 = net.double().requires_grad_()
    want = M.sf_loss(x64, score.double(), outcome.double(), params, lam)
    want.backward()
    xg = net.to(DEV).requires_grad_()
    got = M.sf_loss(xg, score.to(DEV), outcome.to(DEV), params, lam)
    assert got.shape == () and got.dtype == torch.float32
    got.backward()
    assert abs(got.item() - want.item()) <= 1e-5 * abs(want.item())
    scale = x64.grad.abs().max().item()
    tol = 2e-3 if params.w1 != 0.0 else 1e-4
    assert (xg.grad.cpu().double() - x64.grad).abs().max().item() <= tol * scale
    # twice the same bits
    again = M.sf_loss(net.to(DEV), score.to(DEV), outcome.to(DEV), params, lam)
    assert torch.equal(again, got.detach())


def test_synthetic_training_loop_on_gpu():
    """Host batches in the loader's layout, the prefetcher's stream, the model, the fused loss and RangerLite
    together: the loss falls, and a second run from the same seed gives the same losses bit for bit
    (deterministic backward, fixed-order loss sums, no atomics anywhere in the step)."""
    from nnueft import train_synthetic

    old = nnueft.get_backward_mode()
    nnueft.set_backward_mode("deterministic")
    try:
        a, rate = train_synthetic.run(steps=30, batch_size=4096, l1=256, device=DEV, lr=2e-3)
        b, _ = train_synthetic.run(steps=30, batch_size=4096, l1=256, device=DEV, lr=2e-3)
    finally:
        nnueft.set_backward_mode(old)
    assert all(np.isfinite(a)) and a[-1] < a[0] and rate > 0
    assert a == b


@pytest.mark.parametrize("L2", [32, 16], ids=["L2_32", "L2_15plus1"])
def test_config_4_full_size_step(oracle_cpu, L2):
    """BASELINE.json config 4 at its real size: L1=3072 feature transformer, 8 bucketed layer stacks
    (3072 -> L2 -> 32 -> 1; L2=32 is the reference's default, 16 = 15+1 the configuration's literal), B=16384,
    RangerLite.  (a) the feature transformer of the first step, outputs and gradients, bit-equal to the oracle on
    the same merged table; (b) the bucketed first layer at in=3072, B=16384 against the oracle, 1e-5 of the largest
    magnitude; (c) three optimizer steps, losses finite and identical on a second run from the same seed."""
    from nnueft.optim import RangerLite

    old = nnueft.get_backward_mode()
    nnueft.set_backward_mode("deterministic")
    L1, B, R, n_psqt = 3072, 16384, hk.NUM_INPUTS, 8
    host = hk.synthetic_batch(B, 1238)
    us, them, white, black, pc = [torch.from_numpy(a).to(DEV) for a in host]
    psqt_np = ((host[4] - 1) // 4).astype(np.int64)
    g = torch.Generator().manual_seed(1238)
    score = (torch.randn(B, 1, generator=g) * 400).clamp(-3000, 3000).to(DEV)
    outcome = (torch.randint(0, 3, (B, 1), generator=g).float() / 2).to(DEV)

    def fresh():
        torch.manual_seed(0)
        m = M.NNUEModel("HalfKAv2_hm^", M.ModelConfig(L1=L1, L2=L2, L3=32)).to(DEV)
        with torch.no_grad():      # shared weights off zero, so that the merge has something to add
            m.input.features[0].virtual_weight.normal_(0, 0.003)
            m.input.features[0].weight[:, :L1].normal_(0, 0.01)
            m.input.bias[:L1].normal_(0, 0.01)
        return m

    try:
        model = fresh()
        q = model.quantization
        # (a) the feature transformer of step 1
        merged, bias = model.input.merged_weight_and_bias(True)
        l0, wp, bp = model.input(us, them, white, black, (pc - 1) // 4, True, True)
        Wn, bn = merged.detach().cpu().numpy(), bias.detach().cpu().numpy()
        feat = model.input.features[0]
        assert np.array_equal(Wn, oracle_cpu.table_merge(feat.weight.detach().cpu().numpy(),
                                                         feat.virtual_weight.detach().cpu().numpy(), L1))
        r_l0, r_wp, r_bp, r_saved = oracle_cpu.double_fwd(host[0], host[1], host[2], host[3], psqt_np, Wn, bn,
                                                          q.max_ft_activation, L1)
        r_l0 = oracle_cpu.act_fake_quantize(r_l0, q.hidden_quantized_one, M.FAKE_QUANTIZE_EPS, q.l0_correction_factor)
        assert np.array_equal(l0.detach().cpu().numpy(), r_l0)
        assert np.array_equal(wp.detach().cpu().numpy(), r_wp) and np.array_equal(bp.detach().cpu().numpy(), r_bp)
        up = [torch.randn(B, L1, generator=g), torch.randn(B, 1, generator=g), torch.randn(B, 1, generator=g)]
        torch.autograd.backward([l0, wp, bp], [t.to(DEV) for t in up])
        r_gW, r_gb = oracle_cpu.double_bwd(host[0], host[1], host[2], host[3], psqt_np, bn, q.max_ft_activation,
                                           up[0].numpy() * np.float32(q.l0_correction_factor), up[1].numpy(),
                                           up[2].numpy(), r_saved, R, n_psqt)
        assert np.array_equal(feat.weight.grad.cpu().numpy(), r_gW)                     # straight-through
        assert np.array_equal(feat.virtual_weight.grad.cpu().numpy(), oracle_cpu.table_virtual_grad(r_gW, 768))
        assert np.array_equal(model.input.bias.grad.cpu().numpy()[:L1], r_gb[:L1])
        del merged, l0, wp, bp, r_gW, r_saved, Wn
        model.zero_grad(set_to_none=True)

        # (b) the first bucketed layer on this model's own activations
        ls = model.layer_stacks
        with torch.no_grad():
            x = model.input(us, them, white, black, (pc - 1) // 4, True, True)[0]
        bucket = (pc - 1) // 4
        w, b_ = ls.l1._params_one_pass(True)
        out_f = ls.l1.linear.out_features // 8
        xg = x.clone().requires_grad_()
        wg = w.detach().clone().requires_grad_()
        bg = b_.detach().clone().requires_grad_()
        y = M._BucketLinear.apply(xg, bucket, wg, bg, out_f, 8, None)
        gy = torch.randn(B, out_f, generator=g)
        y.backward(gy.to(DEV))
        xn, wn, bucket_n = x.cpu().numpy(), wg.detach().cpu().numpy(), bucket.cpu().numpy()
        ref = oracle_cpu.bucket_linear_fwd(xn, bucket_n, wn, bg.detach().cpu().numpy(), out_f, 8)
        tol = lambda r: 1e-5 * max(float(np.abs(r).max()), 1e-30)
        assert np.abs(y.detach().cpu().numpy() - ref).max() <= tol(ref)
        rx, rW, rb = oracle_cpu.bucket_linear_bwd(xn, bucket_n, wn, gy.numpy(), out_f, 8)
        assert np.abs(xg.grad.cpu().numpy() - rx).max() <= tol(rx)
        assert np.abs(wg.grad.cpu().numpy() - rW).max() <= tol(rW)
        assert np.abs(bg.grad.cpu().numpy() - rb).max() <= tol(rb)
        del x, xg, y, rx, rW, xn

        # (c) three steps, twice
        def run(model):
            opt = RangerLite(M.optimizer_param_groups(model, lr=8.75e-4), normloss_active=False)
            losses = []
            for _ in range(3):
                opt.zero_grad(set_to_none=True)
                out = model(us, them, white, black, pc)
                loss = M.sf_loss(out * model.quantization.nnue2score, score, outcome, M.LossParams(), 0.75)
                loss.backward()
                for name, prm in model.named_parameters():
                    assert prm.grad is not None, name
                opt.step()
                model.clip_weights(include_input=False)
                losses.append(float(loss))
            for name, prm in model.named_parameters():
                assert torch.isfinite(prm).all(), name
            return losses

        a = run(model)
        del model
        torch.cuda.empty_cache()
        b = run(fresh())
        assert all(np.isfinite(a)) and a == b
    finally:
        nnueft.set_backward_mode(old)
