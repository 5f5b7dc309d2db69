"""The Python mirror of the reference interface on the GPU: the reference's own tests restated
(same shapes, seeds and tolerances), the BASELINE configurations at full size against the oracle,
edge cases (empty batch, one hot row, non-default stream) and the error paths of the C ABI."""
import numpy as np
import pytest
import torch

import nnueft
from _cases import double_case, random_lists, sparse_case
from nnueft import _native
from nnueft import halfka_v2_hm as hk
from nnueft.double_ft_functions import double_feature_transform
from nnueft.sparse_linear_functions import SparseLinearFunction
from oracle import ref_torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(autouse=True)
def _restore_mode():
    old, old_sort = nnueft.get_backward_mode(), nnueft.get_sort_placement()
    yield
    nnueft.set_backward_mode(old)
    nnueft.set_sort_placement(old_sort)


def _emulate(indices, weight, bias):
    # tests/test_feature_transformer.py:14-32
    dense = torch.zeros(indices.shape[0], weight.shape[0], dtype=torch.float32)
    for i in range(indices.shape[0]):
        for j in range(indices.shape[1]):
            if indices[i, j] >= 0:
                dense[i, indices[i, j]] += 1.0
    return torch.mm(dense, weight) + bias


@pytest.mark.parametrize("mode", ["atomic", "deterministic"])
def test_reference_sparse_linear_test_on_gpu(mode):
    # tests/test_feature_transformer.py:35-78 with device = cuda
    nnueft.set_backward_mode(mode)
    torch.manual_seed(0)
    weight0 = torch.rand(10, 128, requires_grad=True)
    bias0 = torch.rand(128, requires_grad=True)
    torch.manual_seed(0)
    weight1 = torch.rand(10, 128, requires_grad=True)
    bias1 = torch.rand(128, requires_grad=True)
    indices0 = (torch.rand(16, 32) * 10).to(dtype=torch.int32)
    indices1 = (torch.rand(16, 32) * 10).to(dtype=torch.int32)
    out00 = _emulate(indices0, weight0, bias0)
    out01 = _emulate(indices1, weight0, bias0)
    out10 = SparseLinearFunction.apply(indices0.to(DEV), weight1.to(DEV), bias1.to(DEV))
    out11 = SparseLinearFunction.apply(indices1.to(DEV), weight1.to(DEV), bias1.to(DEV))
    assert torch.max(torch.abs(out00 - out10.cpu())) < 1e-4
    assert torch.max(torch.abs(out01 - out11.cpu())) < 1e-4
    (out00 - out01).sum().backward()
    (out10 - out11).sum().backward()
    assert torch.max(torch.abs(weight0.grad - weight1.grad)) < 1e-4
    assert torch.max(torch.abs(bias0.grad - bias1.grad)) < 1e-4


def test_reference_padding_test_on_gpu():
    # tests/test_feature_transformer.py:81-110
    torch.manual_seed(42)
    weight = torch.rand(10, 64, device=DEV)
    bias = torch.rand(64, device=DEV)
    active = (torch.rand(8, 5) * 10).to(dtype=torch.int32, device=DEV)
    padded = torch.cat([active, torch.full((8, 3), -1, dtype=torch.int32, device=DEV)], dim=1)
    a = SparseLinearFunction.apply(active, weight, bias)
    b = SparseLinearFunction.apply(padded, weight, bias)
    assert torch.max(torch.abs(a - b)) < 1e-4
    assert torch.equal(a, b)


@pytest.mark.parametrize("mode", ["atomic", "deterministic"])
@pytest.mark.parametrize("l1", [32, 2048])
def test_reference_fused_vs_torch_test(l1, mode):
    # tests/test_fused_double_ft.py:19-107
    nnueft.set_backward_mode(mode)
    torch.manual_seed(0)
    torch.cuda.manual_seed_all(0)
    batch_size, max_active, num_inputs, num_psqt = 4, 32, 100, 8
    output_size = l1 + num_psqt
    us = torch.randn(batch_size, 1, device=DEV)
    them = torch.randn(batch_size, 1, device=DEV)
    white = torch.randint(0, num_inputs, (batch_size, max_active), dtype=torch.int32, device=DEV)
    white[:, -2:] = -1
    black = torch.randint(0, num_inputs, (batch_size, max_active), dtype=torch.int32, device=DEV)
    black[:, -2:] = -1
    psqt = torch.randint(0, num_psqt, (batch_size,), dtype=torch.int64, device=DEV)
    weight = torch.randn(num_inputs, output_size, device=DEV, requires_grad=True)
    bias = torch.randn(output_size, device=DEV, requires_grad=True)

    l0_f, wp_f, bp_f = double_feature_transform(us, them, white, black, psqt, weight, bias, 127.0, l1, "fused")
    (l0_f.sum() + wp_f.sum() + bp_f.sum()).backward()
    gw_f, gb_f = weight.grad.clone(), bias.grad.clone()
    weight.grad.zero_()
    bias.grad.zero_()
    l0_t, wp_t, bp_t = double_feature_transform(us, them, white, black, psqt, weight, bias, 127.0, l1, "torch")
    (l0_t.sum() + wp_t.sum() + bp_t.sum()).backward()
    torch.testing.assert_close(l0_f, l0_t, atol=1e-5, rtol=1e-4)
    torch.testing.assert_close(wp_f, wp_t, atol=1e-5, rtol=1e-4)
    torch.testing.assert_close(bp_f, bp_t, atol=1e-5, rtol=1e-4)
    torch.testing.assert_close(gw_f, weight.grad, atol=1e-4, rtol=1e-3)
    torch.testing.assert_close(gb_f, bias.grad, atol=1e-4, rtol=1e-3)
    # the "sparse" backend (two sparse-linear launches + torch ops) agrees as well
    weight.grad.zero_()
    bias.grad.zero_()
    l0_s, wp_s, bp_s = double_feature_transform(us, them, white, black, psqt, weight, bias, 127.0, l1, "sparse")
    (l0_s.sum() + wp_s.sum() + bp_s.sum()).backward()
    torch.testing.assert_close(l0_s, l0_t, atol=1e-5, rtol=1e-4)
    torch.testing.assert_close(weight.grad, gw_f, atol=1e-4, rtol=1e-3)


def test_deterministic_backward_bits_equal_the_reference_cpu_path():
    """GPU deterministic mode vs torch CPU autograd of the reference composition, equality of bits
    (32768 slots per list: torch's CPU backward then accumulates in ascending position order)."""
    nnueft.set_backward_mode("deterministic")
    c = double_case(31, 1024, 128, hk.NUM_INPUTS, halfka=True, max_act=255 / 256, weight_scale=0.05)
    cpu = {k: torch.from_numpy(c[k]) for k in ("us", "them", "widx", "bidx", "psqt_idx", "W", "bias")}
    Wc = cpu["W"].clone().requires_grad_()
    bc = cpu["bias"].clone().requires_grad_()
    out_c = ref_torch.double_feature_transform(cpu["us"], cpu["them"], cpu["widx"], cpu["bidx"], cpu["psqt_idx"],
                                               Wc, bc, c["max_act"], 128)
    grads = [torch.from_numpy(c[k]) for k in ("g_l0", "g_wp", "g_bp")]
    torch.autograd.backward(list(out_c), grads)
    Wg = cpu["W"].to(DEV).requires_grad_()
    bg = cpu["bias"].to(DEV).requires_grad_()
    out_g = double_feature_transform(cpu["us"].to(DEV), cpu["them"].to(DEV), cpu["widx"].to(DEV), cpu["bidx"].to(DEV),
                                     cpu["psqt_idx"].to(DEV), Wg, bg, c["max_act"], 128, "fused")
    torch.autograd.backward(list(out_g), [g.to(DEV) for g in grads])
    for a, b in zip(out_g, out_c):
        assert torch.equal(a.cpu(), b)
    assert torch.equal(Wg.grad.cpu(), Wc.grad)
    torch.testing.assert_close(bg.grad.cpu(), bc.grad, atol=1e-4, rtol=1e-4)


def _strict_vs_reference_cpu_path(L1, B, seed, **batch_kw):
    """Forward and strict-order deterministic backward on the GPU against torch CPU autograd of the
    reference's composition (oracle/ref_torch.py) on the same inputs; returns the two weight gradients."""
    n_psqt, R = 8, hk.NUM_INPUTS
    assert B * 32 >= 32768        # from this many slots per list on, torch's CPU backward adds in (position, slot) order
    us, them, white, black, pc = hk.synthetic_batch(B, seed, **batch_kw)
    g = torch.Generator().manual_seed(seed)
    cpu = [torch.from_numpy(a) for a in (us, them, white, black, (pc - 1) // 4)]
    W0 = torch.randn(R, L1 + n_psqt, generator=g) * 0.01
    b0 = torch.randn(L1 + n_psqt, generator=g) * 0.01
    grads = [torch.randn(B, L1, generator=g), torch.randn(B, 1, generator=g), torch.randn(B, 1, generator=g)]
    max_act = 255.0 / 256.0
    Wc, bc = W0.clone().requires_grad_(), b0.clone().requires_grad_()
    out_c = ref_torch.double_feature_transform(*cpu, Wc, bc, max_act, L1)
    torch.autograd.backward(list(out_c), grads)
    nnueft.set_backward_mode("deterministic_strict")
    Wg, bg = W0.to(DEV).requires_grad_(), b0.to(DEV).requires_grad_()
    out_g = double_feature_transform(*[a.to(DEV) for a in cpu], Wg, bg, max_act, L1, "fused")
    torch.autograd.backward(list(out_g), [x.to(DEV) for x in grads])
    for a, b in zip(out_g, out_c):
        assert torch.equal(a.detach().cpu(), b.detach())
    torch.testing.assert_close(bg.grad.cpu(), bc.grad, atol=1e-4, rtol=1e-4)
    counts = np.bincount(np.concatenate([white[white >= 0], black[black >= 0]]), minlength=R)
    return Wg.grad.cpu(), Wc.grad, counts


def test_strict_deterministic_backward_bits_equal_the_reference_cpu_path_at_config_1():
    """BASELINE.json config 1 at full size (L1=1024, B=8192; 262144 slots per list): the strict mode's weight
    gradient is torch CPU autograd's, bit for bit, rows named by more than nnueft_row_split() slots included."""
    g_gpu, g_cpu, counts = _strict_vs_reference_cpu_path(1024, 8192, 1235)
    assert (counts > _native.load().nnueft_row_split()).sum() >= 1       # rows the default mode would split
    assert torch.equal(g_gpu, g_cpu)


def test_strict_deterministic_backward_bits_equal_the_reference_cpu_path_on_game_like_lists():
    """The same on lists with the bucket statistics of game positions: a few hundred table rows are named by
    thousands of slots each."""
    g_gpu, g_cpu, counts = _strict_vs_reference_cpu_path(256, 8192, 1236, game_like=True)
    split = counts > _native.load().nnueft_row_split()
    assert split.sum() >= 30 and counts.max() > 2000
    assert torch.equal(g_gpu, g_cpu)
    # the default mode on the same inputs: the same bits on the rows it leaves whole, rounding apart on the others
    nnueft.set_backward_mode("deterministic")
    us, them, white, black, pc = hk.synthetic_batch(8192, 1236, game_like=True)
    g = torch.Generator().manual_seed(1236)
    W0 = torch.randn(hk.NUM_INPUTS, 264, generator=g) * 0.01
    b0 = torch.randn(264, generator=g) * 0.01
    grads = [torch.randn(8192, 256, generator=g), torch.randn(8192, 1, generator=g), torch.randn(8192, 1, generator=g)]
    Wg, bg = W0.to(DEV).requires_grad_(), b0.to(DEV).requires_grad_()
    t = lambda a: torch.from_numpy(a).to(DEV)
    out = double_feature_transform(t(us), t(them), t(white), t(black), t((pc - 1) // 4), Wg, bg, 255.0 / 256.0, 256,
                                   "fused")
    torch.autograd.backward(list(out), [x.to(DEV) for x in grads])
    windowed = Wg.grad.cpu()
    whole = torch.from_numpy(~split)
    assert torch.equal(windowed[whole], g_cpu[whole])
    torch.testing.assert_close(windowed, g_cpu, atol=1e-4, rtol=1e-3)


def test_backward_modes_agree_on_game_like_lists_at_the_metric_size():
    """L1=3072, B=16384 with the bucket statistics of game positions (the crowded table blocks hold thousands of pairs:
    several chunks of lists a block for the LDS tiles, hundreds of split rows for the reduction): the windowed order
    against the strict one (same bits on the rows it leaves whole, rounding apart on the others) and the atomic adds
    in LDS tiles against the strict order to the atomic bar; the strict order is pinned against torch CPU autograd
    and the oracle by the tests above."""
    L1, B, n_psqt, R = 3072, 16384, 8, hk.NUM_INPUTS
    us, them, white, black, pc = hk.synthetic_batch(B, 1240, game_like=True)
    counts = np.bincount(np.concatenate([white[white >= 0], black[black >= 0]]), minlength=R)
    assert (counts > 512).sum() > 100 and counts.max() > 4000
    block_pairs = np.bincount(np.concatenate([white[:, 0], black[:, 0]]) // 768, minlength=32)
    assert block_pairs.max() > 2 * 1536      # more pairs in a block than two chunks of lists hold
    g = torch.Generator().manual_seed(1240)
    W0 = (torch.randn(R, L1 + n_psqt, generator=g) * 0.01).to(DEV)
    b0 = (torch.randn(L1 + n_psqt, generator=g) * 0.01).to(DEV)
    grads = [torch.randn(B, L1, generator=g).to(DEV), torch.randn(B, 1, generator=g).to(DEV),
             torch.randn(B, 1, generator=g).to(DEV)]
    t = lambda a: torch.from_numpy(a).to(DEV)
    args = [t(us), t(them), t(white), t(black), t((pc - 1) // 4)]
    got = {}
    old = nnueft.get_backward_mode()
    try:
        for mode in ("deterministic_strict", "deterministic", "atomic"):
            nnueft.set_backward_mode(mode)
            W, bias = W0.clone().requires_grad_(), b0.clone().requires_grad_()
            out = double_feature_transform(*args, W, bias, 255.0 / 256.0, L1, "fused")
            torch.autograd.backward(list(out), grads)
            got[mode] = (W.grad, bias.grad)
    finally:
        nnueft.set_backward_mode(old)
    strict_W, strict_b = got["deterministic_strict"]
    whole = torch.from_numpy(counts <= 512).to(DEV)
    assert torch.equal(got["deterministic"][0][whole], strict_W[whole])
    assert not torch.equal(got["deterministic"][0], strict_W)
    assert torch.equal(got["deterministic"][1], strict_b)
    scale = strict_W.abs().max()
    assert (got["deterministic"][0] - strict_W).abs().max() <= 1e-5 * scale
    assert (got["atomic"][0] - strict_W).abs().max() <= 1e-4 * scale
    assert torch.equal(got["atomic"][1], strict_b)


def test_reduce_rows_stage_equals_the_sparse_backward(oracle_cpu):
    """nnueft_det_sort + nnueft_det_reduce_rows on G = gout is the weight gradient of nnueft_sparse_bwd_det."""
    lib = _native.load()
    B, K, R, oc = 3000, 32, 900, 264
    c = sparse_case(41, B, oc, R, K, allow_holes=True)
    c["idx"][np.random.default_rng(1).random((B, K)) < 0.1] = 17          # a row beyond the split threshold
    idx, g = torch.from_numpy(c["idx"]).to(DEV), torch.from_numpy(c["g"]).to(DEV)
    st = torch.cuda.current_stream().cuda_stream
    for rs in (lib.nnueft_row_split(), 0):
        nbytes = lib.nnueft_det_workspace_bytes(B, K, R, oc, 1, rs)
        sbytes = lib.nnueft_det_sort_bytes(B, K, R, oc, 1)
        ws = torch.empty(nbytes, dtype=torch.uint8, device=DEV)
        lists = torch.empty(sbytes, dtype=torch.uint8, device=DEV)
        gW = torch.full((R, oc), float("nan"), device=DEV)
        _native.check(lib.nnueft_det_sort(idx.data_ptr(), None, B, K, R, oc, 1, rs, lists.data_ptr(), sbytes, st), "sort")
        for _ in range(2):        # the sorted block serves a second reduction
            gW.fill_(float("nan"))
            _native.check(lib.nnueft_det_reduce_rows(g.data_ptr(), gW.data_ptr(), B, K, R, oc, 1, rs, ws.data_ptr(),
                                                     nbytes, lists.data_ptr(), st), "reduce_rows")
            rW, _ = oracle_cpu.sparse_bwd(c["idx"], c["g"], R, row_split=rs)
            assert np.array_equal(gW.cpu().numpy(), rW)
        # the same rows at the pitch the two-perspective backward gives its own upstream rows
        pitch = lib.nnueft_det_upstream_pitch(oc)
        assert pitch >= oc and pitch % 32 == 0
        gp = torch.full((B, pitch), float("nan"), device=DEV)
        gp[:, :oc] = g
        gW.fill_(float("nan"))
        _native.check(lib.nnueft_det_reduce_rows_pitched(gp.data_ptr(), pitch, gW.data_ptr(), B, K, R, oc, 1, rs,
                                                         ws.data_ptr(), nbytes, lists.data_ptr(), st), "reduce_rows_pitched")
        assert np.array_equal(gW.cpu().numpy(), rW)
        assert lib.nnueft_det_reduce_rows_pitched(gp.data_ptr(), oc - 1, gW.data_ptr(), B, K, R, oc, 1, rs, ws.data_ptr(),
                                                  nbytes, lists.data_ptr(), st) == -1


@pytest.mark.parametrize("L1", [256, 1024, 2048],
                         ids=["l2_blocked_forward", "lds_tiled_forward", "lds_tiled_forward_that_writes_the_output_rows"])
def test_forward_and_deterministic_backward_under_graph_capture(L1):
    """The launch path of the operator inside one captured HIP graph: forward + deterministic backward (sort
    inline, workspaces allocated before the capture), replayed with eager work and synchronisations between the
    replays; every replay must give the bits of the eager run, also after the inputs changed in place.  Both
    forward gathers: blocked for L2 (narrow rows) and out of LDS tiles (its unit counters live in the workspace
    and are reset by the sort of every call; from L1 = 2048 on it also writes the output rows, and its sign for a sum
    that is not finite lives there too)."""
    lib = _native.load()
    B, K, R, n_psqt = 4096, 32, hk.NUM_INPUTS, 8
    oc = L1 + n_psqt
    rs = lib.nnueft_row_split()
    t = lambda a: torch.from_numpy(a).to(DEV)
    batches = []
    for seed in (50, 51):
        us, them, white, black, pc = hk.synthetic_batch(B, seed, game_like=(seed == 51))
        batches.append([t(us), t(them), t(white), t(black), t((pc - 1) // 4)])
    g = torch.Generator().manual_seed(3)
    W = (torch.randn(R, oc, generator=g) * 0.02).to(DEV)
    bias = (torch.randn(oc, generator=g) * 0.02).to(DEV)
    g_l0, g_wp, g_bp = (torch.randn(B, L1, generator=g).to(DEV), torch.randn(B, 1, generator=g).to(DEV),
                        torch.randn(B, 1, generator=g).to(DEV))
    cur = [x.clone() for x in batches[0]]            # the graph's input buffers
    fbytes = lib.nnueft_fwd_workspace_bytes(B, K, R, L1, n_psqt)
    dbytes = lib.nnueft_det_workspace_bytes(B, K, R, oc, 2, rs)
    fws = torch.empty(fbytes, dtype=torch.uint8, device=DEV)
    dws = torch.empty(dbytes, dtype=torch.uint8, device=DEV)

    def outputs():
        return (torch.empty(B, L1, device=DEV), torch.empty(B, device=DEV), torch.empty(B, device=DEV),
                torch.empty(2, B, L1, device=DEV), torch.empty(R, oc, device=DEV), torch.empty(oc, device=DEV))

    def launch(o, stream):
        l0, wp, bp, saved, gW, gb = o
        us, them, white, black, psqt = cur
        _native.check(lib.nnueft_double_fwd(us.data_ptr(), them.data_ptr(), white.data_ptr(), black.data_ptr(),
                                            psqt.data_ptr(), W.data_ptr(), bias.data_ptr(), 255.0 / 256.0, l0.data_ptr(),
                                            wp.data_ptr(), bp.data_ptr(), saved.data_ptr(), B, K, R, L1, n_psqt,
                                            fws.data_ptr(), fbytes, stream), "fwd")
        _native.check(lib.nnueft_double_bwd_det(us.data_ptr(), them.data_ptr(), white.data_ptr(), black.data_ptr(),
                                                psqt.data_ptr(), bias.data_ptr(), 255.0 / 256.0, g_l0.data_ptr(),
                                                g_wp.data_ptr(), g_bp.data_ptr(), saved.data_ptr(), gW.data_ptr(),
                                                gb.data_ptr(), B, K, R, L1, n_psqt, rs, dws.data_ptr(), dbytes, None,
                                                stream, None), "bwd")

    eager = []
    for b in batches:                                  # also the first calls on the device, outside any capture
        for dst, src in zip(cur, b):
            dst.copy_(src)
        o = outputs()
        launch(o, torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        eager.append([x.clone() for x in o])
    assert not torch.equal(eager[0][4], eager[1][4])

    captured = outputs()
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            launch(captured, torch.cuda.current_stream().cuda_stream)
    torch.cuda.current_stream().wait_stream(side)
    for replay in range(4):
        which = replay % 2
        for dst, src in zip(cur, batches[which]):
            dst.copy_(src)
        for x in captured:
            x.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        for got, want in zip(captured, eager[which]):
            assert torch.equal(got, want), f"replay {replay} differs from the eager run"
        # the program's own eager work between replays
        launch(outputs(), torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()


@pytest.mark.parametrize("mode", ["deterministic", "atomic"])
@pytest.mark.parametrize("backend", ["aot_eager", "inductor", "cudagraphs"])
def test_operator_stays_inside_a_compiled_graph(backend, mode):
    """The operator under plain torch modules, as when it is dropped under the reference's own
    ComposedFeatureTransformer: table merge and fake quantization in torch ops, double_feature_transform, the
    activation grid, a loss.  torch.compile with fullgraph=True raises on any graph break, so passing means
    the launches are part of the compiled graph; with "cudagraphs" they are then inside the captured HIP graph
    (no 'CUDA Graph is empty' warning), replayed four times and compared with the eager run every time."""
    import warnings

    nnueft.set_backward_mode(mode)
    torch._dynamo.reset()
    L1, B, R = 256, 2048, hk.NUM_INPUTS
    g = torch.Generator().manual_seed(77)
    W = (torch.randn(R, L1 + 8, generator=g) * 0.02).to(DEV).requires_grad_()
    V = (torch.randn(768, L1 + 8, generator=g) * 0.005).to(DEV).requires_grad_()
    bias = (torch.randn(L1 + 8, generator=g) * 0.02).to(DEV).requires_grad_()
    target = torch.rand(B, 1, generator=g).to(DEV)

    def step(us, them, white, black, psqt):
        merged = W + V.repeat(R // 768, 1)
        merged = merged + ((merged * 256.0).round() / 256.0 - merged).detach()          # fake quantization, STE
        l0, wp, bp = double_feature_transform(us, them, white, black, psqt, merged, bias, 255.0 / 256.0, L1, "fused")
        l0 = l0 + ((l0 * 127.0 + 1e-5).floor() / 127.0 - l0).detach()
        out = l0.sum(dim=1, keepdim=True) * 0.01 + (wp - bp) * (us - 0.5)
        return ((out.sigmoid() - target) ** 2).mean()

    def grads(fn, batch):
        for p in (W, V, bias):
            p.grad = None
        loss = fn(*batch)
        loss.backward()
        return [loss.detach().clone()] + [p.grad.clone() for p in (W, V, bias)]

    batches = []
    for seed in (61, 62):
        us, them, white, black, pc = hk.synthetic_batch(B, seed)
        batches.append([torch.from_numpy(a).to(DEV) for a in (us, them, white, black, (pc - 1) // 4)])
    eager = [grads(step, b) for b in batches]
    compiled = torch.compile(step, backend=backend, fullgraph=True)
    with warnings.catch_warnings(record=True) as seen:
        warnings.simplefilter("always")
        for call in range(4):
            got = grads(compiled, batches[call % 2])
            want = eager[call % 2]
            torch.testing.assert_close(got[0], want[0], atol=1e-6, rtol=1e-5)
            if mode == "deterministic" and backend != "inductor":      # same ops around the operator: same bits
                assert torch.equal(got[1], want[1])
            for a, b in zip(got[1:], want[1:]):
                torch.testing.assert_close(a, b, atol=1e-5, rtol=1e-4)
    assert not [w for w in seen if "Graph is empty" in str(w.message)]
    torch._dynamo.reset()


def test_custom_ops_pass_torch_opcheck():
    """torch.library.opcheck on the operator's four launches: the declared schema (nothing mutated, nothing
    aliased) and the shape functions against what the kernels really return."""
    from nnueft import _ops  # noqa: F401

    B, L1, R, K = 300, 64, 900, 32
    c = double_case(5, B, L1, R, K, binary_side=True)
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(DEV)
    us, them, widx, bidx, psqt = t(c["us"]), t(c["them"]), t(c["widx"]), t(c["bidx"]), t(c["psqt_idx"])
    W, bias = t(c["W"]), t(c["bias"])
    checks = ("test_schema", "test_faketensor")
    torch.library.opcheck(torch.ops.nnueft.sparse_fwd.default, (widx, W, bias), test_utils=checks)
    g = torch.randn(B, L1 + 8, device=DEV)
    for mode in ("deterministic", "deterministic_strict", "atomic"):
        torch.library.opcheck(torch.ops.nnueft.sparse_bwd.default, (widx, g, R, mode), test_utils=checks)
    fwd_args = (us, them, widx, bidx, psqt, W, bias, 0.99, L1, False, 1.0, 0.0, 1.0)
    torch.library.opcheck(torch.ops.nnueft.double_fwd.default, fwd_args, test_utils=checks)
    torch.library.opcheck(torch.ops.nnueft.double_fwd.default, fwd_args[:9] + (True, 127.0, 1e-5, 1.0), test_utils=checks)
    l0, wp, bp, saved = torch.ops.nnueft.double_fwd(*fwd_args)
    lists = torch.ops.nnueft.det_sort(widx, bidx, R, L1 + 8, 512)
    torch.library.opcheck(torch.ops.nnueft.det_sort.default, (widx, bidx, R, L1 + 8, 512), test_utils=checks)
    torch.cuda.synchronize()
    for mode, presorted in (("deterministic", None), ("deterministic", lists), ("atomic", None)):
        torch.library.opcheck(torch.ops.nnueft.double_bwd.default,
                              (us, them, widx, bidx, psqt, bias, 0.99, torch.randn_like(l0), torch.randn_like(wp),
                               torch.randn_like(bp), saved, R, L1, L1 + 8, mode, presorted, False), test_utils=checks)


FULL = [(1024, 8192), (128, 16384), (3072, 16384)]   # BASELINE.json configs 1-3


@pytest.mark.parametrize("L1,B", FULL)
def test_baseline_configs_full_size_against_oracle(oracle_cpu, L1, B):
    """fwd bit-exact, both deterministic orders bit-exact (the strict one is the reference CPU path's), atomic
    backward 1e-4 relative, at full size."""
    n_psqt, R = 8, hk.NUM_INPUTS
    us, them, white, black, pc = hk.synthetic_batch(B, 1234 + L1)
    psqt_idx = (pc - 1) // 4
    g = torch.Generator().manual_seed(L1)
    Wn = (torch.randn(R, L1 + n_psqt, generator=g) * 0.01).numpy()
    bn = np.zeros(L1 + n_psqt, np.float32)
    grads = [torch.randn(B, L1, generator=g).numpy(), torch.randn(B, 1, generator=g).numpy(),
             torch.randn(B, 1, generator=g).numpy()]
    max_act = 255.0 / 256.0
    r_l0, r_wp, r_bp, r_saved = oracle_cpu.double_fwd(us, them, white, black, psqt_idx, Wn, bn, max_act, L1)
    r_gW, r_gb = oracle_cpu.double_bwd(us, them, white, black, psqt_idx, bn, max_act, grads[0], grads[1], grads[2],
                                       r_saved, R, n_psqt)
    s_gW, s_gb = oracle_cpu.double_bwd(us, them, white, black, psqt_idx, bn, max_act, grads[0], grads[1], grads[2],
                                       r_saved, R, n_psqt, row_split=0)
    assert not np.array_equal(s_gW, r_gW)   # the two orders differ on the rows named beyond the split threshold
    t = lambda a: torch.from_numpy(a).to(DEV)
    args = [t(us), t(them), t(white), t(black), t(psqt_idx)]
    det = None
    for mode in ("deterministic", "atomic", "deterministic_strict", "deterministic"):
        nnueft.set_backward_mode(mode)
        W = t(Wn).requires_grad_()
        bias = t(bn).requires_grad_()
        out = double_feature_transform(*args, W, bias, max_act, L1, "fused")
        torch.autograd.backward(list(out), [t(x) for x in grads])
        assert np.array_equal(out[0].detach().cpu().numpy(), r_l0)
        assert np.array_equal(out[1].detach().cpu().numpy(), r_wp)
        assert np.array_equal(out[2].detach().cpu().numpy(), r_bp)
        gW, gb = W.grad.cpu().numpy(), bias.grad.cpu().numpy()
        if mode == "deterministic":
            assert np.array_equal(gW, r_gW)
            assert np.array_equal(gb, r_gb)
            if det is not None:          # run to run
                assert np.array_equal(gW, det[0]) and np.array_equal(gb, det[1])
            det = (gW, gb)
        elif mode == "deterministic_strict":
            assert np.array_equal(gW, s_gW)
            assert np.array_equal(gb, s_gb)
        else:
            assert np.abs(gW - r_gW).max() <= 1e-4 * np.abs(r_gW).max()
            assert np.abs(gb - r_gb).max() <= 1e-4 * np.abs(r_gb).max()
        del W, bias, out


def test_int16_full_size_against_oracle(oracle_cpu):
    """BASELINE.json config 5: L1=3072, B=65536, exported numbering (22528 rows), quantized weights."""
    from nnueft import quantized

    L1, B, R = 3072, 65536, hk.NUM_INPUTS_EXPORT
    us, them, white, black, pc = hk.synthetic_batch(B, 1239, fold_kings=True)
    g = torch.Generator().manual_seed(5)
    W = torch.randn(R, L1 + 8, generator=g) * 0.02
    W[:, L1:] = torch.randn(R, 8, generator=g) * 0.5
    bias = torch.randn(L1 + 8, generator=g) * 0.1
    w16, b16, p32 = quantized.quantize_feature_transformer(W, bias, L1)
    stm = (1 - us[:, 0]).astype(np.uint8)
    psqt_idx = (pc - 1) // 4
    t = lambda a: torch.from_numpy(a).to(DEV)
    out, ps = quantized.ft_int16_forward(t(white), t(black), t(stm), w16.to(DEV), b16.to(DEV), p32.to(DEV), t(psqt_idx))
    r_out, r_ps = oracle_cpu.ft_int16_fwd(white, black, stm, w16.numpy(), b16.numpy(), p32.numpy(), psqt_idx)
    assert np.array_equal(out.cpu().numpy(), r_out)
    assert np.array_equal(ps.cpu().numpy(), r_ps)
    assert 0 < r_out.max() <= 127 and (r_out > 0).mean() > 0.05


@pytest.mark.parametrize("mode", ["atomic", "deterministic"])
def test_every_slot_names_the_same_row(oracle_cpu, mode):
    """Worst case for both backward modes: one table row receives all B*K contributions."""
    nnueft.set_backward_mode(mode)
    B, K, R, oc = 2048, 32, 3, 136
    idx = np.full((B, K), 1, np.int32)
    c = sparse_case(5, B, oc, R, K)
    W = torch.from_numpy(c["W"]).to(DEV).requires_grad_()
    bias = torch.from_numpy(c["bias"]).to(DEV).requires_grad_()
    out = SparseLinearFunction.apply(torch.from_numpy(idx).to(DEV), W, bias)
    out.backward(torch.from_numpy(c["g"]).to(DEV))
    assert np.array_equal(out.detach().cpu().numpy(), oracle_cpu.sparse_fwd(idx, c["W"], c["bias"]))
    rW, rb = oracle_cpu.sparse_bwd(idx, c["g"], R)
    if mode == "deterministic":
        assert np.array_equal(W.grad.cpu().numpy(), rW) and np.array_equal(bias.grad.cpu().numpy(), rb)
    else:
        assert np.abs(W.grad.cpu().numpy() - rW).max() <= 1e-4 * np.abs(rW).max()
        assert np.abs(bias.grad.cpu().numpy() - rb).max() <= 1e-4 * np.abs(rb).max()
    assert not W.grad[0].any() and not W.grad[2].any()


@pytest.mark.parametrize("mode", ["atomic", "deterministic"])
def test_empty_batch_and_all_padding(mode):
    nnueft.set_backward_mode(mode)
    W = torch.randn(20, 40, device=DEV, requires_grad=True)
    bias = torch.randn(40, device=DEV, requires_grad=True)
    empty = torch.empty(0, 32, dtype=torch.int32, device=DEV)
    out = SparseLinearFunction.apply(empty, W, bias)
    assert out.shape == (0, 40)
    out.sum().backward()
    assert not W.grad.any() and not bias.grad.any()
    W.grad = None
    bias.grad = None
    pad = torch.full((5, 32), -1, dtype=torch.int32, device=DEV)
    out = SparseLinearFunction.apply(pad, W, bias)
    assert torch.equal(out, bias.detach().expand(5, 40))
    out.backward(torch.ones_like(out))
    assert not W.grad.any()
    assert torch.equal(bias.grad, torch.full((40,), 5.0, device=DEV))


def test_non_default_stream(oracle_cpu):
    c = double_case(41, 300, 256, 500, binary_side=True)
    t = {k: torch.from_numpy(c[k]).to(DEV) for k in ("us", "them", "widx", "bidx", "psqt_idx", "W", "bias")}
    torch.cuda.synchronize()
    s = torch.cuda.Stream()
    nnueft.set_backward_mode("deterministic")
    with torch.cuda.stream(s):
        W = t["W"].clone().requires_grad_()
        bias = t["bias"].clone().requires_grad_()
        out = double_feature_transform(t["us"], t["them"], t["widx"], t["bidx"], t["psqt_idx"], W, bias,
                                       c["max_act"], 256, "fused")
        torch.autograd.backward(list(out), [torch.from_numpy(c[k]).to(DEV) for k in ("g_l0", "g_wp", "g_bp")])
    s.synchronize()
    r = oracle_cpu.double_fwd(c["us"], c["them"], c["widx"], c["bidx"], c["psqt_idx"], c["W"], c["bias"], c["max_act"], 256)
    assert np.array_equal(out[0].detach().cpu().numpy(), r[0])
    rW, rb = oracle_cpu.double_bwd(c["us"], c["them"], c["widx"], c["bidx"], c["psqt_idx"], c["bias"], c["max_act"],
                                   c["g_l0"], c["g_wp"], c["g_bp"], r[3], 500, 8)
    assert np.array_equal(W.grad.cpu().numpy(), rW) and np.array_equal(bias.grad.cpu().numpy(), rb)


@pytest.mark.parametrize("on_stream", [False, True], ids=["default_stream", "side_stream"])
def test_sort_placements_give_the_same_bits(oracle_cpu, on_stream):
    """The index sort inline, on a second stream in the backward pass, or started by the forward
    pass: same outputs and gradients, bit for bit, also when the graph is walked twice."""
    nnueft.set_backward_mode("deterministic")
    B, L1 = 5000, 512
    c = double_case(77, B, L1, hk.NUM_INPUTS, 32, halfka=True, max_act=255 / 256, weight_scale=0.05)
    us, them, widx, bidx, pc = hk.synthetic_batch(B, 77, game_like=True)     # has rows that are split
    c.update(us=us, them=them, widx=widx, bidx=bidx, psqt_idx=((pc - 1) // 4).astype(np.int64))
    t = {k: torch.from_numpy(c[k]).to(DEV) for k in ("us", "them", "widx", "bidx", "psqt_idx", "W", "bias")}
    grads = [torch.from_numpy(c[k]).to(DEV) for k in ("g_l0", "g_wp", "g_bp")]
    torch.cuda.synchronize()
    stream = torch.cuda.Stream() if on_stream else torch.cuda.current_stream()
    got = {}
    for where in ("inline", "backward", "forward"):
        nnueft.set_sort_placement(where)
        with torch.cuda.stream(stream):
            W = t["W"].clone().requires_grad_()
            bias = t["bias"].clone().requires_grad_()
            out = double_feature_transform(t["us"], t["them"], t["widx"], t["bidx"], t["psqt_idx"], W, bias,
                                           c["max_act"], L1, "fused")
            torch.autograd.backward(list(out), grads, retain_graph=True)
            first = (W.grad.clone(), bias.grad.clone())
            W.grad = bias.grad = None
            torch.autograd.backward(list(out), grads)
        stream.synchronize()
        assert torch.equal(first[0], W.grad) and torch.equal(first[1], bias.grad)
        got[where] = (out[0].detach(), W.grad, bias.grad)
    for where in ("backward", "forward"):
        for a, b in zip(got[where], got["inline"]):
            assert torch.equal(a, b)
    r = oracle_cpu.double_fwd(c["us"], c["them"], c["widx"], c["bidx"], c["psqt_idx"], c["W"], c["bias"],
                              c["max_act"], L1)
    rW, rb = oracle_cpu.double_bwd(c["us"], c["them"], c["widx"], c["bidx"], c["psqt_idx"], c["bias"], c["max_act"],
                                   c["g_l0"], c["g_wp"], c["g_bp"], r[3], hk.NUM_INPUTS, 8)
    assert np.array_equal(got["inline"][1].cpu().numpy(), rW) and np.array_equal(got["inline"][2].cpu().numpy(), rb)
    with pytest.raises(ValueError):
        nnueft.set_sort_placement("elsewhere")


def test_fused_function_with_nine_and_ten_arguments(oracle_cpu):
    """The reference calls FusedDoubleFtFunction.apply with nine arguments; the tenth (the activation
    grid applied inside the forward) is this build's.  Both forms differentiate, and the grid is the
    oracle's, with a straight-through gradient scaled by its post-multiplier."""
    from nnueft.fused_ft_functions import FusedDoubleFtFunction

    nnueft.set_backward_mode("deterministic")
    c = double_case(53, 700, 256, 900, binary_side=True)
    t = {k: torch.from_numpy(c[k]).to(DEV) for k in ("us", "them", "widx", "bidx", "psqt_idx", "W", "bias")}
    grads = [torch.from_numpy(c[k]).to(DEV) for k in ("g_l0", "g_wp", "g_bp")]
    got = {}
    for extra in ((), ((127.0, 1e-5, 0.5),), (None,)):
        W = t["W"].clone().requires_grad_()
        bias = t["bias"].clone().requires_grad_()
        out = FusedDoubleFtFunction.apply(t["us"], t["them"], t["widx"], t["bidx"], t["psqt_idx"], W, bias,
                                          c["max_act"], 256, *extra)
        torch.autograd.backward(list(out), grads)
        got[extra] = (out[0].detach().cpu().numpy(), W.grad.cpu().numpy(), bias.grad.cpu().numpy())
    plain, grid, none = got[()], got[((127.0, 1e-5, 0.5),)], got[(None,)]
    for a, b in zip(plain, none):
        assert np.array_equal(a, b)
    assert np.array_equal(grid[0], oracle_cpu.act_fake_quantize(plain[0], 127.0, 1e-5, 0.5))
    # straight-through: the gradient of the plain call with the upstream gradient of l0 halved
    W = t["W"].clone().requires_grad_()
    bias = t["bias"].clone().requires_grad_()
    out = FusedDoubleFtFunction.apply(t["us"], t["them"], t["widx"], t["bidx"], t["psqt_idx"], W, bias, c["max_act"], 256)
    torch.autograd.backward(list(out), [grads[0] * 0.5, grads[1], grads[2]])
    assert np.array_equal(grid[1], W.grad.cpu().numpy()) and np.array_equal(grid[2], bias.grad.cpu().numpy())
    with pytest.raises(TypeError):
        FusedDoubleFtFunction.apply(t["us"], t["them"], t["widx"], t["bidx"], t["psqt_idx"], W, bias, c["max_act"],
                                    256, None, None)


def test_device_presents_the_xcd_layout_the_blocked_kernels_are_made_for():
    # MI355X in its default partition mode: 8 XCDs (0 = the runtime does not say; the blocked kernels then run too)
    assert _native.load().nnueft_device_xcds() in (0, 8)


def test_abi_rejects_bad_arguments():
    lib = _native.load()
    x = torch.zeros(64, device=DEV)
    p = x.data_ptr()
    st = torch.cuda.current_stream().cuda_stream
    assert lib.nnueft_sparse_fwd(p, p, p, p, 4, 0, 10, 8, st) == -1                 # K = 0
    assert lib.nnueft_sparse_fwd(0, p, p, p, 4, 8, 10, 8, st) == -1                 # null pointer
    assert lib.nnueft_double_fwd(p, p, p, p, p, p, p, 1.0, p, p, p, p, 4, 8, 10, 7, 1, None, 0, st) == -1    # odd L1
    assert lib.nnueft_double_fwd(p, p, p, p, p, p, p, 1.0, p, p, p, p, 4, 8, 10, 8, 0, p, 8, st) == -2       # workspace too small
    assert lib.nnueft_sparse_bwd_det(p, p, p, p, 4, 8, 10, 8, 512, p, 16, st) == -2      # workspace too small
    assert lib.nnueft_sparse_bwd_det(p, p, p, p, 4, 8, 10, 8, 512, 0, 1 << 20, st) == -2  # workspace missing
    assert lib.nnueft_sparse_bwd_det(p, p, p, p, 4, 8, 10, 8, 0, p + 4, 1 << 20, st) == -2  # misaligned
    assert lib.nnueft_sparse_bwd_det(p, p, p, p, 4, 8, 10, 8, -1, p, 1 << 20, st) == -1   # negative row_split
    assert lib.nnueft_ft_int16_fwd(p, p, p, p, p, p, p, p, p, 4, 8, 10, 8, 8, 70000, 9, 0, None, 0, st) == -1   # clip_max
    # the entry points around the operator reject what they cannot run, before any launch
    assert lib.nnueft_det_sort(p, p, 4, 8, 10, 8, 2, 512, p, 16, st) == -2                # sorted block too small
    assert lib.nnueft_det_sort(p, p, 4, 8, 10, 8, 2, 0, p + 4, 1 << 20, st) == -2       # misaligned
    assert lib.nnueft_det_sort(p, None, 4, 8, 10, 8, 2, 512, p, 1 << 20, st) == -1        # two lists asked, one given
    assert lib.nnueft_det_reduce_rows(p, p, 4, 8, 10, 8, 2, 512, p, 1 << 30, None, st) == -2   # no sorted lists
    assert lib.nnueft_double_fwd_noalloc(p, p, p, p, p, p, p, 1.0, p, p, p, p, 4, 8, 10, 7, 1, st) == -1      # odd L1
    assert lib.nnueft_double_fwd_noalloc(p, p, p, p, p, p, p, 1.0, p, p, p, p, 1 << 20, 8, 24576, 8, 0, st) == -4   # beyond the fixed scratch
    assert lib.nnueft_det_sort_bytes(4, 8, 10, 8, 3) == 0                            # one or two perspectives
    assert lib.nnueft_double_bwd_det(p, p, p, p, p, p, 1.0, p, p, p, p, p, p, 4, 8, 10, 8, 0, 512, p, 1 << 30, p + 4,
                                     st, None) == -2                                      # sorted lists misaligned
    assert lib.nnueft_ranger_lite_update_multi(None, 0, st) == -1
    assert lib.nnueft_sqr_crelu_fwd(p, p, p, 4, 1, 127.0, 1e-5, 1.0, 1.0, 1, st) == -1     # skip value needs 2 columns
    assert lib.nnueft_sqr_crelu_fwd(p, p, None, 4, 4, 0.0, 1e-5, 1.0, 1.0, 1, st) == -1    # grid without a scale
    assert lib.nnueft_stack_output_fwd(p, p, p, p, p, p, 4, 0, 600, 1, st) == -1           # output grid without den
    assert lib.nnueft_sf_loss_fwd(p, p, p, p, p, p, 4, 270.0, 0.0, 270.0, 380.0, 2.5, 0.0, 0.0, 0.5, 4000.0, 4000.0,
                                  0.85, 1.0, st) == -1                                # scaling must be positive
    assert lib.nnueft_batch_unpack(p, p, p, None, 4, st) == -1
    assert lib.nnueft_bucket_linear_fwd(p, p, p, p, p, 4, 48, 8, 8, p, 1 << 30, 0, st) == -3   # in % 32 != 0
    with pytest.raises(RuntimeError, match="invalid argument"):
        _native.check(-1, "x")
    torch.cuda.synchronize()


def test_python_preconditions_assert_like_the_reference():
    W = torch.randn(20, 40, device=DEV)
    bias = torch.randn(40, device=DEV)
    idx64 = torch.zeros(4, 8, dtype=torch.int64, device=DEV)
    with pytest.raises(AssertionError):
        SparseLinearFunction.apply(idx64, W, bias)                       # sparse_linear_functions.py:59
    idx = torch.zeros(4, 8, dtype=torch.int32, device=DEV)
    with pytest.raises(AssertionError):
        SparseLinearFunction.apply(idx, W.t().contiguous().t(), bias)    # not contiguous, :75
    us = torch.ones(4, 1, device=DEV)
    psqt = torch.zeros(4, dtype=torch.int64, device=DEV)
    with pytest.raises(AssertionError):
        double_feature_transform(us, us, idx, idx, psqt.int(), W, bias, 1.0, 32, "fused")   # fused_ft_functions.py:33
    with pytest.raises(AssertionError):
        double_feature_transform(us, us, idx, idx, psqt, W, bias, 1.0, 31, "fused")         # odd l1_size, :23
