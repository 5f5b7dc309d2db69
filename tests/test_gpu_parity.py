"""HIP kernels (through the C ABI of libnnueft.so) against the CPU oracle on the same seeded inputs.

Bars: forward 1e-5 relative, atomic backward 1e-4 relative, deterministic backward and the int16
path bit-exact.  (The forward and the deterministic weight gradient are in fact compared for
equality too: their summation order is the oracle's.)
"""
import numpy as np
import pytest
import torch

from _cases import double_case, sparse_case

pytestmark = pytest.mark.gpu


def _dev():
    assert torch.cuda.is_available(), "these tests need the GPU"
    return torch.device("cuda:0")


def _t(a):
    return torch.from_numpy(np.ascontiguousarray(a)).to(_dev())


def _rel_err(a, b):
    a = np.asarray(a, np.float64)
    b = np.asarray(b, np.float64)
    return float(np.abs(a - b).max() / max(np.abs(b).max(), 1e-30))


def _native():
    from nnueft import _native

    return _native, _native.load()


def _stream():
    return torch.cuda.current_stream().cuda_stream


# The row_split argument of the deterministic entry points under test: the library's default unless a
# test asks for another through the `row_split` fixture (0 = strict order, no row is split).
_RS_OVERRIDE = None


def RS(lib):
    return lib.nnueft_row_split() if _RS_OVERRIDE is None else _RS_OVERRIDE


@pytest.fixture(params=[None, 0, 100, 3000], ids=["split_default", "strict", "split_100", "split_3000"])
def row_split(request):
    global _RS_OVERRIDE
    _RS_OVERRIDE = request.param
    yield request.param
    _RS_OVERRIDE = None


SPARSE_SHAPES = [
    # B, out_cols, R, K
    (16, 128, 10, 32),      # reference tests/test_feature_transformer.py:36-40 (duplicates)
    (8, 64, 10, 8),         # its padding case, :83-89
    (5, 40, 100, 32),       # l1=32 + 8 psqt
    (33, 1032, 2000, 32),   # L1=1024 row width
    (7, 3080, 500, 32),     # L1=3072 row width
    (9, 37, 50, 70),        # odd width (scalar path), K > 64
    (64, 272, 24576, 32),   # bench_feature_transformer.py:22-25 width, full table height
    # widths a few columns beyond whole 64-lane slices (those columns are reduced many rows per wave):
    (300, 131, 700, 32),    # scalar path, 3 columns over, rows with and without slots
    (257, 70, 90, 16),      # scalar path, 6 over, every row named several times
    (120, 260, 1000, 32),   # 16-byte path, 1 vector over
    (90, 284, 333, 24),     # 16-byte path, 7 vectors over, range ends inside a group of rows
    # long lists over a long table: the sort's staged lists and its row counters together want all of a workgroup's LDS
    (40, 72, 40000, 64),
    (40, 72, 40000, 80),
]


@pytest.mark.parametrize("B,out_cols,R,K", SPARSE_SHAPES)
def test_sparse_forward(oracle_cpu, B, out_cols, R, K):
    c = sparse_case(100 + B, B, out_cols, R, K, allow_holes=True)
    nat, lib = _native()
    idx, W, bias = _t(c["idx"]), _t(c["W"]), _t(c["bias"])
    out = torch.empty(B, out_cols, device=_dev())
    nat.check(lib.nnueft_sparse_fwd(idx.data_ptr(), W.data_ptr(), bias.data_ptr(), out.data_ptr(), B, K, R,
                                    out_cols, _stream()), "sparse_fwd")
    ref = oracle_cpu.sparse_fwd(c["idx"], c["W"], c["bias"])
    got = out.cpu().numpy()
    assert _rel_err(got, ref) <= 1e-5
    assert np.array_equal(got, ref), "forward follows the oracle's summation order, so it is bit-exact"


@pytest.mark.parametrize("B,out_cols,R,K", SPARSE_SHAPES)
def test_sparse_backward_atomic(oracle_cpu, B, out_cols, R, K):
    c = sparse_case(200 + B, B, out_cols, R, K, allow_holes=True)
    nat, lib = _native()
    idx, g = _t(c["idx"]), _t(c["g"])
    gW = torch.zeros(R, out_cols, device=_dev())
    gb = torch.zeros(out_cols, device=_dev())
    nat.check(lib.nnueft_sparse_bwd_atomic(idx.data_ptr(), g.data_ptr(), gW.data_ptr(), gb.data_ptr(), B, K, R,
                                           out_cols, _stream()), "sparse_bwd_atomic")
    rW, rb = oracle_cpu.sparse_bwd(c["idx"], c["g"], R, row_split=_RS_OVERRIDE)
    assert _rel_err(gW.cpu().numpy(), rW) <= 1e-4
    assert _rel_err(gb.cpu().numpy(), rb) <= 1e-4


@pytest.mark.parametrize("B,out_cols,R,K", SPARSE_SHAPES + [(3000, 520, 1800, 32), (700, 1032, 768, 12)])
def test_sparse_backward_atomic_in_lds_tiles(oracle_cpu, B, out_cols, R, K):
    """nnueft_sparse_bwd_atomic_lds: the gradient is written (not accumulated), to the atomic bar; the bias
    gradient is the deterministic one.  Shapes it does not take answer with 0 bytes and NNUEFT_E_UNSUPPORTED."""
    c = sparse_case(250 + B, B, out_cols, R, K, allow_holes=True)
    nat, lib = _native()
    idx, g = _t(c["idx"]), _t(c["g"])
    gW = torch.full((R, out_cols), float("nan"), device=_dev())
    gb = torch.full((out_cols,), float("nan"), device=_dev())
    nbytes = lib.nnueft_atomic_lds_workspace_bytes(B, K, R, out_cols, 1)
    ws = torch.full((max(nbytes, 256),), 0xA5, dtype=torch.uint8, device=_dev())
    rc = lib.nnueft_sparse_bwd_atomic_lds(idx.data_ptr(), g.data_ptr(), gW.data_ptr(), gb.data_ptr(), B, K, R, out_cols,
                                          ws.data_ptr(), ws.numel(), _stream())
    if nbytes == 0:
        assert rc == nat.E_UNSUPPORTED and (K > 32 or out_cols % 4)
        return
    nat.check(rc, "sparse_bwd_atomic_lds")
    rW, rb = oracle_cpu.sparse_bwd(c["idx"], c["g"], R, row_split=0)
    assert _rel_err(gW.cpu().numpy(), rW) <= 1e-4
    assert np.array_equal(gb.cpu().numpy(), rb)
    assert lib.nnueft_sparse_bwd_atomic_lds(idx.data_ptr(), g.data_ptr(), gW.data_ptr(), gb.data_ptr(), B, K, R, out_cols,
                                            ws.data_ptr(), nbytes - 1, _stream()) == -2


def test_reduction_refuses_lists_sorted_for_another_threshold():
    """The sorted lists carry the threshold they were made for; a reduction asked for another one leaves the gradient
    unwritten instead of reading window sums that are not there (the call itself cannot report it: it does not wait
    for the device)."""
    nat, lib = _native()
    B, L1, R, K, n_psqt = 2000, 512, 768, 32, 8
    out_cols = L1 + n_psqt
    c = double_case(43, B, L1, R, K, weight_scale=0.05, max_act=0.9)
    d, l0, wp, bp, saved = _run_double_fwd(c)
    g_l0, g_wp, g_bp = _t(c["g_l0"]), _t(c["g_wp"]), _t(c["g_bp"])
    sbytes = lib.nnueft_det_sort_bytes(B, K, R, out_cols, 2)
    lists = torch.empty(sbytes, dtype=torch.uint8, device=_dev())
    nat.check(lib.nnueft_det_sort(d["widx"].data_ptr(), d["bidx"].data_ptr(), B, K, R, out_cols, 2, 100, lists.data_ptr(),
                                  sbytes, _stream()), "det_sort")
    for rs, written in ((100, True), (512, False), (0, False)):
        nbytes = lib.nnueft_det_workspace_bytes(B, K, R, out_cols, 2, rs)
        ws = torch.empty(nbytes, dtype=torch.uint8, device=_dev())
        gW = torch.full((R, out_cols), float("nan"), device=_dev())
        gb = torch.full((out_cols,), float("nan"), device=_dev())
        nat.check(lib.nnueft_double_bwd_det(d["us"].data_ptr(), d["them"].data_ptr(), d["widx"].data_ptr(), d["bidx"].data_ptr(),
                                            d["psqt_idx"].data_ptr(), d["bias"].data_ptr(), c["max_act"], g_l0.data_ptr(),
                                            g_wp.data_ptr(), g_bp.data_ptr(), saved.data_ptr(), gW.data_ptr(), gb.data_ptr(), B, K, R,
                                            L1, n_psqt, rs, ws.data_ptr(), nbytes, lists.data_ptr(), _stream(), None), "double_bwd_det")
        torch.cuda.synchronize()
        assert bool(torch.isnan(gW).any()) != written
        assert not bool(torch.isnan(gb).any())   # the bias gradient does not depend on the lists


@pytest.mark.parametrize("n_persp", [1, 2])
def test_deterministic_backward_with_more_split_rows_than_window_sums_are_kept_for(oracle_cpu, n_persp):
    """Every one of 700 table rows is named by more slots than the threshold (50): window sums are kept for 384 rows,
    the others are reduced whole, window by window in the same order; all of them bit-equal to the oracle.  The
    workspace does not grow with the number of rows that could be split."""
    nat, lib = _native()
    B, K, R, rs = 3000, 32, 700, 50
    if n_persp == 1:
        out_cols = 520
        c = sparse_case(41, B, out_cols, R, K)
        idx, g = _t(c["idx"]), _t(c["g"])
        nbytes = lib.nnueft_det_workspace_bytes(B, K, R, out_cols, 1, rs)
        assert nbytes < B * out_cols * 4 + 384 * 3 * out_cols * 4 + 16 * B * K + (4 << 20)
        ws = torch.empty(nbytes, dtype=torch.uint8, device=_dev())
        gW = torch.full((R, out_cols), float("nan"), device=_dev())
        gb = torch.full((out_cols,), float("nan"), device=_dev())
        nat.check(lib.nnueft_sparse_bwd_det(idx.data_ptr(), g.data_ptr(), gW.data_ptr(), gb.data_ptr(), B, K, R, out_cols, rs,
                                            ws.data_ptr(), nbytes, _stream()), "sparse_bwd_det")
        rW, rb = oracle_cpu.sparse_bwd(c["idx"], c["g"], R, row_split=rs)
        counts = np.bincount(c["idx"][c["idx"] >= 0], minlength=R)
    else:
        L1, n_psqt = 512, 8
        out_cols = L1 + n_psqt
        c = double_case(42, B, L1, R, K, weight_scale=0.05, max_act=0.9)
        d, l0, wp, bp, saved = _run_double_fwd(c)
        g_l0, g_wp, g_bp = _t(c["g_l0"]), _t(c["g_wp"]), _t(c["g_bp"])
        nbytes = lib.nnueft_det_workspace_bytes(B, K, R, out_cols, 2, rs)
        ws = torch.empty(nbytes, dtype=torch.uint8, device=_dev())
        gW = torch.full((R, out_cols), float("nan"), device=_dev())
        gb = torch.full((out_cols,), float("nan"), device=_dev())
        nat.check(lib.nnueft_double_bwd_det(d["us"].data_ptr(), d["them"].data_ptr(), d["widx"].data_ptr(), d["bidx"].data_ptr(),
                                            d["psqt_idx"].data_ptr(), d["bias"].data_ptr(), c["max_act"], g_l0.data_ptr(),
                                            g_wp.data_ptr(), g_bp.data_ptr(), saved.data_ptr(), gW.data_ptr(), gb.data_ptr(), B, K, R,
                                            L1, n_psqt, rs, ws.data_ptr(), nbytes, None, _stream(), None), "double_bwd_det")
        rW, rb = oracle_cpu.double_bwd(c["us"], c["them"], c["widx"], c["bidx"], c["psqt_idx"], c["bias"], c["max_act"],
                                       c["g_l0"], c["g_wp"], c["g_bp"], saved.cpu().numpy(), R, n_psqt, row_split=rs)
        counts = np.bincount(np.concatenate([c["widx"][c["widx"] >= 0], c["bidx"][c["bidx"] >= 0]]), minlength=R)
    assert (counts > rs).sum() > 600      # far more split rows than the 384 whose window sums are kept
    assert np.array_equal(gW.cpu().numpy(), rW)
    assert np.array_equal(gb.cpu().numpy(), rb)


@pytest.mark.parametrize("B,out_cols,R,K", SPARSE_SHAPES)
def test_sparse_backward_deterministic(oracle_cpu, B, out_cols, R, K):
    c = sparse_case(300 + B, B, out_cols, R, K, allow_holes=True)
    nat, lib = _native()
    idx, g = _t(c["idx"]), _t(c["g"])
    nbytes = lib.nnueft_det_workspace_bytes(B, K, R, out_cols, 1, RS(lib))
    assert nbytes > 0
    ws = torch.empty(nbytes, dtype=torch.uint8, device=_dev())
    # poison the outputs: every element must be written
    gW = torch.full((R, out_cols), float("nan"), device=_dev())
    gb = torch.full((out_cols,), float("nan"), device=_dev())
    nat.check(lib.nnueft_sparse_bwd_det(idx.data_ptr(), g.data_ptr(), gW.data_ptr(), gb.data_ptr(), B, K, R,
                                        out_cols, RS(lib), ws.data_ptr(), nbytes, _stream()), "sparse_bwd_det")
    rW, rb = oracle_cpu.sparse_bwd(c["idx"], c["g"], R, row_split=_RS_OVERRIDE)
    assert np.array_equal(gW.cpu().numpy(), rW)
    assert np.array_equal(gb.cpu().numpy(), rb)


DOUBLE_SHAPES = [
    # B, L1, R, K, kwargs
    (4, 32, 100, 32, {}),                      # reference tests/test_fused_double_ft.py:19-26
    (4, 2048, 100, 32, {}),                    # its second parametrisation
    (19, 264, 3000, 32, dict(binary_side=True)),   # bench_feature_transformer.py width
    (70, 128, 24576, 32, dict(halfka=True, weight_scale=0.05, max_act=255 / 256)),
    (40, 1024, 24576, 32, dict(halfka=True, weight_scale=0.05, max_act=255 / 256)),
    (24, 3072, 24576, 32, dict(halfka=True, weight_scale=0.05, max_act=255 / 256)),
    (6, 6, 20, 5, dict(n_psqt=3)),             # h = 3: scalar path
    (6, 50, 20, 80, dict(n_psqt=8, allow_holes=True)),   # K > 64, holes inside the lists
    (130, 64, 30, 32, dict(n_psqt=0)),         # no psqt columns, more than one sort chunk
    # rows wide enough for the LDS-tiled forward
    (300, 512, 2000, 32, {}),                  # lists that leave their 768-row block (summed from global memory)
    (700, 544, 24576, 32, dict(halfka=True, weight_scale=0.05, max_act=255 / 256)),   # 17 tiles over 8 XCDs
    (1500, 512, 1000, 20, dict(allow_holes=True)),   # K < 32, holes, a last block of 232 rows
    (2000, 576, 768, 32, dict(n_psqt=0)),      # one block, five chunks (as many as hold its list entries)
    (3500, 512, 768, 8, dict(n_psqt=0)),       # one block of short lists, five chunks (1536 pairs each at most)
    (500, 512, 2000, 30, {}),                  # K not a multiple of 4: the sort reads the lists entry by entry
    (300, 512, 50000, 32, {}),                 # 66 table blocks, more than the LDS-tiled kernels index: L2-blocked path
]


def _run_double_fwd(c, with_workspace=True):
    nat, lib = _native()
    B, K, R, L1, n_psqt = c["widx"].shape[0], c["K"], c["R"], c["L1"], c["n_psqt"]
    d = {k: _t(c[k]) for k in ("us", "them", "widx", "bidx", "psqt_idx", "W", "bias")}
    l0 = torch.full((B, L1), float("nan"), device=_dev())
    wp = torch.full((B, 1), float("nan"), device=_dev())
    bp = torch.full((B, 1), float("nan"), device=_dev())
    saved = torch.full((2, B, L1), float("nan"), device=_dev())
    nbytes = lib.nnueft_fwd_workspace_bytes(B, K, R, L1, n_psqt) if with_workspace else 0
    ws = torch.empty(max(nbytes, 1), dtype=torch.uint8, device=_dev())
    nat.check(lib.nnueft_double_fwd(d["us"].data_ptr(), d["them"].data_ptr(), d["widx"].data_ptr(),
                                    d["bidx"].data_ptr(), d["psqt_idx"].data_ptr(), d["W"].data_ptr(),
                                    d["bias"].data_ptr(), c["max_act"], l0.data_ptr(), wp.data_ptr(), bp.data_ptr(),
                                    saved.data_ptr(), B, K, R, L1, n_psqt,
                                    ws.data_ptr() if with_workspace else None, nbytes, _stream()), "double_fwd")
    return d, l0, wp, bp, saved


@pytest.mark.parametrize("with_workspace", [False, True], ids=["plain", "l2blocked"])
@pytest.mark.parametrize("B,L1,R,K,kw", DOUBLE_SHAPES)
def test_double_forward_with_activation_grid(oracle_cpu, B, L1, R, K, kw, with_workspace):
    """nnueft_double_fwd_act = nnueft_double_fwd followed by the activation grid, bit for bit (the grid
    against the oracle's act_fake_quantize)."""
    c = double_case(450 + B, B, L1, R, K, **kw)
    nat, lib = _native()
    d, l0, wp, bp, saved = _run_double_fwd(c, with_workspace)
    n_psqt = c["n_psqt"]
    l0q = torch.full((B, L1), float("nan"), device=_dev())
    wp2, bp2, saved2 = torch.empty_like(wp), torch.empty_like(bp), torch.empty_like(saved)
    nbytes = lib.nnueft_fwd_workspace_bytes(B, K, R, L1, n_psqt) if with_workspace else 0
    ws = torch.empty(max(nbytes, 1), dtype=torch.uint8, device=_dev())
    scale, eps, post_mul = 127.0, 1e-5, 0.75
    nat.check(lib.nnueft_double_fwd_act(d["us"].data_ptr(), d["them"].data_ptr(), d["widx"].data_ptr(),
                                        d["bidx"].data_ptr(), d["psqt_idx"].data_ptr(), d["W"].data_ptr(),
                                        d["bias"].data_ptr(), c["max_act"], l0q.data_ptr(), wp2.data_ptr(),
                                        bp2.data_ptr(), saved2.data_ptr(), B, K, R, L1, n_psqt,
                                        ws.data_ptr() if with_workspace else None, nbytes, scale, eps, post_mul,
                                        _stream()), "double_fwd_act")
    assert torch.equal(wp, wp2) and torch.equal(bp, bp2) and torch.equal(saved, saved2)
    want = oracle_cpu.act_fake_quantize(l0.cpu().numpy(), scale, eps, post_mul)
    assert np.array_equal(l0q.cpu().numpy(), want)
    assert lib.nnueft_double_fwd_act(d["us"].data_ptr(), d["them"].data_ptr(), d["widx"].data_ptr(),
                                     d["bidx"].data_ptr(), d["psqt_idx"].data_ptr(), d["W"].data_ptr(),
                                     d["bias"].data_ptr(), c["max_act"], l0q.data_ptr(), wp2.data_ptr(),
                                     bp2.data_ptr(), saved2.data_ptr(), B, K, R, L1, n_psqt, None, 0, 0.0, eps,
                                     post_mul, _stream()) == -1      # scale must be positive


@pytest.mark.parametrize("with_workspace", [False, True], ids=["plain", "l2blocked"])
@pytest.mark.parametrize("B,L1,R,K,kw", DOUBLE_SHAPES)
def test_double_forward(oracle_cpu, B, L1, R, K, kw, with_workspace):
    c = double_case(400 + B, B, L1, R, K, **kw)
    _, l0, wp, bp, saved = _run_double_fwd(c, with_workspace)
    r_l0, r_wp, r_bp, r_saved = oracle_cpu.double_fwd(c["us"], c["them"], c["widx"], c["bidx"], c["psqt_idx"],
                                                      c["W"], c["bias"], c["max_act"], L1)
    for got, ref in ((l0, r_l0), (wp, r_wp), (bp, r_bp), (saved, r_saved)):
        got = got.cpu().numpy()
        assert _rel_err(got, ref) <= 1e-5
        assert np.array_equal(got, ref)


@pytest.mark.parametrize("kind", ["mixed_sides", "a_sum_that_is_not_finite"])
@pytest.mark.parametrize("B,L1,R,K,kw", [
    (900, 2112, 24576, 32, dict(halfka=True, weight_scale=0.05, max_act=255 / 256)),  # lists inside their blocks; 33
                                                                                      # pairs of tiles over 8 XCDs
    (700, 2048, 2000, 32, dict(allow_holes=True)),                                    # lists that leave them
    (400, 2048, 1000, 20, dict(allow_holes=True, n_psqt=0)),                          # short lists, no psqt columns
    (300, 1024, 24576, 32, dict(halfka=True, weight_scale=0.05, max_act=255 / 256)),  # rows too narrow for it: the sums
                                                                                      # first, then the pass over them
])
def test_double_forward_rows_written_by_the_gather(oracle_cpu, kind, B, L1, R, K, kw):
    """From L1 = 2048 on the LDS-tiled gather writes a position's output row itself when (us, them) is (1, 0) or
    (0, 1), and leaves every other position to the pass behind it; the two must not be told apart in the result.  mixed_sides: both
    kinds of position (and signed zeros, which count as zero) in one batch.  a_sum_that_is_not_finite: an infinite
    weight makes 0 * inf = NaN in the other perspective's half of the row, as the mix of both perspectives gives it."""
    c = double_case(470 + B, B, L1, R, K, **kw)
    rng = np.random.default_rng(9)
    sides = np.array([(1.0, 0.0), (0.0, 1.0), (1.0, -0.0), (-0.0, 1.0), (0.5, 0.5), (1.0, 1.0), (0.0, 0.0), (1.0, 1e-3),
                      (2.0, 0.0)], np.float32)
    pick = sides[rng.integers(0, 4 if kind != "mixed_sides" else len(sides), size=B)]
    c["us"], c["them"] = np.ascontiguousarray(pick[:, :1]), np.ascontiguousarray(pick[:, 1:])
    if kind != "mixed_sides":
        rows = np.unique(c["widx"][c["widx"] >= 0])
        c["W"][rows[len(rows) // 2], 5] = np.inf
        c["W"][rows[len(rows) // 3], L1 // 2 + 40] = -np.inf
    for act in (False, True):
        nat, lib = _native()
        n_psqt = c["n_psqt"]
        d = {k: _t(c[k]) for k in ("us", "them", "widx", "bidx", "psqt_idx", "W", "bias")}
        l0 = torch.full((B, L1), float("nan"), device=_dev())
        wp, bp = torch.empty(B, 1, device=_dev()), torch.empty(B, 1, device=_dev())
        saved = torch.full((2, B, L1), float("nan"), device=_dev())
        nbytes = lib.nnueft_fwd_workspace_bytes(B, K, R, L1, n_psqt)
        ws = torch.empty(nbytes, dtype=torch.uint8, device=_dev())
        args = (d["us"].data_ptr(), d["them"].data_ptr(), d["widx"].data_ptr(), d["bidx"].data_ptr(),
                d["psqt_idx"].data_ptr(), d["W"].data_ptr(), d["bias"].data_ptr(), c["max_act"], l0.data_ptr(),
                wp.data_ptr(), bp.data_ptr(), saved.data_ptr(), B, K, R, L1, n_psqt, ws.data_ptr(), nbytes)
        if act:
            nat.check(lib.nnueft_double_fwd_act(*args, 127.0, 1e-5, 0.75, _stream()), "double_fwd_act")
        else:
            nat.check(lib.nnueft_double_fwd(*args, _stream()), "double_fwd")
        with np.errstate(invalid="ignore"):
            r_l0, r_wp, r_bp, r_saved = oracle_cpu.double_fwd(c["us"], c["them"], c["widx"], c["bidx"], c["psqt_idx"],
                                                              c["W"], c["bias"], c["max_act"], L1)
            if act:
                r_l0 = oracle_cpu.act_fake_quantize(r_l0, 127.0, 1e-5, 0.75)
        if kind != "mixed_sides":
            assert np.isnan(r_l0).any() and not np.isnan(r_l0).all(axis=1).any()
        for got, ref in ((l0, r_l0), (wp, r_wp), (bp, r_bp), (saved, r_saved)):
            assert np.array_equal(got.cpu().numpy(), ref, equal_nan=True)
        # a second forward over the same workspace, now without the weight: the sign that a sum was not finite is gone
        if kind != "mixed_sides" and not act:
            Wf = c["W"].copy()
            Wf[~np.isfinite(Wf)] = 0.25
            d["W"].copy_(_t(Wf))
            nat.check(lib.nnueft_double_fwd(*args, _stream()), "double_fwd")
            r_l0 = oracle_cpu.double_fwd(c["us"], c["them"], c["widx"], c["bidx"], c["psqt_idx"], Wf, c["bias"],
                                         c["max_act"], L1)[0]
            assert np.array_equal(l0.cpu().numpy(), r_l0)
            d["W"].copy_(_t(c["W"]))


def test_double_forward_from_index_lists_that_are_not_16_byte_aligned(oracle_cpu):
    """Index tensors that begin 4 bytes past a 16-byte boundary (a view into a larger buffer): the sort of the
    LDS-tiled forward then reads the lists entry by entry; same bits."""
    B, L1, R, K = 600, 512, 24576, 32
    c = double_case(77, B, L1, R, K, halfka=True, weight_scale=0.05, max_act=255 / 256)
    nat, lib = _native()
    d = {k: _t(c[k]) for k in ("us", "them", "psqt_idx", "W", "bias")}
    bufs = []
    for name in ("widx", "bidx"):
        buf = torch.empty(B * K + 1, dtype=torch.int32, device=_dev())
        buf[1:] = _t(c[name]).reshape(-1)
        assert buf[1:].data_ptr() % 16 == 4
        bufs.append(buf)
    n_psqt = c["n_psqt"]
    l0 = torch.full((B, L1), float("nan"), device=_dev())
    wp = torch.empty(B, 1, device=_dev())
    bp = torch.empty(B, 1, device=_dev())
    saved = torch.full((2, B, L1), float("nan"), device=_dev())
    nbytes = lib.nnueft_fwd_workspace_bytes(B, K, R, L1, n_psqt)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=_dev())
    nat.check(lib.nnueft_double_fwd(d["us"].data_ptr(), d["them"].data_ptr(), bufs[0][1:].data_ptr(), bufs[1][1:].data_ptr(),
                                    d["psqt_idx"].data_ptr(), d["W"].data_ptr(), d["bias"].data_ptr(), c["max_act"],
                                    l0.data_ptr(), wp.data_ptr(), bp.data_ptr(), saved.data_ptr(), B, K, R, L1, n_psqt,
                                    ws.data_ptr(), nbytes, _stream()), "double_fwd")
    r_l0, r_wp, r_bp, r_saved = oracle_cpu.double_fwd(c["us"], c["them"], c["widx"], c["bidx"], c["psqt_idx"], c["W"], c["bias"],
                                                      c["max_act"], L1)
    for got, ref in ((l0, r_l0), (wp, r_wp), (bp, r_bp), (saved, r_saved)):
        assert np.array_equal(got.cpu().numpy(), ref)


def test_double_forward_with_more_chunks_than_the_tiled_sort_indexes(oracle_cpu):
    """2 B / 512 beyond 1024: the sort of the LDS-tiled forward cannot keep the chunk table in LDS, the entry point
    takes the L2-blocked kernels; same bits."""
    B, L1, R, K = 262144, 512, 768, 8
    rng = np.random.default_rng(5)
    c = double_case(78, 8, L1, R, K, n_psqt=0, binary_side=True, weight_scale=0.05, max_act=0.9)
    widx = rng.integers(0, R, size=(B, K)).astype(np.int32)
    bidx = rng.integers(0, R, size=(B, K)).astype(np.int32)
    widx[:, 6:] = -1
    us = rng.integers(0, 2, size=(B, 1)).astype(np.float32)
    them = (1.0 - us).astype(np.float32)
    psqt_idx = np.zeros(B, np.int64)
    nat, lib = _native()
    l0 = torch.empty(B, L1, device=_dev())
    wp = torch.empty(B, 1, device=_dev())
    bp = torch.empty(B, 1, device=_dev())
    saved = torch.empty(2, B, L1, device=_dev())
    nbytes = lib.nnueft_fwd_workspace_bytes(B, K, R, L1, 0)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=_dev())
    W, bias = _t(c["W"]), _t(c["bias"])
    d_us, d_them, d_w, d_b, d_p = _t(us), _t(them), _t(widx), _t(bidx), _t(psqt_idx)
    nat.check(lib.nnueft_double_fwd(d_us.data_ptr(), d_them.data_ptr(), d_w.data_ptr(), d_b.data_ptr(),
                                    d_p.data_ptr(), W.data_ptr(), bias.data_ptr(), c["max_act"], l0.data_ptr(),
                                    wp.data_ptr(), bp.data_ptr(), saved.data_ptr(), B, K, R, L1, 0, ws.data_ptr(), nbytes,
                                    _stream()), "double_fwd")
    r_l0, r_wp, r_bp, r_saved = oracle_cpu.double_fwd(us, them, widx, bidx, psqt_idx, c["W"], c["bias"], c["max_act"], L1)
    assert np.array_equal(l0.cpu().numpy(), r_l0)
    assert np.array_equal(saved.cpu().numpy(), r_saved)
    # the atomic adds in LDS tiles walk the same tables: this batch is beyond them too
    assert lib.nnueft_atomic_lds_workspace_bytes(B, K, R, L1, 2) == 0


@pytest.mark.parametrize("mode", ["atomic", "atomic_lds", "deterministic"])
@pytest.mark.parametrize("B,L1,R,K,kw", DOUBLE_SHAPES)
def test_double_backward(oracle_cpu, B, L1, R, K, kw, mode):
    c = double_case(500 + B, B, L1, R, K, **kw)
    nat, lib = _native()
    n_psqt = c["n_psqt"]
    out_cols = L1 + n_psqt
    d, l0, wp, bp, saved = _run_double_fwd(c)
    g_l0, g_wp, g_bp = _t(c["g_l0"]), _t(c["g_wp"]), _t(c["g_bp"])
    head = (d["us"].data_ptr(), d["them"].data_ptr(), d["widx"].data_ptr(), d["bidx"].data_ptr(),
            d["psqt_idx"].data_ptr(), d["bias"].data_ptr(), c["max_act"], g_l0.data_ptr(), g_wp.data_ptr(),
            g_bp.data_ptr(), saved.data_ptr())
    if mode == "atomic":
        gW = torch.zeros(R, out_cols, device=_dev())
        gb = torch.zeros(out_cols, device=_dev())
        nat.check(lib.nnueft_double_bwd_atomic(*head, gW.data_ptr(), gb.data_ptr(), B, K, R, L1, n_psqt, _stream()),
                  "double_bwd_atomic")
    elif mode == "atomic_lds":
        # the atomic adds in LDS tiles: every element written, twice on one workspace; shapes it does not
        # take (lists longer than 32 slots, rows that are not whole 16-byte vectors) say so
        nbytes = lib.nnueft_atomic_lds_workspace_bytes(B, K, R, out_cols, 2)
        ws = torch.full((max(nbytes, 256),), 0xA5, dtype=torch.uint8, device=_dev())
        for _ in range(2):
            gW = torch.full((R, out_cols), float("nan"), device=_dev())
            gb = torch.full((out_cols,), float("nan"), device=_dev())
            rc = lib.nnueft_double_bwd_atomic_lds(*head, gW.data_ptr(), gb.data_ptr(), B, K, R, L1, n_psqt, ws.data_ptr(),
                                                  ws.numel(), _stream())
            if nbytes == 0:
                assert rc == nat.E_UNSUPPORTED and (K > 32 or out_cols % 4 or R > 62 * 768)
                return
            nat.check(rc, "double_bwd_atomic_lds")
    else:
        nbytes = lib.nnueft_det_workspace_bytes(B, K, R, out_cols, 2, RS(lib))
        ws = torch.empty(nbytes, dtype=torch.uint8, device=_dev())
        gW = torch.full((R, out_cols), float("nan"), device=_dev())
        gb = torch.full((out_cols,), float("nan"), device=_dev())
        nat.check(lib.nnueft_double_bwd_det(*head, gW.data_ptr(), gb.data_ptr(), B, K, R, L1, n_psqt, RS(lib), ws.data_ptr(),
                                            nbytes, None, _stream(), None), "double_bwd_det")
        # the same with the sort on a second stream
        gW2 = torch.full((R, out_cols), float("nan"), device=_dev())
        gb2 = torch.full((out_cols,), float("nan"), device=_dev())
        aux = torch.cuda.Stream()
        nat.check(lib.nnueft_double_bwd_det(*head, gW2.data_ptr(), gb2.data_ptr(), B, K, R, L1, n_psqt, RS(lib), ws.data_ptr(),
                                            nbytes, None, _stream(), aux.cuda_stream), "double_bwd_det")
        assert torch.equal(gW, gW2) and torch.equal(gb, gb2)
        # the same with lists sorted beforehand, used twice
        # (the block holds what a sort for any threshold writes: for the strict order also the tables of the
        # reduction out of LDS tiles, which a workspace for another threshold has no room for)
        sbytes = lib.nnueft_det_sort_bytes(B, K, R, out_cols, 2)
        assert 0 < sbytes < lib.nnueft_det_workspace_bytes(B, K, R, out_cols, 2, 0)
        lists = torch.full((sbytes,), 0x5A, dtype=torch.uint8, device=_dev())
        nat.check(lib.nnueft_det_sort(d["widx"].data_ptr(), d["bidx"].data_ptr(), B, K, R, out_cols, 2, RS(lib),
                                      lists.data_ptr(), sbytes, _stream()), "det_sort")
        for _ in range(2):
            gW2.fill_(float("nan"))
            gb2.fill_(float("nan"))
            ws.fill_(0xC3)
            nat.check(lib.nnueft_double_bwd_det(*head, gW2.data_ptr(), gb2.data_ptr(), B, K, R, L1, n_psqt, RS(lib),
                                                ws.data_ptr(), nbytes, lists.data_ptr(), _stream(), None),
                      "double_bwd_det")
            assert torch.equal(gW, gW2) and torch.equal(gb, gb2)
    rW, rb = oracle_cpu.double_bwd(c["us"], c["them"], c["widx"], c["bidx"], c["psqt_idx"], c["bias"], c["max_act"],
                                   c["g_l0"], c["g_wp"], c["g_bp"], saved.cpu().numpy(), R, n_psqt, row_split=_RS_OVERRIDE)
    gW, gb = gW.cpu().numpy(), gb.cpu().numpy()
    if mode == "atomic":
        assert _rel_err(gW, rW) <= 1e-4
        assert _rel_err(gb, rb) <= 1e-4
    elif mode == "atomic_lds":
        assert _rel_err(gW, rW) <= 1e-4
        assert np.array_equal(gb, rb)   # its bias gradient is the deterministic one
    else:
        assert np.array_equal(gW, rW)
        assert np.array_equal(gb, rb)


# Batches in which a few table rows are named by a large part of the positions (as in game data,
# where most kings stand on their castled squares): rows beyond nnueft_row_split() slots are summed
# window by window, several windows at these sizes.
def _skewed_double_case(seed, B, L1, castled, fold=0):
    """castled < 0: game-like positions; else that share of the kings on g1 / g8."""
    from nnueft import halfka_v2_hm as hk

    c = double_case(seed, B, L1, hk.NUM_INPUTS, 32, halfka=True, weight_scale=0.05, max_act=255 / 256)
    us, them, widx, bidx, pc = hk.synthetic_batch(B, seed, castled_kings=castled, game_like=castled < 0)
    if fold:
        # crowd every king bucket's features onto its first `fold` rows (lists then hold duplicates)
        for ix in (widx, bidx):
            v = ix >= 0
            ix[v] = ix[v] // hk.NUM_PLANES * hk.NUM_PLANES + ix[v] % hk.NUM_PLANES % fold
    c.update(us=us, them=them, widx=widx, bidx=bidx, psqt_idx=((pc - 1) // 4).astype(np.int64))
    return c


# (the last case is wide and crowded enough for the XCDs that own the crowded king buckets to walk their row
# ranges in 64-lane slices)
@pytest.mark.parametrize("B,L1,castled,fold", [(4096, 64, 1.0, 0), (6000, 256, 0.6, 96), (16384, 128, 0.5, 200),
                                                (3000, 1024, 0.9, 40), (16384, 64, -1, 0), (5000, 3072, -1, 0),
                                                (16384, 1024, -1, 0)])
def test_double_backward_deterministic_with_split_rows(oracle_cpu, row_split, B, L1, castled, fold):
    c = _skewed_double_case(900 + B, B, L1, castled, fold)
    nat, lib = _native()
    R, K, n_psqt = c["R"], c["K"], c["n_psqt"]
    out_cols = L1 + n_psqt
    counts = np.bincount(np.concatenate([c["widx"][c["widx"] >= 0], c["bidx"][c["bidx"] >= 0]]), minlength=R)
    assert (counts > lib.nnueft_row_split()).sum() >= (8 if fold else 2) and B > lib.nnueft_row_window(B)
    d, l0, wp, bp, saved = _run_double_fwd(c)
    g_l0, g_wp, g_bp = _t(c["g_l0"]), _t(c["g_wp"]), _t(c["g_bp"])
    nbytes = lib.nnueft_det_workspace_bytes(B, K, R, out_cols, 2, RS(lib))
    ws = torch.empty(nbytes, dtype=torch.uint8, device=_dev())
    gW = torch.full((R, out_cols), float("nan"), device=_dev())
    gb = torch.full((out_cols,), float("nan"), device=_dev())
    nat.check(lib.nnueft_double_bwd_det(d["us"].data_ptr(), d["them"].data_ptr(), d["widx"].data_ptr(),
                                        d["bidx"].data_ptr(), d["psqt_idx"].data_ptr(), d["bias"].data_ptr(),
                                        c["max_act"], g_l0.data_ptr(), g_wp.data_ptr(), g_bp.data_ptr(),
                                        saved.data_ptr(), gW.data_ptr(), gb.data_ptr(), B, K, R, L1, n_psqt, RS(lib),
                                        ws.data_ptr(), nbytes, None, _stream(), torch.cuda.Stream().cuda_stream),
              "double_bwd_det")
    rW, rb = oracle_cpu.double_bwd(c["us"], c["them"], c["widx"], c["bidx"], c["psqt_idx"], c["bias"], c["max_act"],
                                   c["g_l0"], c["g_wp"], c["g_bp"], saved.cpu().numpy(), R, n_psqt, row_split=_RS_OVERRIDE)
    assert np.array_equal(gW.cpu().numpy(), rW)
    assert np.array_equal(gb.cpu().numpy(), rb)
    # lists sorted beforehand: same bits, also on the second use of the sorted block
    sbytes = lib.nnueft_det_sort_bytes(B, K, R, out_cols, 2)
    lists = torch.empty(sbytes, dtype=torch.uint8, device=_dev())
    nat.check(lib.nnueft_det_sort(d["widx"].data_ptr(), d["bidx"].data_ptr(), B, K, R, out_cols, 2, RS(lib),
                                  lists.data_ptr(), sbytes, _stream()), "det_sort")
    for _ in range(2):
        gW2 = torch.full((R, out_cols), float("nan"), device=_dev())
        gb2 = torch.full((out_cols,), float("nan"), device=_dev())
        nat.check(lib.nnueft_double_bwd_det(d["us"].data_ptr(), d["them"].data_ptr(), d["widx"].data_ptr(),
                                            d["bidx"].data_ptr(), d["psqt_idx"].data_ptr(), d["bias"].data_ptr(),
                                            c["max_act"], g_l0.data_ptr(), g_wp.data_ptr(), g_bp.data_ptr(),
                                            saved.data_ptr(), gW2.data_ptr(), gb2.data_ptr(), B, K, R, L1, n_psqt, RS(lib),
                                            ws.data_ptr(), nbytes, lists.data_ptr(), _stream(), None),
                  "double_bwd_det")
        assert torch.equal(gW, gW2) and torch.equal(gb, gb2)


# (the last two tables are taller than the row scan stages at once: several passes, totals summed first)
@pytest.mark.parametrize("B,out_cols,R,K", [(5000, 72, 40, 16), (9000, 37, 300, 8), (20000, 264, 64, 4),
                                            (3000, 8, 70001, 8), (2500, 12, 40000, 16)])
def test_sparse_backward_deterministic_with_split_rows(oracle_cpu, row_split, B, out_cols, R, K):
    c = sparse_case(950 + B, B, out_cols, R, K, allow_holes=True)
    rng = np.random.default_rng(B)
    c["idx"][rng.random((B, K)) < 0.3] = 3      # one row named by a third of all slots
    nat, lib = _native()
    assert B > lib.nnueft_row_window(B)
    idx, g = _t(c["idx"]), _t(c["g"])
    nbytes = lib.nnueft_det_workspace_bytes(B, K, R, out_cols, 1, RS(lib))
    ws = torch.empty(nbytes, dtype=torch.uint8, device=_dev())
    gW = torch.full((R, out_cols), float("nan"), device=_dev())
    gb = torch.full((out_cols,), float("nan"), device=_dev())
    nat.check(lib.nnueft_sparse_bwd_det(idx.data_ptr(), g.data_ptr(), gW.data_ptr(), gb.data_ptr(), B, K, R,
                                        out_cols, RS(lib), ws.data_ptr(), nbytes, _stream()), "sparse_bwd_det")
    rW, rb = oracle_cpu.sparse_bwd(c["idx"], c["g"], R, row_split=_RS_OVERRIDE)
    assert np.array_equal(gW.cpu().numpy(), rW)
    assert np.array_equal(gb.cpu().numpy(), rb)


def _strict_tile_lists(kind, B, R, K, rng):
    """Index lists for the strict order's reduction out of LDS tiles (every list inside one 768-row block)."""
    nblocks = (R + 767) // 768

    def lists(blocks, n_valid):
        out = np.full((B, K), -1, np.int32)
        for b in range(B):
            rows_here = min(768, R - blocks[b] * 768)
            out[b, :n_valid[b]] = blocks[b] * 768 + rng.choice(rows_here, size=n_valid[b], replace=False)
        return out

    n_valid = rng.integers(1, K + 1, size=B)
    if kind == "one_block":
        # several chunks of 624 pairs for either perspective: the chains go from chunk to chunk through LDS, the
        # white sums wait in the gradient while the black ones are made
        w, b = lists(np.full(B, 1), n_valid), lists(np.full(B, 1), n_valid[::-1])
        w[:, 0] = 768 + 5     # a row that every white list names (summed without a list)
        for ix in (w, b):     # ... entered once only
            for r in range(B):
                dup = np.flatnonzero(ix[r, 1:] == ix[r, 0]) + 1
                ix[r, dup] = -1
    elif kind == "white_heavy":
        # one block with many white chunks and a single black one; other blocks with black pairs only
        w, b = lists(np.full(B, 0), n_valid), lists(rng.integers(0, nblocks, size=B), n_valid)
    elif kind == "last_block":
        # a table whose last block is short, blocks without any pair, an empty list
        blocks = rng.choice([0, nblocks - 1], size=B)
        w, b = lists(blocks, n_valid), lists(blocks[::-1], n_valid)
        w[3] = -1
    elif kind == "two_blocks_in_a_list":
        w, b = lists(rng.integers(0, nblocks, size=B), n_valid), lists(rng.integers(0, nblocks, size=B), n_valid)
        w[B // 2, :2] = (5, 768 * (nblocks - 1) + 1)     # left to the segmented reduction, all of the batch
    elif kind == "a_row_twice":
        w, b = lists(rng.integers(0, nblocks, size=B), n_valid), lists(rng.integers(0, nblocks, size=B), n_valid)
        b[B // 3, :2] = b[B // 3, 0]
    else:
        raise ValueError(kind)
    return w, b


@pytest.mark.parametrize("kind,B,L1,R", [("one_block", 2100, 256, 2000), ("white_heavy", 1500, 512, 3000),
                                         ("last_block", 700, 264, 768 * 3 + 100), ("two_blocks_in_a_list", 900, 256, 2400),
                                         ("a_row_twice", 900, 256, 2400)])
def test_double_backward_strict_order_out_of_lds_tiles(oracle_cpu, kind, B, L1, R):
    """Rows of 256 columns and more, lists of up to 32 slots, strict order: the chains are summed out of LDS tiles."""
    K, n_psqt = 32, 8
    rng = np.random.default_rng(len(kind) * 1000 + B)
    c = double_case(1300 + B, B, L1, R, K, binary_side=True)
    c["widx"], c["bidx"] = _strict_tile_lists(kind, B, R, K, rng)
    nat, lib = _native()
    out_cols = L1 + n_psqt
    d, l0, wp, bp, saved = _run_double_fwd(c)
    g_l0, g_wp, g_bp = _t(c["g_l0"]), _t(c["g_wp"]), _t(c["g_bp"])
    head = (d["us"].data_ptr(), d["them"].data_ptr(), d["widx"].data_ptr(), d["bidx"].data_ptr(),
            d["psqt_idx"].data_ptr(), d["bias"].data_ptr(), c["max_act"], g_l0.data_ptr(), g_wp.data_ptr(),
            g_bp.data_ptr(), saved.data_ptr())
    nbytes = lib.nnueft_det_workspace_bytes(B, K, R, out_cols, 2, 0)
    ws = torch.full((nbytes,), 0x3C, dtype=torch.uint8, device=_dev())
    rW, rb = oracle_cpu.double_bwd(c["us"], c["them"], c["widx"], c["bidx"], c["psqt_idx"], c["bias"], c["max_act"],
                                   c["g_l0"], c["g_wp"], c["g_bp"], saved.cpu().numpy(), R, n_psqt, row_split=0)
    # a gradient at a 16-byte boundary, and one 4 bytes past it (stored a float at a time)
    flat = torch.full((R * out_cols + 1,), float("nan"), device=_dev())
    for gW in (flat[:R * out_cols].view(R, out_cols), flat[1:].view(R, out_cols)):
        gb = torch.full((out_cols,), float("nan"), device=_dev())
        nat.check(lib.nnueft_double_bwd_det(*head, gW.data_ptr(), gb.data_ptr(), B, K, R, L1, n_psqt, 0, ws.data_ptr(),
                                            nbytes, None, _stream(), None), "double_bwd_det")
        assert np.array_equal(gW.cpu().numpy(), rW)
        assert np.array_equal(gb.cpu().numpy(), rb)
        flat.fill_(float("nan"))
    # lists sorted beforehand, used twice (the reduction leaves its counters as it found them)
    sbytes = lib.nnueft_det_sort_bytes(B, K, R, out_cols, 2)
    lists = torch.full((sbytes,), 0x5A, dtype=torch.uint8, device=_dev())
    nat.check(lib.nnueft_det_sort(d["widx"].data_ptr(), d["bidx"].data_ptr(), B, K, R, out_cols, 2, 0,
                                  lists.data_ptr(), sbytes, _stream()), "det_sort")
    gW = torch.empty(R, out_cols, device=_dev())
    for _ in range(2):
        gW.fill_(float("nan"))
        gb = torch.full((out_cols,), float("nan"), device=_dev())
        nat.check(lib.nnueft_double_bwd_det(*head, gW.data_ptr(), gb.data_ptr(), B, K, R, L1, n_psqt, 0, ws.data_ptr(),
                                            nbytes, lists.data_ptr(), _stream(), None), "double_bwd_det")
        assert np.array_equal(gW.cpu().numpy(), rW)
        assert np.array_equal(gb.cpu().numpy(), rb)


def test_deterministic_backward_repeats_bitwise():
    """Two runs of the deterministic backward give the same bits (the atomic one need not)."""
    c = double_case(77, 300, 256, 600, 32, binary_side=True)
    nat, lib = _native()
    B, K, R, L1, n_psqt = 300, 32, 600, 256, 8
    d, l0, wp, bp, saved = _run_double_fwd(c)
    g_l0, g_wp, g_bp = _t(c["g_l0"]), _t(c["g_wp"]), _t(c["g_bp"])
    nbytes = lib.nnueft_det_workspace_bytes(B, K, R, L1 + n_psqt, 2, RS(lib))
    outs = []
    for fill in (0.0, 123.0):
        ws = torch.full((nbytes,), int(fill) % 251, dtype=torch.uint8, device=_dev())
        gW = torch.empty(R, L1 + n_psqt, device=_dev())
        gb = torch.empty(L1 + n_psqt, device=_dev())
        nat.check(lib.nnueft_double_bwd_det(d["us"].data_ptr(), d["them"].data_ptr(), d["widx"].data_ptr(),
                                            d["bidx"].data_ptr(), d["psqt_idx"].data_ptr(), d["bias"].data_ptr(),
                                            c["max_act"],
                                            g_l0.data_ptr(), g_wp.data_ptr(), g_bp.data_ptr(), saved.data_ptr(),
                                            gW.data_ptr(), gb.data_ptr(), B, K, R, L1, n_psqt, RS(lib), ws.data_ptr(), nbytes,
                                            None, _stream(), None), "double_bwd_det")
        outs.append((gW.cpu().numpy().copy(), gb.cpu().numpy().copy()))
    assert np.array_equal(outs[0][0], outs[1][0])
    assert np.array_equal(outs[0][1], outs[1][1])


@pytest.mark.parametrize("B,L1", [(700, 1024), (3000, 512), (64, 3072)])
def test_int16_forward_on_exported_lists(oracle_cpu, B, L1):
    """Lists as the loader makes them for an exported net (22528 rows, king buckets of 704 rows, every list inside
    one bucket): with a workspace the sums come out of LDS tiles of the int16 table (3000 positions: several
    chunks of lists per bucket)."""
    from nnueft import halfka_v2_hm as hk
    from nnueft.quantized import ft_int16_forward

    rng = np.random.default_rng(640 + B)
    R = hk.NUM_INPUTS_EXPORT
    us, _, widx, bidx, _ = hk.synthetic_batch(B, 77 + B, fold_kings=True)
    stm = (1 - us[:, 0]).astype(np.uint8)
    W16 = rng.integers(-3000, 3000, size=(R, L1)).astype(np.int16)
    W16[:, : L1 // 3] = rng.integers(-40, 60, size=(R, L1 // 3)).astype(np.int16)
    b16 = rng.integers(-200, 400, size=L1).astype(np.int16)
    psqt32 = rng.integers(-100000, 100000, size=(R, 8)).astype(np.int32)
    psqt_idx = rng.integers(0, 8, size=B).astype(np.int64)
    r_out, r_ps = oracle_cpu.ft_int16_fwd(widx, bidx, stm, W16, b16, psqt32, psqt_idx, 255, 9)
    for use_workspace in (True, False):
        out, ps = ft_int16_forward(_t(widx), _t(bidx), _t(stm), _t(W16), _t(b16), _t(psqt32), _t(psqt_idx), 255, 9,
                                   use_workspace=use_workspace)
        assert np.array_equal(out.cpu().numpy(), r_out)
        assert np.array_equal(ps.cpu().numpy(), r_ps)


INT16_SHAPES = [(5, 32, 50, 32), (33, 1024, 22528, 32), (17, 3072, 22528, 32), (9, 38, 40, 70)]


@pytest.mark.parametrize("use_workspace", [False, True], ids=["plain", "l2blocked"])
@pytest.mark.parametrize("B,L1,R,K", INT16_SHAPES)
@pytest.mark.parametrize("clip_max,shift", [(255, 9), (127, 7)])
def test_int16_forward(oracle_cpu, B, L1, R, K, clip_max, shift, use_workspace):
    rng = np.random.default_rng(600 + B)
    from _cases import random_lists

    widx = random_lists(rng, B, K, R, allow_holes=True)
    bidx = random_lists(rng, B, K, R, allow_holes=True)
    stm = rng.integers(0, 2, size=B).astype(np.uint8)
    # large enough that some accumulators wrap around int16
    W16 = rng.integers(-3000, 3000, size=(R, L1)).astype(np.int16)
    W16[:, : L1 // 3] = rng.integers(-40, 60, size=(R, L1 // 3)).astype(np.int16)
    b16 = rng.integers(-200, 400, size=L1).astype(np.int16)
    psqt32 = rng.integers(-100000, 100000, size=(R, 8)).astype(np.int32)
    psqt_idx = rng.integers(0, 8, size=B).astype(np.int64)
    from nnueft.quantized import ft_int16_forward

    out, ps = ft_int16_forward(_t(widx), _t(bidx), _t(stm), _t(W16), _t(b16), _t(psqt32), _t(psqt_idx), clip_max, shift,
                               use_workspace=use_workspace)
    r_out, r_ps = oracle_cpu.ft_int16_fwd(widx, bidx, stm, W16, b16, psqt32, psqt_idx, clip_max, shift)
    assert np.array_equal(out.cpu().numpy(), r_out)
    assert np.array_equal(ps.cpu().numpy(), r_ps)
