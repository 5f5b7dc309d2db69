"""Pins the CPU oracle (oracle/nnueft_oracle.c) without any GPU.

Each check is chosen so that a plausible mistake (a dropped term, a wrong index, swapped
perspectives, a wrong clamp mask, the wrong half paired) fails it:
  * closed forms: the dense count-matrix product the reference's own test uses
    (tests/test_feature_transformer.py:14-32), exact on integer-valued data;
  * the same torch library calls the reference's CPU path makes (embedding_bag, autograd),
    compared for equality of bits;
  * brute force in Python integers for the quantized path, and its agreement with the float path
    on inputs where no rounding can occur;
  * special cases with a known answer.
"""
import numpy as np
import pytest
import torch

from _cases import double_case, random_lists, sparse_case
from oracle import ref_torch


def count_matrix(idx, R):
    B, K = idx.shape
    C = np.zeros((B, R), np.float64)
    for b in range(B):
        for k in range(K):
            if 0 <= idx[b, k] < R:
                C[b, idx[b, k]] += 1.0
    return C


# ------------------------------------------------------------------ sparse linear

def test_sparse_forward_closed_form_exact_on_integers(oracle_cpu):
    rng = np.random.default_rng(0)
    B, K, R, oc = 16, 32, 10, 128          # duplicates are certain with R = 10
    idx = random_lists(rng, B, K, R, allow_holes=True)
    W = rng.integers(-50, 50, size=(R, oc)).astype(np.float32)
    bias = rng.integers(-50, 50, size=oc).astype(np.float32)
    out = oracle_cpu.sparse_fwd(idx, W, bias)
    ref = count_matrix(idx, R) @ W.astype(np.float64) + bias
    assert np.array_equal(out.astype(np.float64), ref)


def test_sparse_forward_matches_dense_emulation_to_reference_tolerance(oracle_cpu):
    # shapes, seeds and tolerance of tests/test_feature_transformer.py:35-72
    torch.manual_seed(0)
    W = torch.rand(10, 128)
    bias = torch.rand(128)
    idx = (torch.rand(16, 32) * 10).to(torch.int32)
    out = oracle_cpu.sparse_fwd(idx.numpy(), W.numpy(), bias.numpy())
    ref = count_matrix(idx.numpy(), 10) @ W.numpy().astype(np.float64) + bias.numpy()
    assert np.abs(out - ref).max() < 1e-4


def test_sparse_forward_padding_contributes_nothing(oracle_cpu):
    # tests/test_feature_transformer.py:81-110
    torch.manual_seed(42)
    W = torch.rand(10, 64).numpy()
    bias = torch.rand(64).numpy()
    active = (torch.rand(8, 5) * 10).to(torch.int32).numpy()
    padded = np.concatenate([active, np.full((8, 3), -1, np.int32)], axis=1)
    assert np.array_equal(oracle_cpu.sparse_fwd(active, W, bias), oracle_cpu.sparse_fwd(padded, W, bias))
    # a hole in the middle and an index past the table are ignored as well
    holes = np.concatenate([active[:, :2], np.full((8, 1), -1, np.int32), active[:, 2:],
                            np.full((8, 1), 10, np.int32)], axis=1)
    assert np.array_equal(oracle_cpu.sparse_fwd(active, W, bias), oracle_cpu.sparse_fwd(holes, W, bias))


@pytest.mark.parametrize("B,oc,R,K", [(16, 128, 10, 32), (257, 40, 300, 32), (64, 1032, 500, 32)])
def test_sparse_forward_bits_equal_torch_cpu_path(oracle_cpu, B, oc, R, K):
    c = sparse_case(11, B, oc, R, K)
    out = oracle_cpu.sparse_fwd(c["idx"], c["W"], c["bias"])
    ref = ref_torch.sparse_linear(torch.from_numpy(c["idx"]), torch.from_numpy(c["W"]), torch.from_numpy(c["bias"]))
    assert np.array_equal(out, ref.numpy())


def test_sparse_backward_closed_form_exact_on_integers(oracle_cpu):
    rng = np.random.default_rng(1)
    B, K, R, oc = 70, 32, 12, 48
    idx = random_lists(rng, B, K, R, allow_holes=True)
    g = rng.integers(-20, 20, size=(B, oc)).astype(np.float32)
    gW, gb = oracle_cpu.sparse_bwd(idx, g, R)
    C = count_matrix(idx, R)
    assert np.array_equal(gW.astype(np.float64), C.T @ g.astype(np.float64))
    assert np.array_equal(gb.astype(np.float64), g.astype(np.float64).sum(0))


# torch's CPU embedding_bag backward sorts the flat index list; from 32768 slots on that sort is a
# stable radix sort and the accumulation order is ascending (position, slot) -- the oracle's order.
# Below that size torch uses an unstable sort, its own order is unspecified, and only closeness holds.
@pytest.mark.parametrize("B,oc,R,K", [(1024, 128, 10, 32), (2048, 40, 300, 32), (512, 24, 50, 64)])
def test_sparse_backward_weight_bits_equal_torch_cpu_autograd(oracle_cpu, B, oc, R, K):
    assert B * K >= 32768
    c = sparse_case(12, B, oc, R, K)
    W = torch.from_numpy(c["W"]).requires_grad_()
    bias = torch.from_numpy(c["bias"]).requires_grad_()
    ref_torch.sparse_linear(torch.from_numpy(c["idx"]), W, bias).backward(torch.from_numpy(c["g"]))
    gW, gb = oracle_cpu.sparse_bwd(c["idx"], c["g"], R)
    assert np.array_equal(gW, W.grad.numpy())
    # torch reduces the bias gradient in its own order: equal to rounding only
    assert np.allclose(gb, bias.grad.numpy(), rtol=1e-4, atol=1e-4)
    # rows no slot names are exactly zero
    named = np.zeros(R, bool)
    named[c["idx"][c["idx"] >= 0]] = True
    assert not gW[~named].any()


# ---------------------------------------------------------------------------------------------
# Rows named by more than row_split() slots: summed window by window.  The checks below fix that
# order through sums whose value under each candidate order is known in closed form: in fp32,
# 2**24 + 1 rounds back to 2**24, so a chain that starts with 2**24 loses every following 1.0,
# while ones collected in another window first arrive as one exact integer.
BIG = float(2 ** 24)


def test_row_window_lengths(oracle_cpu):
    assert oracle_cpu.row_split() == 512
    # one window up to 1024 positions, then as few as keep each at 1024 or fewer, at most 16, multiples of 128
    assert [oracle_cpu.row_window(B) for B in (1, 100, 1024, 2048, 2049, 4096, 8192, 16384, 16385, 65536, 100000)] == \
        [128, 128, 1024, 1024, 768, 1024, 1024, 1024, 1152, 4096, 6272]


def _ones_after_big(B, K, R, row, positions):
    """Lists in which `row` is named once by each of `positions`; upstream rows 2**24 at position 0, else 1."""
    idx = np.full((B, K), -1, np.int32)
    idx[positions, 0] = row
    g = np.ones((B, 1), np.float32)
    g[0, 0] = BIG
    return idx, g


def test_sparse_backward_split_row_sums_windows_separately(oracle_cpu):
    B, K, R = 4096, 2, 5
    W = oracle_cpu.row_window(B)
    assert W == 1024
    # 600 slots > row_split: position 0 (2**24), 299 ones in window 0, 300 ones in window 1
    pos = np.r_[0:300, W:W + 300]
    idx, g = _ones_after_big(B, K, R, 3, pos)
    gW, _ = oracle_cpu.sparse_bwd(idx, g, R)
    # window 0 chain: 2**24 swallows its 299 ones; window 1: exactly 300; chain over windows: 2**24 + 300
    assert gW[3, 0] == BIG + 300.0
    # the same slots, one fewer than the threshold allows splitting: a plain chain, every 1.0 lost
    pos = np.r_[0:256, W:W + 256]
    assert len(pos) == oracle_cpu.row_split()
    idx, g = _ones_after_big(B, K, R, 3, pos)
    gW, _ = oracle_cpu.sparse_bwd(idx, g, R)
    assert gW[3, 0] == BIG
    # one slot more: split
    pos = np.r_[0:256, W:W + 257 + 1]
    idx, g = _ones_after_big(B, K, R, 3, pos)
    gW, _ = oracle_cpu.sparse_bwd(idx, g, R)
    assert gW[3, 0] == BIG + 258.0


def test_sparse_backward_split_row_window_sums_are_chained_in_order(oracle_cpu):
    B, K, R = 8192, 1, 2
    W = oracle_cpu.row_window(B)
    assert W == 1024
    # windows 0..3 hold 2**24, 200 ones, 200 ones, 200 ones: ((2**24 + 200) + 200) + 200, all exact
    pos = np.r_[0:1, W:W + 200, 2 * W:2 * W + 200, 3 * W:3 * W + 200]
    idx, g = _ones_after_big(B, K, R, 1, pos)
    gW, _ = oracle_cpu.sparse_bwd(idx, g, R)
    assert gW[1, 0] == BIG + 600.0
    # a window sum of 1 is lost against 2**24 wherever it comes after it, kept (as part of 201) before
    g2 = g.copy()
    g2[0, 0] = 1.0
    g2[3 * W, 0] = BIG          # the big addend now opens the last window
    gW, _ = oracle_cpu.sparse_bwd(idx, g2, R)
    # window sums 1, 200, 200, (2**24 then 199 ones lost) -> 401 + 2**24: odd, ties to even = 2**24 + 400
    assert gW[1, 0] == BIG + 400.0


def test_sparse_backward_split_rows_exact_on_integers_and_others_untouched(oracle_cpu):
    rng = np.random.default_rng(5)
    B, K, R, oc = 6000, 8, 40, 24
    idx = random_lists(rng, B, K, R, allow_holes=True)
    idx[rng.random((B, K)) < 0.5] = 7            # row 7: ~24000 slots, far beyond the threshold
    g_int = rng.integers(-8, 8, size=(B, oc)).astype(np.float32)
    gW, gb = oracle_cpu.sparse_bwd(idx, g_int, R)
    C = count_matrix(idx, R)
    assert np.array_equal(gW.astype(np.float64), C.T @ g_int.astype(np.float64))
    # real-valued upstream rows: the split rows agree with a float64 sum to rounding, and rows
    # below the threshold keep the plain chain (checked against a chain written out here)
    g = rng.standard_normal((B, oc)).astype(np.float32)
    gW, _ = oracle_cpu.sparse_bwd(idx, g, R)
    ref = C.T @ g.astype(np.float64)
    assert np.allclose(gW, ref, rtol=1e-4, atol=1e-3)
    counts = C.sum(0)
    small = int(np.argmin(np.where(counts > 0, counts, 1 << 30)))
    assert 0 < counts[small] <= oracle_cpu.row_split()
    chain = np.zeros(oc, np.float32)
    for b in range(B):
        for k in range(K):
            if idx[b, k] == small:
                chain = chain + g[b]
    assert np.array_equal(gW[small], chain)


def test_double_backward_split_counts_both_perspectives_together(oracle_cpu):
    # row 2 is named by 300 white and 302 black slots: neither list alone exceeds row_split, together
    # they do.  The PSQT column passes grad_wpsqt / grad_bpsqt straight to the table row.
    B, K, R, L1, n_psqt = 4096, 2, 4, 8, 2
    W = oracle_cpu.row_window(B)
    widx = np.full((B, K), -1, np.int32)
    bidx = np.full((B, K), -1, np.int32)
    widx[np.r_[0:1, W:W + 299], 0] = 2         # white: 2**24 in window 0, 299 ones in window 1
    bidx[np.r_[0:1, W:W + 301], 0] = 2         # black: 1 in window 0, 301 ones in window 1
    us = np.ones((B, 1), np.float32)
    them = np.zeros((B, 1), np.float32)
    psqt_idx = np.zeros(B, np.int64)
    g_wp = np.ones((B, 1), np.float32)
    g_wp[0, 0] = BIG
    g_bp = np.ones((B, 1), np.float32)
    saved = np.zeros((2, B, L1), np.float32)
    bias = np.zeros(L1 + n_psqt, np.float32)
    g_l0 = np.zeros((B, L1), np.float32)
    gW, _ = oracle_cpu.double_bwd(us, them, widx, bidx, psqt_idx, bias, 127.0, g_l0, g_wp, g_bp, saved, R, n_psqt)
    # split: white = 2**24 + 299 -> odd, ties to even = 2**24 + 300; black = 1 + 301; sum exact
    assert gW[2, L1] == BIG + 300.0 + 302.0
    # with one black slot fewer the row has 601 slots, still split; with the lists cut so the row has
    # 512 slots in all it is not: white plain chain = 2**24 (ones lost), black = plain 212
    widx[:] = -1
    bidx[:] = -1
    widx[np.r_[0:1, W:W + 299], 0] = 2
    bidx[np.r_[0:1, W:W + 211], 0] = 2
    gW, _ = oracle_cpu.double_bwd(us, them, widx, bidx, psqt_idx, bias, 127.0, g_l0, g_wp, g_bp, saved, R, n_psqt)
    assert gW[2, L1] == BIG + 212.0


def test_row_split_argument_selects_the_order(oracle_cpu):
    B, K, R = 4096, 2, 5
    W = oracle_cpu.row_window(B)
    # 600 slots: position 0 carries 2**24, 299 ones follow in window 0, 300 ones in window 1
    pos = np.r_[0:300, W:W + 300]
    idx, g = _ones_after_big(B, K, R, 3, pos)
    # strict order (0) and a threshold the row stays below: one plain chain, every 1.0 lost
    for rs in (0, 600, 3000):
        assert oracle_cpu.sparse_bwd(idx, g, R, row_split=rs)[0][3, 0] == BIG
    # any threshold below the row's slot count splits it, the default included
    for rs in (None, 512, 599, 100, 1):
        assert oracle_cpu.sparse_bwd(idx, g, R, row_split=rs)[0][3, 0] == BIG + 300.0
    # the same for the two-perspective gradient (300 white + 300 black slots, PSQT column)
    widx = np.full((B, K), -1, np.int32)
    bidx = np.full((B, K), -1, np.int32)
    widx[np.r_[0:1, W:W + 299], 0] = 2
    bidx[np.r_[0:1, W:W + 299], 0] = 2
    one, zero = np.ones((B, 1), np.float32), np.zeros((B, 1), np.float32)
    g_wp = np.ones((B, 1), np.float32)
    g_wp[0, 0] = BIG
    args = (one, zero, widx, bidx, np.zeros(B, np.int64), np.zeros(10, np.float32), 127.0, np.zeros((B, 8), np.float32),
            g_wp, one, np.zeros((2, B, 8), np.float32), 4, 2)
    assert oracle_cpu.double_bwd(*args, row_split=0)[0][2, 8] == BIG + 300.0          # white: ones lost; black: 300
    assert oracle_cpu.double_bwd(*args, row_split=599)[0][2, 8] == BIG + 300.0 + 300.0  # white: 2**24 + 299 -> ties to even


@pytest.mark.parametrize("B,oc,R,K", [(4096, 24, 500, 16), (3000, 40, 300, 32)])
def test_strict_order_bits_equal_torch_cpu_autograd_with_crowded_rows(oracle_cpu, B, oc, R, K):
    """row_split = 0 is the reference's CPU path for every row, also for rows named by thousands of slots
    (which the default order sums window by window and therefore rounds differently)."""
    assert B * K >= 32768
    c = sparse_case(14, B, oc, R, K)
    rng = np.random.default_rng(B)
    c["idx"][rng.random((B, K)) < 0.25] = 5          # one row named by a quarter of all slots
    assert (c["idx"] == 5).sum() > 8 * oracle_cpu.row_split()
    W = torch.from_numpy(c["W"]).requires_grad_()
    bias = torch.from_numpy(c["bias"]).requires_grad_()
    ref_torch.sparse_linear(torch.from_numpy(c["idx"]), W, bias).backward(torch.from_numpy(c["g"]))
    strict, _ = oracle_cpu.sparse_bwd(c["idx"], c["g"], R, row_split=0)
    assert np.array_equal(strict, W.grad.numpy())
    windowed, _ = oracle_cpu.sparse_bwd(c["idx"], c["g"], R)
    assert not np.array_equal(windowed[5], strict[5])                  # the crowded row: another order
    assert np.allclose(windowed[5], strict[5], rtol=1e-4, atol=1e-2)    # ... the same sum to rounding (24 000 addends)
    counts = np.bincount(c["idx"][c["idx"] >= 0], minlength=R)
    short = counts <= oracle_cpu.row_split()                           # rows the default order leaves whole
    assert np.array_equal(windowed[short], strict[short])


def test_strict_order_double_bits_equal_torch_cpu_autograd_with_crowded_rows(oracle_cpu):
    from nnueft import halfka_v2_hm as hk

    B, L1, R = 2048, 32, hk.NUM_INPUTS
    c = double_case(23, B, L1, R, 32, halfka=True, weight_scale=0.05, max_act=255 / 256)
    us, them, widx, bidx, pc = hk.synthetic_batch(B, 23, castled_kings=0.9)
    c.update(us=us, them=them, widx=widx, bidx=bidx, psqt_idx=((pc - 1) // 4).astype(np.int64))
    counts = np.bincount(np.concatenate([widx[widx >= 0], bidx[bidx >= 0]]), minlength=R)
    assert counts.max() > 2 * oracle_cpu.row_split() and B * 32 >= 32768
    W, bias, outs = _torch_double(c, need_grad=True)
    torch.autograd.backward(list(outs), [torch.from_numpy(c[k]) for k in ("g_l0", "g_wp", "g_bp")])
    _, _, _, saved = oracle_cpu.double_fwd(us, them, widx, bidx, c["psqt_idx"], c["W"], c["bias"], c["max_act"], L1)
    gW, _ = oracle_cpu.double_bwd(us, them, widx, bidx, c["psqt_idx"], c["bias"], c["max_act"], c["g_l0"], c["g_wp"],
                                  c["g_bp"], saved, R, c["n_psqt"], row_split=0)
    assert np.array_equal(gW, W.grad.numpy())


def test_bias_gradient_tile_order_brute_force(oracle_cpu):
    tile = oracle_cpu.bias_tile()
    rng = np.random.default_rng(2)
    B, oc = 3 * tile + 5, 7
    g = (rng.standard_normal((B, oc)) * 1e3).astype(np.float32)
    idx = np.full((B, 4), -1, np.int32)
    _, gb = oracle_cpu.sparse_bwd(idx, g, 3)
    want = np.zeros(oc, np.float32)
    for c in range(oc):
        total = np.float32(0)
        for t0 in range(0, B, tile):
            part = np.float32(0)
            for b in range(t0, min(t0 + tile, B)):
                part = np.float32(part + g[b, c])
            total = np.float32(total + part)
        want[c] = total
    assert np.array_equal(gb, want)


# ------------------------------------------------------------------ fused double transform

DOUBLE = [
    (4, 32, 100, {}),
    (4, 2048, 100, {}),
    (50, 64, 400, dict(binary_side=True, max_act=255 / 256, weight_scale=0.1)),
    (33, 128, 24576, dict(halfka=True, max_act=255 / 256, weight_scale=0.05)),
]
# backward comparisons for equality of bits need >= 32768 slots per list (see above)
DOUBLE_BIG = [
    (1024, 32, 100, {}),
    (1100, 64, 400, dict(binary_side=True, max_act=255 / 256, weight_scale=0.1)),
    (1024, 128, 24576, dict(halfka=True, max_act=255 / 256, weight_scale=0.05)),
]


def _torch_double(c, need_grad=False):
    W = torch.from_numpy(c["W"]).requires_grad_(need_grad)
    bias = torch.from_numpy(c["bias"]).requires_grad_(need_grad)
    out = ref_torch.double_feature_transform(
        torch.from_numpy(c["us"]), torch.from_numpy(c["them"]), torch.from_numpy(c["widx"]),
        torch.from_numpy(c["bidx"]), torch.from_numpy(c["psqt_idx"]), W, bias, c["max_act"], c["L1"])
    return W, bias, out


@pytest.mark.parametrize("B,L1,R,kw", DOUBLE)
def test_double_forward_bits_equal_torch_cpu_path(oracle_cpu, B, L1, R, kw):
    c = double_case(21, B, L1, R, **kw)
    l0, wp, bp, saved = oracle_cpu.double_fwd(c["us"], c["them"], c["widx"], c["bidx"], c["psqt_idx"], c["W"],
                                              c["bias"], c["max_act"], L1)
    _, _, (t_l0, t_wp, t_bp) = _torch_double(c)
    assert np.array_equal(l0, t_l0.numpy())
    assert np.array_equal(wp, t_wp.numpy())
    assert np.array_equal(bp, t_bp.numpy())
    # `saved` holds the two perspectives' row sums before the bias
    assert saved.shape == (2, B, L1)
    assert np.array_equal(saved[0] + c["bias"][:L1], oracle_cpu.sparse_fwd(c["widx"], c["W"], c["bias"])[:, :L1])
    assert np.array_equal(saved[1] + c["bias"][:L1], oracle_cpu.sparse_fwd(c["bidx"], c["W"], c["bias"])[:, :L1])


@pytest.mark.parametrize("B,L1,R,kw", DOUBLE + DOUBLE_BIG)
def test_double_backward_weight_bits_equal_torch_cpu_autograd(oracle_cpu, B, L1, R, kw):
    c = double_case(22, B, L1, R, **kw)
    W, bias, (t_l0, t_wp, t_bp) = _torch_double(c, need_grad=True)
    torch.autograd.backward([t_l0, t_wp, t_bp],
                            [torch.from_numpy(c["g_l0"]), torch.from_numpy(c["g_wp"]), torch.from_numpy(c["g_bp"])])
    _, _, _, saved = oracle_cpu.double_fwd(c["us"], c["them"], c["widx"], c["bidx"], c["psqt_idx"], c["W"],
                                           c["bias"], c["max_act"], L1)
    gW, gb = oracle_cpu.double_bwd(c["us"], c["them"], c["widx"], c["bidx"], c["psqt_idx"], c["bias"], c["max_act"],
                                   c["g_l0"], c["g_wp"], c["g_bp"], saved, R, c["n_psqt"])
    if B * c["K"] >= 32768:
        assert np.array_equal(gW, W.grad.numpy())
    else:
        # the reference's own tolerance for this comparison, tests/test_fused_double_ft.py:104-107
        assert np.allclose(gW, W.grad.numpy(), atol=1e-4, rtol=1e-3)
    scale = max(np.abs(bias.grad.numpy()).max(), 1.0)
    assert np.abs(gb - bias.grad.numpy()).max() <= 1e-4 * scale


def test_double_special_cases(oracle_cpu):
    rng = np.random.default_rng(3)
    B, L1, R, K, n_psqt = 6, 16, 30, 8, 4
    h = L1 // 2
    W = rng.uniform(0.01, 0.05, size=(R, L1 + n_psqt)).astype(np.float32)
    bias = rng.uniform(0.01, 0.05, size=L1 + n_psqt).astype(np.float32)
    widx = random_lists(rng, B, K, R, min_active=1)
    bidx = random_lists(rng, B, K, R, min_active=1)
    bidx[0, :] = -1                      # a position with an empty black list
    psqt_idx = rng.integers(0, n_psqt, size=B).astype(np.int64)
    one, zero = np.ones((B, 1), np.float32), np.zeros((B, 1), np.float32)
    inf = float("inf")
    # us = 1, them = 0, no upper clamp, positive weights: x_w is the white accumulator itself and
    # l0 is the plain product of its halves; the second half of l0 comes from the black one.
    l0, wp, bp, saved = oracle_cpu.double_fwd(one, zero, widx, bidx, psqt_idx, W, bias, inf, L1)
    w_acc = oracle_cpu.sparse_fwd(widx, W, bias)
    b_acc = oracle_cpu.sparse_fwd(bidx, W, bias)
    assert np.array_equal(l0[:, :h], w_acc[:, :h] * w_acc[:, h:L1])
    assert np.array_equal(l0[:, h:], b_acc[:, :h] * b_acc[:, h:L1])
    assert np.array_equal(wp[:, 0], w_acc[np.arange(B), L1 + psqt_idx])
    assert np.array_equal(bp[:, 0], b_acc[np.arange(B), L1 + psqt_idx])
    assert np.array_equal(b_acc[0], bias)         # empty list: bias only
    # swapping the side to move swaps the two halves of l0
    l0s, _, _, _ = oracle_cpu.double_fwd(zero, one, widx, bidx, psqt_idx, W, bias, inf, L1)
    assert np.array_equal(l0s[:, :h], l0[:, h:]) and np.array_equal(l0s[:, h:], l0[:, :h])
    # swapping the index lists instead does the same and swaps the psqt outputs
    l0x, wpx, bpx, _ = oracle_cpu.double_fwd(one, zero, bidx, widx, psqt_idx, W, bias, inf, L1)
    assert np.array_equal(l0x, l0s) and np.array_equal(wpx, bp) and np.array_equal(bpx, wp)
    # an upper clamp below every accumulator value gives max*max everywhere
    l0c, _, _, _ = oracle_cpu.double_fwd(one, zero, widx, bidx, psqt_idx, W, bias, 0.001, L1)
    assert np.array_equal(l0c, np.full_like(l0c, np.float32(0.001) * np.float32(0.001)))


def test_clamp_gradient_passes_at_the_boundaries_like_torch(oracle_cpu):
    # x exactly 0 and exactly max: torch.clamp passes gradient (0 <= x <= max); the reference's
    # fused kernel would zero it (fused_ft_kernel.py:215-218).  The oracle follows torch.
    B, L1, n_psqt, max_act = 1, 4, 0, 1.0
    # with us = 1, them = 0 and a zero bias the mixed values are the row sums themselves:
    # x_w = (0, 1 | .5, .5) sits on both clamp boundaries, x_b = (-.1, 1.1 | .5, .5) outside them
    saved = np.array([[[0.0, 1.0, 0.5, 0.5]], [[-0.1, 1.1, 0.5, 0.5]]], np.float32)
    g = np.ones((B, L1), np.float32)
    one, zero = np.ones((B, 1), np.float32), np.zeros((B, 1), np.float32)
    G = oracle_cpu.double_bwd_rows(one, zero, np.zeros(B, np.int64), np.zeros(L1, np.float32), max_act, g, zero, zero,
                                   saved, n_psqt)
    # white rows: d/dx_w0 = g*c_w1 where the mask holds: [0.5, 0.5] (both boundary values pass)
    assert np.array_equal(G[0, 0], np.array([0.5, 0.5, 0.0, 1.0], np.float32))
    # black rows: x_b0 = -0.1 and 1.1 are outside: no gradient; x_b1 inside: g*c_b0 = [0, 1]
    assert np.array_equal(G[1, 0], np.array([0.0, 0.0, 0.0, 1.0], np.float32))
    x = torch.tensor(saved[:, 0].reshape(4, 2), requires_grad=True)     # rows: x_w[:h], x_w[h:], x_b[:h], x_b[h:]
    cl = torch.clamp(x, 0.0, max_act)
    torch.cat([cl[0] * cl[1], cl[2] * cl[3]]).backward(torch.ones(4))
    assert np.array_equal(G[0, 0], torch.cat([x.grad[0], x.grad[1]]).numpy())
    assert np.array_equal(G[1, 0], torch.cat([x.grad[2], x.grad[3]]).numpy())


def test_double_backward_invariants(oracle_cpu):
    c = double_case(23, 40, 32, 60, binary_side=True)
    R, L1, n_psqt = 60, 32, 8
    _, _, _, saved = oracle_cpu.double_fwd(c["us"], c["them"], c["widx"], c["bidx"], c["psqt_idx"], c["W"],
                                           c["bias"], c["max_act"], L1)
    G = oracle_cpu.double_bwd_rows(c["us"], c["them"], c["psqt_idx"], c["bias"], c["max_act"], c["g_l0"], c["g_wp"],
                                   c["g_bp"], saved, n_psqt)
    gW, gb = oracle_cpu.double_bwd(c["us"], c["them"], c["widx"], c["bidx"], c["psqt_idx"], c["bias"], c["max_act"],
                                   c["g_l0"], c["g_wp"], c["g_bp"], saved, R, n_psqt)
    # column sums: sum_r gW[r] = sum_b n_w(b) G_w[b] + n_b(b) G_b[b]
    nw = (c["widx"] >= 0).sum(1).astype(np.float64)
    nb = (c["bidx"] >= 0).sum(1).astype(np.float64)
    want = (nw[:, None] * G[0].astype(np.float64)).sum(0) + (nb[:, None] * G[1].astype(np.float64)).sum(0)
    assert np.allclose(gW.astype(np.float64).sum(0), want, rtol=1e-5, atol=1e-4)
    assert np.allclose(gb, (G[0].astype(np.float64) + G[1]).sum(0), rtol=1e-5, atol=1e-4)
    # only the selected psqt column of a position carries gradient
    for b in range(40):
        others = [j for j in range(n_psqt) if j != c["psqt_idx"][b]]
        assert not G[:, b, L1 + np.array(others)].any()
        assert G[0, b, L1 + c["psqt_idx"][b]] == c["g_wp"][b, 0]
        assert G[1, b, L1 + c["psqt_idx"][b]] == c["g_bp"][b, 0]


# ------------------------------------------------------------------ quantized path

def _brute_int16(widx, bidx, stm, W16, b16, psqt32, psqt_idx, clip_max, shift):
    B, K = widx.shape
    R, L1 = W16.shape
    h = L1 // 2
    out = np.zeros((B, L1), np.uint8)
    ps_out = np.zeros(B, np.int32)
    wrap = lambda v: ((int(v) + 32768) % 65536) - 32768
    for b in range(B):
        accs, ps = [], []
        for ix in (widx[b], bidx[b]):
            a = [int(v) for v in b16]
            s = 0
            for r in ix:
                if 0 <= r < R:
                    a = [wrap(x + int(w)) for x, w in zip(a, W16[r])]
                    s += int(psqt32[r, psqt_idx[b]])
            accs.append(a)
            ps.append(s)
        order = (1, 0) if stm[b] else (0, 1)
        for o, p in enumerate(order):
            for j in range(h):
                c0 = min(max(accs[p][j], 0), clip_max)
                c1 = min(max(accs[p][j + h], 0), clip_max)
                out[b, o * h + j] = ((c0 * c1) >> shift) & 0xFF
        d = ps[order[0]] - ps[order[1]]
        ps_out[b] = int(d / 2)          # C division truncates toward zero
    return out, ps_out


@pytest.mark.parametrize("clip_max,shift", [(255, 9), (127, 7)])
def test_int16_forward_brute_force(oracle_cpu, clip_max, shift):
    rng = np.random.default_rng(4)
    B, K, R, L1 = 12, 9, 20, 10
    widx = random_lists(rng, B, K, R, allow_holes=True)
    bidx = random_lists(rng, B, K, R, allow_holes=True)
    stm = rng.integers(0, 2, size=B).astype(np.uint8)
    W16 = rng.integers(-9000, 9000, size=(R, L1)).astype(np.int16)     # sums of 9 rows wrap
    W16[:, ::2] = rng.integers(-30, 60, size=(R, L1 // 2)).astype(np.int16)
    b16 = rng.integers(-100, 300, size=L1).astype(np.int16)
    psqt32 = rng.integers(-50000, 50000, size=(R, 8)).astype(np.int32)
    psqt_idx = rng.integers(0, 8, size=B).astype(np.int64)
    out, ps = oracle_cpu.ft_int16_fwd(widx, bidx, stm, W16, b16, psqt32, psqt_idx, clip_max, shift)
    r_out, r_ps = _brute_int16(widx, bidx, stm, W16, b16, psqt32, psqt_idx, clip_max, shift)
    assert np.array_equal(out, r_out)
    assert np.array_equal(ps, r_ps)
    assert (ps != 0).any() and (out != 0).any()


def test_int16_forward_agrees_with_float_path_when_nothing_rounds(oracle_cpu):
    # weights that are multiples of 1/256 and small enough that no sum leaves int16: the integer
    # accumulator is exactly 256 x the float one, the clip is the same, and the product >> 9 is
    # floor(c0*c1*128) of the float path (model/quantize.py:66-73: one=256, max=255, /512).
    rng = np.random.default_rng(5)
    B, K, R, L1 = 40, 32, 300, 64
    h = L1 // 2
    widx = random_lists(rng, B, K, R, min_active=2)
    bidx = random_lists(rng, B, K, R, min_active=2)
    W16 = rng.integers(-20, 40, size=(R, L1)).astype(np.int16)
    b16 = rng.integers(-50, 100, size=L1).astype(np.int16)
    psqt32 = np.zeros((R, 8), np.int32)
    psqt_idx = np.zeros(B, np.int64)
    stm = rng.integers(0, 2, size=B).astype(np.uint8)
    out, _ = oracle_cpu.ft_int16_fwd(widx, bidx, stm, W16, b16, psqt32, psqt_idx, 255, 9)
    Wf = np.concatenate([W16.astype(np.float32) / 256.0, np.zeros((R, 8), np.float32)], axis=1)
    bf = np.concatenate([b16.astype(np.float32) / 256.0, np.zeros(8, np.float32)])
    us = (1 - stm).astype(np.float32)[:, None]
    l0, _, _, saved = oracle_cpu.double_fwd(us, 1 - us, widx, bidx, psqt_idx, Wf, bf, 255.0 / 256.0, L1)
    acc = saved.astype(np.float64) + bf[:L1]                      # [2, B, L1]: white, black accumulators
    mover = np.where(us[None] == 1.0, acc, acc[::-1])               # side to move first
    cl = np.clip(mover, 0.0, 255.0 / 256.0) * 256.0
    want = np.concatenate([np.floor(cl[0, :, :h] * cl[0, :, h:] / 512.0),
                           np.floor(cl[1, :, :h] * cl[1, :, h:] / 512.0)], axis=1)
    assert np.array_equal(out.astype(np.float64), want)
    assert out.max() <= 127
