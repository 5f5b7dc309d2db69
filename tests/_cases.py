"""Seeded inputs shared by the CPU and GPU tests (numpy arrays; the GPU tests upload them)."""
import numpy as np

from nnueft import halfka_v2_hm as hk


def random_lists(rng, B, K, R, min_active=0, max_active=None, allow_holes=False):
    """Index lists with duplicates allowed; trailing -1 padding, optionally -1 holes inside."""
    max_active = K if max_active is None else max_active
    idx = rng.integers(0, R, size=(B, K)).astype(np.int32)
    n = rng.integers(min_active, max_active + 1, size=B)
    idx[np.arange(K)[None, :] >= n[:, None]] = -1
    if allow_holes:
        holes = rng.random((B, K)) < 0.1
        idx[holes] = -1
    return idx


def double_case(seed, B, L1, R, K=32, n_psqt=8, max_act=127.0, binary_side=False, halfka=False,
                weight_scale=1.0, allow_holes=False):
    rng = np.random.default_rng(seed)
    if halfka:
        us, them, widx, bidx, pc = hk.synthetic_batch(B, seed)
        psqt_idx = ((pc - 1) // 4).astype(np.int64)
        assert R >= hk.NUM_INPUTS
    else:
        widx = random_lists(rng, B, K, R, allow_holes=allow_holes)
        bidx = random_lists(rng, B, K, R, allow_holes=allow_holes)
        psqt_idx = rng.integers(0, max(n_psqt, 1), size=B).astype(np.int64)
        if binary_side:
            us = rng.integers(0, 2, size=(B, 1)).astype(np.float32)
            them = (1.0 - us).astype(np.float32)
        else:
            us = rng.standard_normal((B, 1)).astype(np.float32)
            them = rng.standard_normal((B, 1)).astype(np.float32)
    W = (rng.standard_normal((R, L1 + n_psqt)) * weight_scale).astype(np.float32)
    bias = (rng.standard_normal(L1 + n_psqt) * weight_scale).astype(np.float32)
    g_l0 = rng.standard_normal((B, L1)).astype(np.float32)
    g_wp = rng.standard_normal((B, 1)).astype(np.float32)
    g_bp = rng.standard_normal((B, 1)).astype(np.float32)
    return dict(us=us, them=them, widx=widx, bidx=bidx, psqt_idx=psqt_idx, W=W, bias=bias, max_act=float(max_act),
                L1=L1, R=R, K=K, n_psqt=n_psqt, g_l0=g_l0, g_wp=g_wp, g_bp=g_bp)


def sparse_case(seed, B, out_cols, R, K=32, allow_holes=False):
    rng = np.random.default_rng(seed)
    idx = random_lists(rng, B, K, R, allow_holes=allow_holes)
    W = rng.standard_normal((R, out_cols)).astype(np.float32)
    bias = rng.standard_normal(out_cols).astype(np.float32)
    g = rng.standard_normal((B, out_cols)).astype(np.float32)
    return dict(idx=idx, W=W, bias=bias, g=g, R=R, K=K, out_cols=out_cols)
