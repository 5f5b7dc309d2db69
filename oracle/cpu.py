"""numpy front end of libnnueft_oracle.so (see nnueft_oracle.c for what each function follows).

TEST INFRASTRUCTURE: the checker, never the thing measured or shipped.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libnnueft_oracle.so")
_lib = None


def build(force: bool = False) -> str:
    """Compile the C restatement (and, where the reference checkout exists, _ref)."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s", "all"])
    return _LIB_PATH


def lib():
    global _lib
    if _lib is None:
        build()
        _lib = ctypes.CDLL(_LIB_PATH)
    return _lib


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def _c(a, dtype):
    a = np.ascontiguousarray(a, dtype=dtype)
    return a


def bias_tile() -> int:
    return int(lib().nnueft_oracle_bias_tile())


def row_split() -> int:
    """Default threshold: most slots that may name a table row before its gradient is summed window by
    window.  sparse_bwd / double_bwd take row_split=None for this value, 0 for the strict order (no row
    is split: the order of the reference's CPU path) or any other threshold."""
    return int(lib().nnueft_oracle_row_split())


def _rs(threshold) -> int:
    return row_split() if threshold is None else int(threshold)


def row_window(B: int) -> int:
    """Positions per window of the split rows' order for a batch of B."""
    return int(lib().nnueft_oracle_row_window(int(B)))


def sparse_fwd(idx, W, bias):
    idx, W, bias = _c(idx, np.int32), _c(W, np.float32), _c(bias, np.float32)
    B, K = idx.shape
    R, oc = W.shape
    out = np.empty((B, oc), np.float32)
    rc = lib().nnueft_oracle_sparse_fwd(_p(idx), _p(W), _p(bias), _p(out), B, K, R, oc)
    assert rc == 0
    return out


def sparse_bwd(idx, gout, R, row_split=None):
    idx, gout = _c(idx, np.int32), _c(gout, np.float32)
    B, K = idx.shape
    oc = gout.shape[1]
    gW = np.empty((R, oc), np.float32)
    gb = np.empty((oc,), np.float32)
    rc = lib().nnueft_oracle_sparse_bwd(_p(idx), _p(gout), _p(gW), _p(gb), B, K, R, oc, _rs(row_split))
    assert rc == 0
    return gW, gb


def double_fwd(us, them, widx, bidx, psqt_idx, W, bias, max_act, L1):
    us, them = _c(us, np.float32).reshape(-1), _c(them, np.float32).reshape(-1)
    widx, bidx = _c(widx, np.int32), _c(bidx, np.int32)
    psqt_idx = _c(psqt_idx, np.int64)
    W, bias = _c(W, np.float32), _c(bias, np.float32)
    B, K = widx.shape
    R, oc = W.shape
    n_psqt = oc - L1
    l0 = np.empty((B, L1), np.float32)
    wp = np.empty((B, 1), np.float32)
    bp = np.empty((B, 1), np.float32)
    saved = np.empty((2, B, L1), np.float32)
    rc = lib().nnueft_oracle_double_fwd(_p(us), _p(them), _p(widx), _p(bidx), _p(psqt_idx), _p(W), _p(bias),
                                        ctypes.c_float(max_act), _p(l0), _p(wp), _p(bp), _p(saved),
                                        B, K, R, L1, n_psqt)
    assert rc == 0
    return l0, wp, bp, saved


def double_bwd_rows(us, them, psqt_idx, bias, max_act, grad_l0, grad_wpsqt, grad_bpsqt, saved, n_psqt):
    us, them = _c(us, np.float32).reshape(-1), _c(them, np.float32).reshape(-1)
    psqt_idx = _c(psqt_idx, np.int64)
    bias = _c(bias, np.float32)
    grad_l0 = _c(grad_l0, np.float32)
    gwp, gbp = _c(grad_wpsqt, np.float32).reshape(-1), _c(grad_bpsqt, np.float32).reshape(-1)
    saved = _c(saved, np.float32)
    B, L1 = grad_l0.shape
    G = np.empty((2, B, L1 + n_psqt), np.float32)
    rc = lib().nnueft_oracle_double_bwd_rows(_p(us), _p(them), _p(psqt_idx), _p(bias), ctypes.c_float(max_act),
                                             _p(grad_l0), _p(gwp), _p(gbp), _p(saved), _p(G), B, L1, n_psqt)
    assert rc == 0
    return G


def double_bwd(us, them, widx, bidx, psqt_idx, bias, max_act, grad_l0, grad_wpsqt, grad_bpsqt, saved, R, n_psqt,
               row_split=None):
    us, them = _c(us, np.float32).reshape(-1), _c(them, np.float32).reshape(-1)
    widx, bidx = _c(widx, np.int32), _c(bidx, np.int32)
    psqt_idx = _c(psqt_idx, np.int64)
    bias = _c(bias, np.float32)
    grad_l0 = _c(grad_l0, np.float32)
    gwp, gbp = _c(grad_wpsqt, np.float32).reshape(-1), _c(grad_bpsqt, np.float32).reshape(-1)
    saved = _c(saved, np.float32)
    B, K = widx.shape
    L1 = grad_l0.shape[1]
    oc = L1 + n_psqt
    gW = np.empty((R, oc), np.float32)
    gb = np.empty((oc,), np.float32)
    rc = lib().nnueft_oracle_double_bwd(_p(us), _p(them), _p(widx), _p(bidx), _p(psqt_idx), _p(bias),
                                        ctypes.c_float(max_act), _p(grad_l0), _p(gwp), _p(gbp), _p(saved),
                                        _p(gW), _p(gb), B, K, R, L1, n_psqt, _rs(row_split))
    assert rc == 0
    return gW, gb


def ft_int16_fwd(widx, bidx, stm, W16, b16, psqt32, psqt_idx, clip_max=255, shift=9):
    widx, bidx = _c(widx, np.int32), _c(bidx, np.int32)
    stm = _c(stm, np.uint8)
    W16, b16, psqt32 = _c(W16, np.int16), _c(b16, np.int16), _c(psqt32, np.int32)
    psqt_idx = _c(psqt_idx, np.int64)
    B, K = widx.shape
    R, L1 = W16.shape
    n_psqt = psqt32.shape[1]
    out = np.empty((B, L1), np.uint8)
    ps = np.empty((B,), np.int32)
    rc = lib().nnueft_oracle_ft_int16_fwd(_p(widx), _p(bidx), _p(stm), _p(W16), _p(b16), _p(psqt32), _p(psqt_idx),
                                          _p(out), _p(ps), B, K, R, L1, n_psqt, int(clip_max), int(shift))
    assert rc == 0
    return out, ps


def table_merge(W, V, L1, scale_ft=256.0, scale_psqt=9600.0, fake_quantize=True):
    W, V = _c(W, np.float32), _c(V, np.float32)
    R, cols = W.shape
    out = np.empty_like(W)
    rc = lib().nnueft_oracle_table_merge(_p(W), _p(V), _p(out), R, cols, int(L1), V.shape[0],
                                         ctypes.c_float(scale_ft), ctypes.c_float(scale_psqt), int(bool(fake_quantize)))
    assert rc == 0
    return out


def table_virtual_grad(gW, vrows):
    gW = _c(gW, np.float32)
    R, cols = gW.shape
    gV = np.empty((vrows, cols), np.float32)
    rc = lib().nnueft_oracle_table_virtual_grad(_p(gW), _p(gV), R, cols, int(vrows))
    assert rc == 0
    return gV


STACK_DEFAULTS = dict(lin1=7, sqr1=21, lin2=6, sqr2=19, act_max=127, out_mult=9600, out_den=32768)


def stack_int8_fwd(x, bucket, W1, b1, W2, b2, Wo, bo, L2, L3, count, **kw):
    k = dict(STACK_DEFAULTS)
    k.update(kw)
    x = _c(x, np.uint8)
    bucket = _c(bucket, np.int64)
    W1, W2, Wo = _c(W1, np.int8), _c(W2, np.int8), _c(Wo, np.int8)
    b1, b2, bo = _c(b1, np.int32), _c(b2, np.int32), _c(bo, np.int32)
    B, L1 = x.shape
    out = np.empty((B,), np.int32)
    rc = lib().nnueft_oracle_stack_int8_fwd(_p(x), _p(bucket), _p(W1), _p(b1), _p(W2), _p(b2), _p(Wo), _p(bo), _p(out),
                                            B, L1, int(L2), int(L3), int(count), k["lin1"], k["sqr1"], k["lin2"],
                                            k["sqr2"], k["act_max"], k["out_mult"], k["out_den"])
    assert rc == 0
    return out


def ranger_lite_update(p, grad, grad_ma, neg_grad_ma, variance_ma, lookahead, *, beta2, bias_correction2, beta1,
                       one_minus_beta1, one_plus_pnm=0.0, pnm_factor=0.0, noise_norm=1.0, lr_div_bc1, eps, step=1,
                       wd_factor=0.0, update_variance=True, alpha=0.5):
    """In place on float32 numpy arrays (neg_grad_ma / lookahead may be None).  beta1 / one_minus_beta1 are the
    squared ones when neg_grad_ma is given, as in the reference's kernels."""
    f = ctypes.c_float
    for a in (p, grad, grad_ma, variance_ma) + tuple(x for x in (neg_grad_ma, lookahead) if x is not None):
        assert a.dtype == np.float32 and a.flags.c_contiguous
    rc = lib().nnueft_oracle_ranger_lite_update(
        _p(p), _p(grad), _p(grad_ma), _p(neg_grad_ma) if neg_grad_ma is not None else None, _p(variance_ma),
        _p(lookahead) if lookahead is not None else None, ctypes.c_longlong(p.size),
        f(beta2), f(np.float32(1.0 - beta2)), f(bias_correction2), f(beta1), f(one_minus_beta1), f(one_plus_pnm),
        f(pnm_factor), f(noise_norm), f(lr_div_bc1), f(eps), ctypes.c_longlong(step), f(wd_factor),
        int(bool(update_variance)), f(alpha))
    assert rc == 0


def ranger_lite_update_variance(grad, variance_ma, beta2):
    rc = lib().nnueft_oracle_ranger_lite_update_variance(_p(grad), _p(variance_ma), ctypes.c_longlong(grad.size),
                                                         ctypes.c_float(beta2), ctypes.c_float(np.float32(1.0 - beta2)))
    assert rc == 0


def act_fake_quantize(x, scale=128.0, eps=1e-5, post_mul=1.0):
    x = _c(x, np.float32)
    out = np.empty_like(x)
    rc = lib().nnueft_oracle_act_fake_quantize(_p(x), _p(out), ctypes.c_longlong(x.size), ctypes.c_float(scale),
                                               ctypes.c_float(eps), ctypes.c_float(post_mul))
    assert rc == 0
    return out


def bucket_linear_fwd(x, bucket, W, bias, out, count):
    x, W, bias = _c(x, np.float32), _c(W, np.float32), _c(bias, np.float32)
    bucket = _c(bucket, np.int64)
    B, n_in = x.shape
    y = np.zeros((B, out), np.float32)
    rc = lib().nnueft_oracle_bucket_linear_fwd(_p(x), _p(bucket), _p(W), _p(bias), _p(y), B, n_in, out, count)
    assert rc == 0
    return y


def bucket_linear_bwd(x, bucket, W, gy, out, count):
    x, W, gy = _c(x, np.float32), _c(W, np.float32), _c(gy, np.float32)
    bucket = _c(bucket, np.int64)
    B, n_in = x.shape
    gx = np.zeros((B, n_in), np.float32)
    gW = np.empty((count * out, n_in), np.float32)
    gb = np.empty((count * out,), np.float32)
    rc = lib().nnueft_oracle_bucket_linear_bwd(_p(x), _p(bucket), _p(W), _p(gy), _p(gx), _p(gW), _p(gb), B, n_in, out,
                                               count)
    assert rc == 0
    return gx, gW, gb
