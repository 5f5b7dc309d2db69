"""ctypes binding of libnnueft.so (declarations in include/nnueft.h).

The library is built in-tree by nnueft._build.build() (hipcc, gfx950).  Loading never falls back
to another implementation: if the shared object is missing or does not export a symbol,
`load()` raises, and `available()` is False.
"""
import ctypes
import os
from ctypes import c_double, c_float, c_int, c_longlong, c_size_t, c_void_p

_PKG = os.path.dirname(os.path.abspath(__file__))
# NNUEFT_LIBRARY points at another build of the same library (kernel tuning)
LIB_PATH = os.environ.get("NNUEFT_LIBRARY") or os.path.join(_PKG, "libnnueft.so")

class RangerArgs(ctypes.Structure):
    """nnueft_ranger_args of the header, field for field."""

    _fields_ = [(n, c_void_p) for n in ("p", "grad", "grad_ma", "neg_grad_ma", "variance_ma", "lookahead_params")] + \
               [("n", c_longlong)] + \
               [(n, c_float) for n in ("beta2", "one_minus_beta2", "bias_correction2", "beta1", "one_minus_beta1",
                                       "one_plus_pnm", "pnm_factor", "noise_norm", "lr_div_bc1", "eps", "wd_factor",
                                       "lookahead_alpha", "one_minus_lookahead_alpha")] + \
               [("odd_step", c_int), ("update_variance", c_int)]


# name -> (restype, argtypes); mirrors include/nnueft.h one to one
PROTOTYPES = {
    "nnueft_version": (c_int, []),
    "nnueft_error_string": (ctypes.c_char_p, [c_int]),
    "nnueft_bias_tile": (c_int, []),
    "nnueft_row_split": (c_int, []),
    "nnueft_row_window": (c_int, [c_int]),
    "nnueft_sparse_fwd": (c_int, [c_void_p] * 4 + [c_int] * 4 + [c_void_p]),
    "nnueft_sparse_bwd_atomic": (c_int, [c_void_p] * 4 + [c_int] * 4 + [c_void_p]),
    "nnueft_device_xcds": (c_int, []),
    "nnueft_det_workspace_bytes": (c_size_t, [c_int] * 6),
    "nnueft_sparse_bwd_det": (c_int, [c_void_p] * 4 + [c_int] * 5 + [c_void_p, c_size_t, c_void_p]),
    "nnueft_fwd_workspace_bytes": (c_size_t, [c_int] * 5),
    "nnueft_double_fwd": (
        c_int,
        [c_void_p] * 7 + [c_float] + [c_void_p] * 4 + [c_int] * 5 + [c_void_p, c_size_t, c_void_p],
    ),
    "nnueft_double_fwd_act": (
        c_int,
        [c_void_p] * 7 + [c_float] + [c_void_p] * 4 + [c_int] * 5 + [c_void_p, c_size_t] + [c_float] * 3 + [c_void_p],
    ),
    "nnueft_double_fwd_virtual_fits": (c_int, [c_int] * 6),
    "nnueft_double_fwd_virtual": (
        c_int,
        [c_void_p] * 8 + [c_float] + [c_void_p] * 4 + [c_int] * 6 + [c_float] * 2 + [c_int]
        + [c_void_p, c_size_t] + [c_int] + [c_float] * 3 + [c_void_p],
    ),
    "nnueft_double_fwd_noalloc": (c_int, [c_void_p] * 7 + [c_float] + [c_void_p] * 4 + [c_int] * 5 + [c_void_p]),
    "nnueft_double_bwd_atomic": (c_int, [c_void_p] * 6 + [c_float] + [c_void_p] * 6 + [c_int] * 5 + [c_void_p]),
    "nnueft_atomic_lds_workspace_bytes": (c_size_t, [c_int] * 5),
    "nnueft_sparse_bwd_atomic_lds": (c_int, [c_void_p] * 4 + [c_int] * 4 + [c_void_p, c_size_t, c_void_p]),
    "nnueft_double_bwd_atomic_lds": (
        c_int, [c_void_p] * 6 + [c_float] + [c_void_p] * 6 + [c_int] * 5 + [c_void_p, c_size_t, c_void_p],
    ),
    "nnueft_double_bwd_det": (
        c_int,
        [c_void_p] * 6 + [c_float] + [c_void_p] * 6 + [c_int] * 6 + [c_void_p, c_size_t, c_void_p, c_void_p, c_void_p],
    ),
    "nnueft_det_sort_bytes": (c_size_t, [c_int] * 5),
    "nnueft_det_sort": (c_int, [c_void_p] * 2 + [c_int] * 6 + [c_void_p, c_size_t, c_void_p]),
    "nnueft_det_reduce_rows": (c_int, [c_void_p] * 2 + [c_int] * 6 + [c_void_p, c_size_t, c_void_p, c_void_p]),
    "nnueft_det_upstream_pitch": (c_int, [c_int]),
    "nnueft_det_reduce_rows_pitched": (c_int, [c_void_p, c_int, c_void_p] + [c_int] * 6
                                       + [c_void_p, c_size_t, c_void_p, c_void_p]),
    "nnueft_table_merge": (c_int, [c_void_p] * 3 + [c_int] * 4 + [c_float] * 2 + [c_int, c_void_p]),
    "nnueft_table_virtual_grad": (c_int, [c_void_p] * 2 + [c_int] * 3 + [c_void_p]),
    "nnueft_int16_workspace_bytes": (c_size_t, [c_int] * 5),
    "nnueft_ft_int16_fwd": (c_int, [c_void_p] * 9 + [c_int] * 8 + [c_void_p, c_size_t, c_void_p]),
    "nnueft_stack_int8_fwd": (c_int, [c_void_p] * 9 + [c_int] * 12 + [c_void_p]),
    "nnueft_bucket_linear_workspace_bytes": (c_size_t, [c_int] * 2),
    "nnueft_bucket_linear_group": (c_int, [c_void_p] + [c_int] * 2 + [c_void_p, c_size_t, c_void_p]),
    "nnueft_bucket_linear_fwd": (c_int, [c_void_p] * 5 + [c_int] * 4 + [c_void_p, c_size_t, c_int, c_void_p]),
    "nnueft_bucket_linear_bwd": (c_int, [c_void_p] * 7 + [c_int] * 4 + [c_void_p, c_size_t, c_int, c_void_p]),
    "nnueft_act_fake_quantize": (c_int, [c_void_p] * 2 + [c_longlong] + [c_float] * 3 + [c_void_p]),
    "nnueft_sqr_crelu_fwd": (c_int, [c_void_p] * 3 + [c_int] * 2 + [c_float] * 4 + [c_int, c_void_p]),
    "nnueft_sqr_crelu_bwd": (c_int, [c_void_p] * 4 + [c_int] * 2 + [c_float] * 4 + [c_int, c_void_p]),
    "nnueft_stack_output_fwd": (c_int, [c_void_p] * 6 + [c_int, c_longlong, c_longlong, c_int, c_void_p]),
    "nnueft_stack_output_bwd": (c_int, [c_void_p] * 4 + [c_int, c_void_p]),
    "nnueft_sf_loss_fwd": (c_int, [c_void_p] * 6 + [c_int] + [c_float] * 11 + [c_double, c_void_p]),
    "nnueft_sf_loss_bwd": (c_int, [c_void_p] * 4 + [c_int, c_void_p]),
    "nnueft_batch_unpack": (c_int, [c_void_p] * 4 + [c_int, c_void_p]),
    "nnueft_ranger_lite_update_pnm": (
        c_int,
        [c_void_p] * 5 + [c_longlong] + [c_float] * 10 + [c_longlong, c_float, c_int, c_void_p, c_float, c_void_p],
    ),
    "nnueft_ranger_lite_update_adam": (
        c_int, [c_void_p] * 4 + [c_longlong] + [c_float] * 7 + [c_float, c_int, c_void_p, c_float, c_void_p],
    ),
    "nnueft_ranger_lite_update_multi": (c_int, [ctypes.POINTER(RangerArgs), c_int, c_void_p]),
    "nnueft_ranger_lite_update_variance": (c_int, [c_void_p] * 2 + [c_longlong] + [c_float] * 2 + [c_void_p]),
    "nnueft_ranger_lite_lookahead_merge": (c_int, [c_void_p] * 2 + [c_longlong, c_float, c_void_p]),
    "nnueft_probe_l2_gather": (c_int, [c_void_p, c_size_t, c_void_p] + [c_int] * 4 + [ctypes.POINTER(c_longlong), c_void_p]),
    "nnueft_probe_lds_read": (c_int, [c_void_p, c_int, c_int, ctypes.POINTER(c_longlong), c_void_p]),
}

E_UNSUPPORTED = -3   # NNUEFT_E_UNSUPPORTED of the header

_lib = None
_load_error = None


def load():
    """Return the loaded library, raising if it cannot be loaded."""
    global _lib, _load_error
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        _load_error = RuntimeError(
            f"{LIB_PATH} not found: build it with `python -c 'import __graft_entry__ as g; g.build()'` "
            "(or nnueft._build.build()); there is no fallback implementation"
        )
        raise _load_error
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in PROTOTYPES.items():
        fn = getattr(lib, name)  # AttributeError if the symbol is not exported
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def available() -> bool:
    try:
        load()
        return True
    except (OSError, RuntimeError, AttributeError):
        return False


def check(rc: int, what: str) -> None:
    if rc != 0:
        msg = load().nnueft_error_string(rc).decode()
        raise RuntimeError(f"{what} failed with code {rc}: {msg}")
