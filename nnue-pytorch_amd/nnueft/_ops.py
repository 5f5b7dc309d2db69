"""The four launches of the operator as torch custom ops (namespace `nnueft`).

A custom op is opaque to dynamo and carries a shape function, so `torch.compile` keeps the operator inside
its graph instead of breaking the graph around it (which is what the reference's own kernels do: they are
wrapped in `torch.compiler.disable`, sparse_linear_kernel.py:50, fused_ft_kernel.py:12): with the
"cudagraphs" backend, or inductor's cudagraph mode, the HIP kernels are then part of the captured graph.
Everything that touches raw pointers, streams and scratch memory lives in the op bodies (`*_impl`); the
autograd functions of sparse_linear_functions.py / fused_ft_functions.py call them through `launch()`: as the
registered op while dynamo traces, directly otherwise (the dispatcher costs about 25 us per call, a quarter
of a step at the reference's micro-benchmark shape).

  nnueft::sparse_fwd   nnueft_sparse_fwd
  nnueft::sparse_bwd   nnueft_sparse_bwd_{atomic,det}
  nnueft::double_fwd   nnueft_double_fwd / nnueft_double_fwd_act
  nnueft::double_bwd   nnueft_double_bwd_{atomic,atomic_lds,det}

and what ComposedFeatureTransformer launches around the operator, so that the module compiles as one graph too:

  nnueft::double_fwd_virtual   nnueft_double_fwd_virtual (real + virtual weights merged inside the gather)
  nnueft::table_merge          nnueft_table_merge
  nnueft::table_virtual_grad   nnueft_table_virtual_grad
  nnueft::act_fake_quantize    nnueft_act_fake_quantize
"""
from typing import Optional, Tuple

import torch
from torch import Tensor

from . import _native

_AUX_STREAMS = {}


def aux_stream(device):
    """A second stream per device (default priority) for work that is independent of what runs on the
    caller's stream; whoever uses it orders it against the caller's stream with events."""
    key = torch.device(device).index if torch.device(device).index is not None else torch.cuda.current_device()
    if key not in _AUX_STREAMS:
        _AUX_STREAMS[key] = torch.cuda.Stream(device=key)
    return _AUX_STREAMS[key]


def stream_ptr(device) -> int:
    return torch.cuda.current_stream(device).cuda_stream


def workspace(nbytes: int, device) -> Tensor:
    # torch's caching allocator hands out blocks aligned to 512 bytes
    return torch.empty(max(int(nbytes), 1), dtype=torch.uint8, device=device)


def row_split_of(mode: str) -> int:
    """The row_split argument of the deterministic entry points for a backward mode.  NNUEFT_ROW_SPLIT in the
    environment replaces the library's threshold for the "deterministic" mode (kernel tuning: the threshold is
    part of the summation order, so results change in the last bits of the rows it moves across)."""
    import os

    if mode == "deterministic_strict":
        return 0
    override = os.environ.get("NNUEFT_ROW_SPLIT", "")
    return int(override) if override.isdigit() else _native.load().nnueft_row_split()


_XCDS_CHECKED = set()


def _warn_once_about_xcds(lib, device) -> None:
    """The blocked kernels are laid out for 8 XCDs; on a device that presents another number (a partitioned
    GPU) the library takes slower paths with the same results.  Say so once per device."""
    key = torch.device(device).index
    if key in _XCDS_CHECKED:
        return
    _XCDS_CHECKED.add(key)
    n = lib.nnueft_device_xcds()
    if n not in (0, 8):
        import warnings

        warnings.warn(f"nnueft: device {device} presents {n} XCDs; the L2-blocked kernels are laid out for 8 and are "
                      "not used (results are the same, the gathers run two to three times slower)")


# Rows from which the atomic backward adds in LDS tiles (narrower rows give an XCD too few column tiles to share).
ATOMIC_LDS_MIN_COLS = 512


def _atomic_lds_bytes(lib, B: int, K: int, num_rows: int, out_cols: int, n_persp: int, device) -> int:
    """Workspace of the LDS-tiled atomic backward for this shape, 0 when it is not to be taken."""
    if B <= 0 or out_cols < ATOMIC_LDS_MIN_COLS or lib.nnueft_device_xcds() != 8:
        return 0
    return int(lib.nnueft_atomic_lds_workspace_bytes(B, K, num_rows, out_cols, n_persp))


# ------------------------------------------------------------------------------------------ sparse linear

def sparse_fwd_impl(feature_indices: Tensor, weight: Tensor, bias: Tensor) -> Tensor:
    lib = _native.load()
    B, K = feature_indices.shape
    R, out_cols = weight.shape
    output = torch.empty(B, out_cols, dtype=torch.float32, device=weight.device)
    with torch.cuda.device(weight.device):
        rc = lib.nnueft_sparse_fwd(feature_indices.data_ptr(), weight.data_ptr(), bias.data_ptr(), output.data_ptr(),
                                   B, K, R, out_cols, stream_ptr(weight.device))
    _native.check(rc, "nnueft_sparse_fwd")
    return output


sparse_fwd = torch.library.custom_op("nnueft::sparse_fwd", sparse_fwd_impl, mutates_args=(), device_types="cuda")


@sparse_fwd.register_fake
def _(feature_indices, weight, bias):
    return weight.new_empty(feature_indices.shape[0], weight.shape[1])


def sparse_bwd_impl(feature_indices: Tensor, grad_output: Tensor, num_rows: int, mode: str) -> Tuple[Tensor, Tensor]:
    lib = _native.load()
    B, K = feature_indices.shape
    out_cols = grad_output.shape[1]
    device = grad_output.device
    with torch.cuda.device(device):
        if mode != "atomic":
            weight_grad = torch.empty(num_rows, out_cols, dtype=torch.float32, device=device)
            bias_grad = torch.empty(out_cols, dtype=torch.float32, device=device)
            if B == 0:
                return weight_grad.zero_(), bias_grad.zero_()
            row_split = row_split_of(mode)
            nbytes = lib.nnueft_det_workspace_bytes(B, K, num_rows, out_cols, 1, row_split)
            ws = workspace(nbytes, device)
            rc = lib.nnueft_sparse_bwd_det(
                feature_indices.data_ptr(), grad_output.data_ptr(), weight_grad.data_ptr(), bias_grad.data_ptr(),
                B, K, num_rows, out_cols, row_split, ws.data_ptr(), nbytes, stream_ptr(device),
            )
            _native.check(rc, "nnueft_sparse_bwd_det")
        else:
            # atomic adds in LDS tiles where the shape and the device can take them (rows of 512 columns and
            # more; the gradient is then written, not accumulated), else atomics on the zeroed gradient
            nbytes = _atomic_lds_bytes(lib, B, K, num_rows, out_cols, 1, device)
            if nbytes:
                weight_grad = torch.empty(num_rows, out_cols, dtype=torch.float32, device=device)
                bias_grad = torch.empty(out_cols, dtype=torch.float32, device=device)
                ws = workspace(nbytes, device)
                rc = lib.nnueft_sparse_bwd_atomic_lds(
                    feature_indices.data_ptr(), grad_output.data_ptr(), weight_grad.data_ptr(), bias_grad.data_ptr(),
                    B, K, num_rows, out_cols, ws.data_ptr(), nbytes, stream_ptr(device),
                )
                if rc != _native.E_UNSUPPORTED:
                    _native.check(rc, "nnueft_sparse_bwd_atomic_lds")
                    return weight_grad, bias_grad
            weight_grad = torch.zeros(num_rows, out_cols, dtype=torch.float32, device=device)
            bias_grad = torch.zeros(out_cols, dtype=torch.float32, device=device)
            if B > 0:
                rc = lib.nnueft_sparse_bwd_atomic(
                    feature_indices.data_ptr(), grad_output.data_ptr(), weight_grad.data_ptr(), bias_grad.data_ptr(),
                    B, K, num_rows, out_cols, stream_ptr(device),
                )
                _native.check(rc, "nnueft_sparse_bwd_atomic")
    return weight_grad, bias_grad


sparse_bwd = torch.library.custom_op("nnueft::sparse_bwd", sparse_bwd_impl, mutates_args=(), device_types="cuda")


@sparse_bwd.register_fake
def _(feature_indices, grad_output, num_rows, mode):
    return grad_output.new_empty(num_rows, grad_output.shape[1]), grad_output.new_empty(grad_output.shape[1])


# ------------------------------------------------------------------------------------------ fused double FT

def double_fwd_impl(us: Tensor, them: Tensor, white_indices: Tensor, black_indices: Tensor, psqt_indices: Tensor,
               weight: Tensor, bias: Tensor, max_ft_activation: float, l1_size: int, act_on: bool,
               act_scale: float, act_eps: float, act_post_mul: float) -> Tuple[Tensor, Tensor, Tensor, Tensor]:
    """l0, wpsqt, bpsqt and the two perspectives' row sums kept for the backward.  act_on: l0 comes out as
    (floor(l0 * act_scale + act_eps) / act_scale) * act_post_mul."""
    lib = _native.load()
    device = weight.device
    _warn_once_about_xcds(lib, device)
    B, K = white_indices.shape
    R, out_cols = weight.shape
    l0_ = torch.empty(B, l1_size, dtype=torch.float32, device=device)
    wpsqt = torch.empty(B, 1, dtype=torch.float32, device=device)
    bpsqt = torch.empty(B, 1, dtype=torch.float32, device=device)
    row_sums = torch.empty(2, B, l1_size, dtype=torch.float32, device=device)
    with torch.cuda.device(device):
        nbytes = lib.nnueft_fwd_workspace_bytes(B, K, R, l1_size, out_cols - l1_size)
        ws = workspace(nbytes, device)
        head = (
            us.data_ptr(), them.data_ptr(), white_indices.data_ptr(), black_indices.data_ptr(),
            psqt_indices.data_ptr(), weight.data_ptr(), bias.data_ptr(), float(max_ft_activation),
            l0_.data_ptr(), wpsqt.data_ptr(), bpsqt.data_ptr(), row_sums.data_ptr(),
            B, K, R, l1_size, out_cols - l1_size, ws.data_ptr(), nbytes,
        )
        if not act_on:
            rc = lib.nnueft_double_fwd(*head, stream_ptr(device))
            _native.check(rc, "nnueft_double_fwd")
        else:
            rc = lib.nnueft_double_fwd_act(*head, float(act_scale), float(act_eps), float(act_post_mul),
                                           stream_ptr(device))
            _native.check(rc, "nnueft_double_fwd_act")
    return l0_, wpsqt, bpsqt, row_sums


double_fwd = torch.library.custom_op("nnueft::double_fwd", double_fwd_impl, mutates_args=(), device_types="cuda")


@double_fwd.register_fake
def _(us, them, white_indices, black_indices, psqt_indices, weight, bias, max_ft_activation, l1_size, act_on,
      act_scale, act_eps, act_post_mul):
    B = white_indices.shape[0]
    return (weight.new_empty(B, l1_size), weight.new_empty(B, 1), weight.new_empty(B, 1),
            weight.new_empty(2, B, l1_size))


def det_sort_impl(white_indices: Tensor, black_indices: Tensor, num_rows: int, output_size: int, row_split: int) -> Tensor:
    """The sort of the deterministic backward reads nothing but the index lists, so it can start in the forward
    pass, on a second stream, and is long done when the backward pass wants it.  Returns the sorted lists, an
    opaque byte tensor that is complete once the second stream has run."""
    lib = _native.load()
    B, K = white_indices.shape
    device = white_indices.device
    with torch.cuda.device(device):
        nbytes = lib.nnueft_det_sort_bytes(B, K, num_rows, output_size, 2)
        buf = workspace(nbytes, device)
        cur, aux = torch.cuda.current_stream(device), aux_stream(device)
        aux.wait_stream(cur)                     # the lists and buf are ordered on the caller's stream
        rc = lib.nnueft_det_sort(white_indices.data_ptr(), black_indices.data_ptr(), B, K, num_rows, output_size, 2,
                                 row_split, buf.data_ptr(), nbytes, aux.cuda_stream)
        _native.check(rc, "nnueft_det_sort")
        for t in (buf, white_indices, black_indices):
            t.record_stream(aux)                 # their memory is not handed out again before the sort has run
    return buf


det_sort = torch.library.custom_op("nnueft::det_sort", det_sort_impl, mutates_args=(), device_types="cuda")


@det_sort.register_fake
def _(white_indices, black_indices, num_rows, output_size, row_split):
    B, K = white_indices.shape
    nbytes = _native.load().nnueft_det_sort_bytes(B, K, num_rows, output_size, 2)      # a host-only call
    return white_indices.new_empty(max(int(nbytes), 1), dtype=torch.uint8)


def double_bwd_impl(us: Tensor, them: Tensor, white_indices: Tensor, black_indices: Tensor, psqt_indices: Tensor,
               bias: Tensor, max_ft_activation: float, grad_l0: Tensor, grad_wpsqt: Tensor, grad_bpsqt: Tensor,
               row_sums: Tensor, num_rows: int, l1_size: int, output_size: int, mode: str,
               presorted: Optional[Tensor], second_stream: bool) -> Tuple[Tensor, Tensor]:
    lib = _native.load()
    B, K = white_indices.shape
    device = us.device
    n_psqt = output_size - l1_size
    grad_l0, grad_wpsqt, grad_bpsqt = grad_l0.contiguous(), grad_wpsqt.contiguous(), grad_bpsqt.contiguous()
    head = (
        us.data_ptr(), them.data_ptr(), white_indices.data_ptr(), black_indices.data_ptr(),
        psqt_indices.data_ptr(), bias.data_ptr(), float(max_ft_activation),
        grad_l0.data_ptr(), grad_wpsqt.data_ptr(), grad_bpsqt.data_ptr(), row_sums.data_ptr(),
    )
    with torch.cuda.device(device):
        if mode != "atomic":
            grad_weight = torch.empty(num_rows, output_size, dtype=torch.float32, device=device)
            grad_bias = torch.empty(output_size, dtype=torch.float32, device=device)
            if B == 0:
                return grad_weight.zero_(), grad_bias.zero_()
            row_split = row_split_of(mode)
            nbytes = lib.nnueft_det_workspace_bytes(B, K, num_rows, output_size, 2, row_split)
            ws = workspace(nbytes, device)
            # presorted: the lists sorted during the forward pass on the second stream; the entry point makes
            # its reduction (not its first kernel) wait for that stream
            sorted_ptr = presorted.data_ptr() if presorted is not None else None
            rc = lib.nnueft_double_bwd_det(
                *head, grad_weight.data_ptr(), grad_bias.data_ptr(), B, K, num_rows, l1_size, n_psqt, row_split,
                ws.data_ptr(), nbytes, sorted_ptr, stream_ptr(device),
                aux_stream(device).cuda_stream if second_stream else None,
            )
            _native.check(rc, "nnueft_double_bwd_det")
        else:
            nbytes = _atomic_lds_bytes(lib, B, K, num_rows, output_size, 2, device)
            if nbytes:
                grad_weight = torch.empty(num_rows, output_size, dtype=torch.float32, device=device)
                grad_bias = torch.empty(output_size, dtype=torch.float32, device=device)
                ws = workspace(nbytes, device)
                rc = lib.nnueft_double_bwd_atomic_lds(
                    *head, grad_weight.data_ptr(), grad_bias.data_ptr(), B, K, num_rows, l1_size, n_psqt,
                    ws.data_ptr(), nbytes, stream_ptr(device),
                )
                if rc != _native.E_UNSUPPORTED:
                    _native.check(rc, "nnueft_double_bwd_atomic_lds")
                    return grad_weight, grad_bias
            grad_weight = torch.zeros(num_rows, output_size, dtype=torch.float32, device=device)
            grad_bias = torch.zeros(output_size, dtype=torch.float32, device=device)
            if B > 0:
                rc = lib.nnueft_double_bwd_atomic(
                    *head, grad_weight.data_ptr(), grad_bias.data_ptr(), B, K, num_rows, l1_size, n_psqt,
                    stream_ptr(device),
                )
                _native.check(rc, "nnueft_double_bwd_atomic")
    return grad_weight, grad_bias


double_bwd = torch.library.custom_op("nnueft::double_bwd", double_bwd_impl, mutates_args=(), device_types="cuda")


@double_bwd.register_fake
def _(us, them, white_indices, black_indices, psqt_indices, bias, max_ft_activation, grad_l0, grad_wpsqt, grad_bpsqt,
      row_sums, num_rows, l1_size, output_size, mode, presorted, second_stream):
    return grad_l0.new_empty(num_rows, output_size), grad_l0.new_empty(output_size)


# ------------------------------------------------------------------------------------------ module layer

def double_fwd_virtual_impl(us: Tensor, them: Tensor, white_indices: Tensor, black_indices: Tensor, psqt_indices: Tensor,
                            weight: Tensor, virtual: Tensor, bias: Tensor, max_ft_activation: float, l1_size: int,
                            scale_ft: float, scale_psqt: float, quantize: bool, act_on: bool, act_scale: float,
                            act_eps: float, act_post_mul: float) -> Tuple[Tensor, Tensor, Tensor, Tensor]:
    """double_fwd over the table q(weight + virtual[row % virtual rows]) without that table being written."""
    lib = _native.load()
    device = weight.device
    B, K = white_indices.shape
    R, cols = weight.shape
    l0_ = torch.empty(B, l1_size, dtype=torch.float32, device=device)
    wpsqt = torch.empty(B, 1, dtype=torch.float32, device=device)
    bpsqt = torch.empty(B, 1, dtype=torch.float32, device=device)
    row_sums = torch.empty(2, B, l1_size, dtype=torch.float32, device=device)
    with torch.cuda.device(device):
        nbytes = lib.nnueft_fwd_workspace_bytes(B, K, R, l1_size, cols - l1_size)
        ws = workspace(nbytes, device)
        rc = lib.nnueft_double_fwd_virtual(
            us.data_ptr(), them.data_ptr(), white_indices.data_ptr(), black_indices.data_ptr(),
            psqt_indices.data_ptr(), weight.data_ptr(), virtual.data_ptr(), bias.data_ptr(), float(max_ft_activation),
            l0_.data_ptr(), wpsqt.data_ptr(), bpsqt.data_ptr(), row_sums.data_ptr(), B, K, R, l1_size,
            cols - l1_size, virtual.shape[0], float(scale_ft), float(scale_psqt), int(bool(quantize)),
            ws.data_ptr(), nbytes, int(bool(act_on)), float(act_scale), float(act_eps), float(act_post_mul),
            stream_ptr(device))
    _native.check(rc, "nnueft_double_fwd_virtual")
    return l0_, wpsqt, bpsqt, row_sums


double_fwd_virtual = torch.library.custom_op("nnueft::double_fwd_virtual", double_fwd_virtual_impl, mutates_args=(),
                                             device_types="cuda")


@double_fwd_virtual.register_fake
def _(us, them, white_indices, black_indices, psqt_indices, weight, virtual, bias, max_ft_activation, l1_size, scale_ft,
      scale_psqt, quantize, act_on, act_scale, act_eps, act_post_mul):
    B = white_indices.shape[0]
    return (weight.new_empty(B, l1_size), weight.new_empty(B, 1), weight.new_empty(B, 1),
            weight.new_empty(2, B, l1_size))


def table_merge_impl(weight: Tensor, virtual: Optional[Tensor], l1_size: int, scale_ft: float, scale_psqt: float,
                     quantize: bool) -> Tensor:
    """q(weight + virtual[row % virtual rows]) in one pass (virtual None: the grid alone)."""
    lib = _native.load()
    R, cols = weight.shape
    merged = torch.empty_like(weight)
    with torch.cuda.device(weight.device):
        rc = lib.nnueft_table_merge(weight.data_ptr(), None if virtual is None else virtual.data_ptr(),
                                    merged.data_ptr(), R, cols, l1_size, 1 if virtual is None else virtual.shape[0],
                                    float(scale_ft), float(scale_psqt), int(bool(quantize)), stream_ptr(weight.device))
    _native.check(rc, "nnueft_table_merge")
    return merged


table_merge = torch.library.custom_op("nnueft::table_merge", table_merge_impl, mutates_args=(), device_types="cuda")


@table_merge.register_fake
def _(weight, virtual, l1_size, scale_ft, scale_psqt, quantize):
    return torch.empty_like(weight)


def table_virtual_grad_impl(grad: Tensor, vrows: int) -> Tensor:
    """The gradient of the virtual rows: the sum of the table's blocks of `vrows` rows."""
    lib = _native.load()
    R, cols = grad.shape
    gv = torch.empty(vrows, cols, dtype=grad.dtype, device=grad.device)
    with torch.cuda.device(grad.device):
        rc = lib.nnueft_table_virtual_grad(grad.data_ptr(), gv.data_ptr(), R, cols, vrows, stream_ptr(grad.device))
    _native.check(rc, "nnueft_table_virtual_grad")
    return gv


table_virtual_grad = torch.library.custom_op("nnueft::table_virtual_grad", table_virtual_grad_impl, mutates_args=(),
                                             device_types="cuda")


@table_virtual_grad.register_fake
def _(grad, vrows):
    return grad.new_empty(vrows, grad.shape[1])


def act_fake_quantize_impl(x: Tensor, scale: float, eps: float, post_mul: float) -> Tensor:
    """(floor(x * scale + eps) / scale) * post_mul in one pass."""
    lib = _native.load()
    out = torch.empty_like(x)
    with torch.cuda.device(x.device):
        rc = lib.nnueft_act_fake_quantize(x.data_ptr(), out.data_ptr(), x.numel(), float(scale), float(eps),
                                          float(post_mul), stream_ptr(x.device))
    _native.check(rc, "nnueft_act_fake_quantize")
    return out


act_fake_quantize = torch.library.custom_op("nnueft::act_fake_quantize", act_fake_quantize_impl, mutates_args=(),
                                            device_types="cuda")


@act_fake_quantize.register_fake
def _(x, scale, eps, post_mul):
    return torch.empty_like(x)


_IMPLS = {"sparse_fwd": sparse_fwd_impl, "sparse_bwd": sparse_bwd_impl, "double_fwd": double_fwd_impl,
          "det_sort": det_sort_impl, "double_bwd": double_bwd_impl, "double_fwd_virtual": double_fwd_virtual_impl,
          "table_merge": table_merge_impl, "table_virtual_grad": table_virtual_grad_impl,
          "act_fake_quantize": act_fake_quantize_impl}


_OPS = {"sparse_fwd": torch.ops.nnueft.sparse_fwd, "sparse_bwd": torch.ops.nnueft.sparse_bwd,
        "double_fwd": torch.ops.nnueft.double_fwd, "det_sort": torch.ops.nnueft.det_sort,
        "double_bwd": torch.ops.nnueft.double_bwd, "double_fwd_virtual": torch.ops.nnueft.double_fwd_virtual,
        "table_merge": torch.ops.nnueft.table_merge, "table_virtual_grad": torch.ops.nnueft.table_virtual_grad,
        "act_fake_quantize": torch.ops.nnueft.act_fake_quantize}


def launch(name: str, *args):
    """The op `nnueft::<name>`: through the dispatcher while a graph is being traced, as a plain call otherwise."""
    if torch.compiler.is_compiling():
        return _OPS[name](*args)
    return _IMPLS[name](*args)
