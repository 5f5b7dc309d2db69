"""Fused two-perspective feature transformer as an autograd function.

Same name, argument order, outputs and assertions as the reference's
model/modules/feature_transformer/fused_ft_functions.py:18-122; the two CuPy kernels it launches
are replaced by nnueft_double_fwd / nnueft_double_bwd_{atomic,det} of libnnueft.so.

Differences that a caller can observe:
  * the activation tensor kept for the backward holds the two perspectives' row sums (the reference
    keeps the clamped mixed values, fused_ft_kernel.py:95-99); the backward recomputes the mix from
    them, so the clamp passes gradient at exactly 0 and exactly max like torch.clamp does in the
    reference's CPU path;
  * the backward mode (NNUEFT_BACKWARD or set_backward_mode): "deterministic" (default) and
    "deterministic_strict" give results that do not depend on scheduling, the strict one bit for bit
    the weight gradient of the reference's CPU path; "atomic" is the reference's GPU scheme.
"""
import torch
from torch import autograd

from . import _native
from . import sparse_linear_functions as _slf
from .sparse_linear_functions import _aux_stream, _aux_stream_ptr, _stream_ptr, _workspace

_HAS_CUPY_KERNELS = _native.available()

# Positions a wave of the atomic backward walks before it flushes its bias partial sums
# (fused_ft_kernel.py:127 has the same constant for the reference's kernel).
BACKWARD_TILE_SIZE = 4


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


@torch.compiler.disable(recursive=False)
def _launch_double_fwd(us, them, white_indices, black_indices, psqt_indices, weight, bias, max_ft_activation,
                       l1_size, l0_, wpsqt, bpsqt, saved, act_grid=None):
    lib = _native.load()
    _warn_once_about_xcds(lib, weight.device)
    B, K = white_indices.shape
    R, out_cols = weight.shape
    nbytes = lib.nnueft_fwd_workspace_bytes(B, K, R, l1_size, out_cols - l1_size)
    ws = _workspace(nbytes, weight.device)
    head = (
        us.data_ptr(), them.data_ptr(), white_indices.data_ptr(), black_indices.data_ptr(),
        psqt_indices.data_ptr(), weight.data_ptr(), bias.data_ptr(), float(max_ft_activation),
        l0_.data_ptr(), wpsqt.data_ptr(), bpsqt.data_ptr(), saved.data_ptr(),
        B, K, R, l1_size, out_cols - l1_size, ws.data_ptr(), nbytes,
    )
    if act_grid is None:
        rc = lib.nnueft_double_fwd(*head, _stream_ptr(weight.device))
        _native.check(rc, "nnueft_double_fwd")
    else:
        scale, eps, post_mul = act_grid
        rc = lib.nnueft_double_fwd_act(*head, float(scale), float(eps), float(post_mul), _stream_ptr(weight.device))
        _native.check(rc, "nnueft_double_fwd_act")


@torch.compiler.disable(recursive=False)
def _launch_det_sort(white_indices, black_indices, num_rows, output_size, row_split):
    """The sort of the deterministic backward reads nothing but the index lists, so it starts here, in
    the forward pass, on a second stream, and is long done when the backward pass wants it.
    Returns the sorted lists, an opaque byte tensor that is complete once the second stream has run."""
    lib = _native.load()
    B, K = white_indices.shape
    device = white_indices.device
    nbytes = lib.nnueft_det_sort_bytes(B, K, num_rows, output_size, 2)
    buf = _workspace(nbytes, device)
    cur, aux = torch.cuda.current_stream(device), _aux_stream(device)
    aux.wait_stream(cur)                     # the lists and buf are ordered on the caller's stream
    rc = lib.nnueft_det_sort(white_indices.data_ptr(), black_indices.data_ptr(), B, K, num_rows, output_size, 2,
                             row_split, buf.data_ptr(), nbytes, aux.cuda_stream)
    _native.check(rc, "nnueft_det_sort")
    for t in (buf, white_indices, black_indices):
        t.record_stream(aux)                 # their memory is not handed out again before the sort has run
    return buf


@torch.compiler.disable(recursive=False)
def _launch_double_bwd(us, them, white_indices, black_indices, psqt_indices, bias, max_ft_activation, grad_l0,
                       grad_wpsqt, grad_bpsqt, saved, num_rows, l1_size, output_size, mode, presorted=None,
                       second_stream=False):
    lib = _native.load()
    B, K = white_indices.shape
    device = us.device
    n_psqt = output_size - l1_size
    head = (
        us.data_ptr(), them.data_ptr(), white_indices.data_ptr(), black_indices.data_ptr(),
        psqt_indices.data_ptr(), bias.data_ptr(), float(max_ft_activation),
        grad_l0.data_ptr(), grad_wpsqt.data_ptr(), grad_bpsqt.data_ptr(), saved.data_ptr(),
    )
    if mode != "atomic":
        grad_weight = torch.empty(num_rows, output_size, dtype=torch.float32, device=device)
        grad_bias = torch.empty(output_size, dtype=torch.float32, device=device)
        if B == 0:
            return grad_weight.zero_(), grad_bias.zero_()
        row_split = _slf.row_split_of(mode)
        nbytes = lib.nnueft_det_workspace_bytes(B, K, num_rows, output_size, 2, row_split)
        ws = _workspace(nbytes, device)
        # presorted: the lists sorted during the forward pass on the second stream; the entry point makes
        # its reduction (not its first kernel) wait for that stream
        sorted_ptr = presorted.data_ptr() if presorted is not None else None
        rc = lib.nnueft_double_bwd_det(
            *head, grad_weight.data_ptr(), grad_bias.data_ptr(), B, K, num_rows, l1_size, n_psqt, row_split,
            ws.data_ptr(), nbytes, sorted_ptr, _stream_ptr(device),
            _aux_stream_ptr(device) if second_stream else None,
        )
        _native.check(rc, "nnueft_double_bwd_det")
    else:
        grad_weight = torch.zeros(num_rows, output_size, dtype=torch.float32, device=device)
        grad_bias = torch.zeros(output_size, dtype=torch.float32, device=device)
        rc = lib.nnueft_double_bwd_atomic(
            *head, grad_weight.data_ptr(), grad_bias.data_ptr(), B, K, num_rows, l1_size, n_psqt,
            _stream_ptr(device),
        )
        _native.check(rc, "nnueft_double_bwd_atomic")
    return grad_weight, grad_bias


class FusedDoubleFtFunction(autograd.Function):
    @staticmethod
    def forward(ctx, us, them, white_indices, black_indices, psqt_indices, weight, bias, max_ft_activation, l1_size,
                *extra):
        """The reference's nine arguments, and optionally a tenth, act_grid: None, or (scale, eps, post_mul):
        l0 then comes out as (floor(l0 * scale + eps) / scale) * post_mul, the activation grid and
        correction factor that ComposedFeatureTransformer applies next, with a straight-through gradient."""
        if len(extra) > 1:
            raise TypeError("FusedDoubleFtFunction takes nine arguments and optionally act_grid")
        act_grid = extra[0] if extra else None
        ctx.n_extra = len(extra)
        ctx.act_grid = None if act_grid is None else tuple(float(v) for v in act_grid)
        ctx.max_ft_activation = float(max_ft_activation)
        ctx.l1_size = int(l1_size)
        ctx.backward_mode = _slf.get_backward_mode()
        ctx.sort_placement = _slf.get_sort_placement()

        assert l1_size % 2 == 0

        assert us.is_cuda and them.is_cuda
        assert white_indices.is_cuda and black_indices.is_cuda and psqt_indices.is_cuda
        assert weight.is_cuda and bias.is_cuda
        assert (
            us.device == them.device == white_indices.device == black_indices.device
            == psqt_indices.device == weight.device == bias.device
        )

        assert us.dtype == torch.float32 and them.dtype == torch.float32
        assert white_indices.dtype == torch.int32 and black_indices.dtype == torch.int32
        assert psqt_indices.dtype == torch.int64
        assert weight.dtype == torch.float32 and bias.dtype == torch.float32

        assert white_indices.ndim == 2 and black_indices.ndim == 2
        assert psqt_indices.ndim == 1
        assert len(weight.shape) == 2
        assert len(bias.shape) == 1
        assert weight.shape[1] == bias.shape[0]
        assert white_indices.shape == black_indices.shape
        assert white_indices.shape[0] == psqt_indices.shape[0]
        assert us.numel() == white_indices.shape[0] and them.numel() == white_indices.shape[0]
        assert 0 < l1_size <= weight.shape[1]

        assert us.is_contiguous() and them.is_contiguous()
        assert white_indices.is_contiguous() and black_indices.is_contiguous() and psqt_indices.is_contiguous()
        assert weight.is_contiguous() and bias.is_contiguous()

        batch_size = white_indices.shape[0]
        device = us.device

        l0_ = torch.empty(batch_size, l1_size, dtype=torch.float32, device=device)
        wpsqt = torch.empty(batch_size, 1, dtype=torch.float32, device=device)
        bpsqt = torch.empty(batch_size, 1, dtype=torch.float32, device=device)
        row_sums = torch.empty(2, batch_size, l1_size, dtype=torch.float32, device=device)

        with torch.cuda.device(device):
            # first, so that it runs beside the forward kernel
            ctx.presorted = None
            if (ctx.sort_placement == "forward" and ctx.backward_mode != "atomic" and batch_size > 0
                    and (ctx.needs_input_grad[5] or ctx.needs_input_grad[6])):
                ctx.presorted = _launch_det_sort(white_indices, black_indices, weight.shape[0], weight.shape[1],
                                                 _slf.row_split_of(ctx.backward_mode))

            _launch_double_fwd(
                us, them, white_indices, black_indices, psqt_indices, weight, bias,
                max_ft_activation, int(l1_size), l0_, wpsqt, bpsqt, row_sums, ctx.act_grid,
            )

        ctx.save_for_backward(us, them, white_indices, black_indices, psqt_indices, weight, bias, row_sums)
        return l0_, wpsqt, bpsqt

    @staticmethod
    def backward(ctx, grad_l0, grad_wpsqt, grad_bpsqt):
        us, them, white_indices, black_indices, psqt_indices, weight, bias, row_sums = ctx.saved_tensors

        grad_l0 = grad_l0.contiguous()
        grad_wpsqt = grad_wpsqt.contiguous()
        grad_bpsqt = grad_bpsqt.contiguous()
        if ctx.act_grid is not None and ctx.act_grid[2] != 1.0:
            grad_l0 = grad_l0 * ctx.act_grid[2]

        with torch.cuda.device(us.device):
            grad_weight, grad_bias = _launch_double_bwd(
                us, them, white_indices, black_indices, psqt_indices, bias, ctx.max_ft_activation,
                grad_l0, grad_wpsqt, grad_bpsqt, row_sums,
                weight.shape[0], ctx.l1_size, bias.shape[0], ctx.backward_mode, ctx.presorted,
                ctx.sort_placement != "inline",
            )

        return (None, None, None, None, None, grad_weight, grad_bias, None, None) + (None,) * ctx.n_extra
