"""Fused two-perspective feature transformer as an autograd function.

Same name, argument order, outputs and assertions as the reference's
model/modules/feature_transformer/fused_ft_functions.py:18-122; the two CuPy kernels it launches
are replaced by nnueft_double_fwd / nnueft_double_bwd_{atomic,det} of libnnueft.so.

Differences that a caller can observe:
  * the activation tensor kept for the backward holds the two perspectives' row sums (the reference
    keeps the clamped mixed values, fused_ft_kernel.py:95-99); the backward recomputes the mix from
    them, so the clamp passes gradient at exactly 0 and exactly max like torch.clamp does in the
    reference's CPU path;
  * the launches are torch custom ops (nnueft/_ops.py): under torch.compile the operator stays inside the
    compiled graph, where the reference's CuPy launches break the graph (fused_ft_kernel.py:12);
  * the backward mode (NNUEFT_BACKWARD or set_backward_mode): "deterministic" (default) and
    "deterministic_strict" give results that do not depend on scheduling, the strict one bit for bit
    the weight gradient of the reference's CPU path; "atomic" is the reference's GPU scheme.
"""
import torch
from torch import autograd

from . import _native
from . import _ops
from . import sparse_linear_functions as _slf

_HAS_CUPY_KERNELS = _native.available()

# Positions a wave of the atomic backward walks before it flushes its bias partial sums
# (fused_ft_kernel.py:127 has the same constant for the reference's kernel).
BACKWARD_TILE_SIZE = 4


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

        # first, so that it runs beside the forward kernel (a second stream: eager mode only)
        ctx.presorted = None
        if (ctx.sort_placement == "forward" and ctx.backward_mode != "atomic" and batch_size > 0
                and (ctx.needs_input_grad[5] or ctx.needs_input_grad[6]) and not torch.compiler.is_compiling()):
            ctx.presorted = _ops.launch("det_sort", white_indices, black_indices, weight.shape[0], weight.shape[1],
                                                      _slf.row_split_of(ctx.backward_mode))

        act = ctx.act_grid if ctx.act_grid is not None else (1.0, 0.0, 1.0)
        l0_, wpsqt, bpsqt, row_sums = _ops.launch("double_fwd", 
            us, them, white_indices, black_indices, psqt_indices, weight, bias, ctx.max_ft_activation, ctx.l1_size,
            ctx.act_grid is not None, act[0], act[1], act[2])

        ctx.save_for_backward(us, them, white_indices, black_indices, psqt_indices, weight, bias, row_sums)
        return l0_, wpsqt, bpsqt

    @staticmethod
    def backward(ctx, grad_l0, grad_wpsqt, grad_bpsqt):
        us, them, white_indices, black_indices, psqt_indices, weight, bias, row_sums = ctx.saved_tensors

        if ctx.act_grid is not None and ctx.act_grid[2] != 1.0:
            grad_l0 = grad_l0 * ctx.act_grid[2]

        second_stream = ctx.sort_placement != "inline" and not torch.compiler.is_compiling()
        grad_weight, grad_bias = _ops.launch("double_bwd", 
            us, them, white_indices, black_indices, psqt_indices, bias, ctx.max_ft_activation,
            grad_l0, grad_wpsqt, grad_bpsqt, row_sums,
            weight.shape[0], ctx.l1_size, bias.shape[0], ctx.backward_mode, ctx.presorted, second_stream)

        return (None, None, None, None, None, grad_weight, grad_bias, None, None) + (None,) * ctx.n_extra
