"""Sparse-input linear layer: out[b] = sum_k weight[indices[b,k]] + bias.

Same names, arguments and error behaviour as the reference's
model/modules/feature_transformer/sparse_linear_functions.py; the CuPy kernels it launches
(:85-99 forward, :118-134 backward) are replaced by libnnueft.so (hand-written HIP for gfx950).

`_HAS_CUPY_KERNELS` keeps its name because callers and the reference's tests test it; here it
means "libnnueft.so is loaded".  The launches are torch custom ops (nnueft/_ops.py), so torch.compile keeps
them inside its graph (the reference's kernels break the graph around themselves).  There is no silent fallback for device tensors: with
backend="auto", tensors on the GPU and no library, apply() raises.  The "torch" backend (and
"auto" on CPU tensors) is the reference's device-agnostic embedding_bag path, unchanged.
"""
import os

import torch
import torch.nn.functional as F
from torch import autograd

from . import _native
from . import _ops

_HAS_CUPY_KERNELS = _native.available()

# "deterministic": sort + segmented reduction (any result of it is one the reference's unordered atomics
#     could have produced, the same bits on every run, and on MI355X it is five times faster than atomics).
#     Table rows named by more than nnueft_row_split() slots of a batch are summed window by window,
#     which differs from the reference's CPU path in the last bits of those rows.
# "deterministic_strict": the same with every row summed in one chain: bit for bit the weight gradient of
#     the reference's CPU path (torch embedding_bag backward under autograd); slower on batches where a
#     few table rows are named by thousands of positions.
# "atomic": the reference's GPU scheme, unordered fp32 atomics.
BACKWARD_MODES = ("atomic", "deterministic", "deterministic_strict")
_BACKWARD_MODE = os.environ.get("NNUEFT_BACKWARD", "deterministic")
if _BACKWARD_MODE not in BACKWARD_MODES:
    raise ValueError(f"NNUEFT_BACKWARD={_BACKWARD_MODE!r}: expected one of {BACKWARD_MODES}")


def set_backward_mode(mode: str) -> None:
    global _BACKWARD_MODE
    if mode not in BACKWARD_MODES:
        raise ValueError(f"Invalid backward mode: {mode}")
    _BACKWARD_MODE = mode


def get_backward_mode() -> str:
    return _BACKWARD_MODE


row_split_of = _ops.row_split_of


# Where the index sort of the fused deterministic backward runs (the results are the same bits):
#   "inline"    on the caller's stream inside the backward pass (default)
#   "backward"  on a second stream inside the backward pass, beside the upstream-rows kernel
#   "forward"   on a second stream, started by the forward pass
# A second stream pays when the FT passes run back to back on an otherwise idle GPU (measured
# 1.27 -> 1.23 ms per forward+backward with "forward").  In a whole training step it loses: the
# sort's kernels take their time out of the kernels they run beside, and the extra stream costs
# host time that a step with many small launches does not have (2.92 -> 3.06 ms).
_SORT_PLACEMENT = os.environ.get("NNUEFT_SORT_PLACEMENT", "inline")


def set_sort_placement(where: str) -> None:
    global _SORT_PLACEMENT
    if where not in ("inline", "backward", "forward"):
        raise ValueError(f"Invalid sort placement: {where}")
    _SORT_PLACEMENT = where


def get_sort_placement() -> str:
    return _SORT_PLACEMENT


# the launches of this file are torch custom ops (nnueft/_ops.py); these helpers serve the launchers of the
# module layer, which dynamo steps around (opaque to it: traced, current_stream() is a torch.Stream proxy
# without a raw handle)
@torch.compiler.disable
def _stream_ptr(device) -> int:
    return _ops.stream_ptr(device)


@torch.compiler.disable
def _aux_stream(device):
    return _ops.aux_stream(device)


@torch.compiler.disable
def _aux_stream_ptr(device) -> int:
    return _ops.aux_stream(device).cuda_stream


_workspace = _ops.workspace


def _torch_sparse_linear(feature_indices, weight, bias):
    """Device-agnostic path of the reference (sparse_linear_functions.py:16-50)."""
    batch_size, max_active = feature_indices.shape
    mask = feature_indices >= 0
    safe_indices = feature_indices.clamp(min=0).long().reshape(-1)
    per_sample_weights = mask.to(weight.dtype).reshape(-1)
    offsets = torch.arange(0, batch_size * max_active, max_active, device=feature_indices.device)
    output = F.embedding_bag(safe_indices, weight, offsets, mode="sum", per_sample_weights=per_sample_weights)
    return output + bias


class _CudaSparseLinearFunction(autograd.Function):
    @staticmethod
    def forward(ctx, feature_indices, weight, bias):
        ctx.save_for_backward(feature_indices, weight, bias)
        ctx.backward_mode = _BACKWARD_MODE

        assert len(feature_indices.shape) == 2
        assert feature_indices.dtype == torch.int32
        assert len(weight.shape) == 2
        assert weight.dtype == torch.float32
        assert len(bias.shape) == 1
        assert bias.dtype == torch.float32
        assert weight.shape[1] == bias.shape[0]

        assert feature_indices.is_cuda
        assert weight.is_cuda
        assert bias.is_cuda
        assert weight.device == feature_indices.device
        assert bias.device == feature_indices.device

        assert feature_indices.is_contiguous()
        assert weight.is_contiguous()
        assert bias.is_contiguous()

        return _ops.launch("sparse_fwd", feature_indices, weight, bias)

    @staticmethod
    def backward(ctx, grad_output):
        assert not ctx.needs_input_grad[0]
        grad_output = grad_output.contiguous()
        feature_indices, weight, _bias = ctx.saved_tensors
        weight_grad, bias_grad = _ops.launch("sparse_bwd", feature_indices, grad_output, weight.shape[0],
                                                             ctx.backward_mode)
        return None, weight_grad, bias_grad


# Allowed modes: "auto", "fused", "sparse", "torch"


class SparseLinearFunction:
    """Hand-written HIP kernels for tensors on the GPU; the torch path for other devices."""

    @staticmethod
    def apply(feature_indices, weight, bias, backend: str = "auto"):
        on_gpu = feature_indices.is_cuda and weight.is_cuda and bias.is_cuda
        if backend == "auto":
            if on_gpu:
                if not _HAS_CUPY_KERNELS:
                    raise RuntimeError(
                        "Tensors are on the GPU but libnnueft.so is not loaded; build it "
                        "(nnueft._build.build()) or request backend='torch' explicitly."
                    )
                return _CudaSparseLinearFunction.apply(feature_indices, weight, bias)
            return _torch_sparse_linear(feature_indices, weight, bias)

        elif backend == "sparse":
            if not _HAS_CUPY_KERNELS:
                raise RuntimeError("Sparse linear kernel library (libnnueft.so) is not available.")
            if not on_gpu:
                raise RuntimeError("Sparse GPU kernel requested but tensors are not on the GPU.")
            return _CudaSparseLinearFunction.apply(feature_indices, weight, bias)

        elif backend == "torch":
            return _torch_sparse_linear(feature_indices, weight, bias)

        else:
            raise ValueError(f"Invalid SparseLinear backend requested: {backend}")
