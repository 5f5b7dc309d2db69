"""Sparse-input linear layer: out[b] = sum_k weight[indices[b,k]] + bias.

Same names, arguments and error behaviour as the reference's
model/modules/feature_transformer/sparse_linear_functions.py; the CuPy kernels it launches
(:85-99 forward, :118-134 backward) are replaced by libnnueft.so (hand-written HIP for gfx950).

`_HAS_CUPY_KERNELS` keeps its name because callers and the reference's tests test it; here it
means "libnnueft.so is loaded".  There is no silent fallback for device tensors: with
backend="auto", tensors on the GPU and no library, apply() raises.  The "torch" backend (and
"auto" on CPU tensors) is the reference's device-agnostic embedding_bag path, unchanged.
"""
import os

import torch
import torch.nn.functional as F
from torch import autograd

from . import _native

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


def row_split_of(mode: str) -> int:
    """The row_split argument of the deterministic entry points for a backward mode.  NNUEFT_ROW_SPLIT in the
    environment replaces the library's threshold for the "deterministic" mode (kernel tuning: the threshold is
    part of the summation order, so results change in the last bits of the rows it moves across)."""
    if mode == "deterministic_strict":
        return 0
    override = os.environ.get("NNUEFT_ROW_SPLIT", "")
    return int(override) if override.isdigit() else _native.load().nnueft_row_split()


def get_backward_mode() -> str:
    return _BACKWARD_MODE


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


@torch.compiler.disable
def _stream_ptr(device) -> int:
    # opaque to dynamo: traced, current_stream() is a torch.Stream proxy without a raw handle
    return torch.cuda.current_stream(device).cuda_stream


_AUX_STREAMS = {}


@torch.compiler.disable
def _aux_stream(device):
    """A second stream per device (default priority) for work that is independent of what runs on the
    caller's stream; whoever uses it orders it against the caller's stream with events."""
    key = torch.device(device).index if torch.device(device).index is not None else torch.cuda.current_device()
    if key not in _AUX_STREAMS:
        _AUX_STREAMS[key] = torch.cuda.Stream(device=key)
    return _AUX_STREAMS[key]


@torch.compiler.disable
def _aux_stream_ptr(device) -> int:
    return _aux_stream(device).cuda_stream


def _workspace(nbytes: int, device) -> torch.Tensor:
    # torch's caching allocator hands out blocks aligned to 512 bytes
    return torch.empty(max(int(nbytes), 1), dtype=torch.uint8, device=device)


def _torch_sparse_linear(feature_indices, weight, bias):
    """Device-agnostic path of the reference (sparse_linear_functions.py:16-50)."""
    batch_size, max_active = feature_indices.shape
    mask = feature_indices >= 0
    safe_indices = feature_indices.clamp(min=0).long().reshape(-1)
    per_sample_weights = mask.to(weight.dtype).reshape(-1)
    offsets = torch.arange(0, batch_size * max_active, max_active, device=feature_indices.device)
    output = F.embedding_bag(safe_indices, weight, offsets, mode="sum", per_sample_weights=per_sample_weights)
    return output + bias


@torch.compiler.disable(recursive=False)
def _launch_sparse_fwd(feature_indices, weight, bias, output):
    lib = _native.load()
    B, K = feature_indices.shape
    R, out_cols = weight.shape
    rc = lib.nnueft_sparse_fwd(
        feature_indices.data_ptr(), weight.data_ptr(), bias.data_ptr(), output.data_ptr(),
        B, K, R, out_cols, _stream_ptr(weight.device),
    )
    _native.check(rc, "nnueft_sparse_fwd")


@torch.compiler.disable(recursive=False)
def _launch_sparse_bwd(feature_indices, grad_output, num_rows, mode):
    lib = _native.load()
    B, K = feature_indices.shape
    out_cols = grad_output.shape[1]
    device = grad_output.device
    if mode != "atomic":
        weight_grad = torch.empty(num_rows, out_cols, dtype=torch.float32, device=device)
        bias_grad = torch.empty(out_cols, dtype=torch.float32, device=device)
        if B == 0:
            return weight_grad.zero_(), bias_grad.zero_()
        row_split = row_split_of(mode)
        nbytes = lib.nnueft_det_workspace_bytes(B, K, num_rows, out_cols, 1, row_split)
        ws = _workspace(nbytes, device)
        rc = lib.nnueft_sparse_bwd_det(
            feature_indices.data_ptr(), grad_output.data_ptr(), weight_grad.data_ptr(), bias_grad.data_ptr(),
            B, K, num_rows, out_cols, row_split, ws.data_ptr(), nbytes, _stream_ptr(device),
        )
        _native.check(rc, "nnueft_sparse_bwd_det")
    else:
        weight_grad = torch.zeros(num_rows, out_cols, dtype=torch.float32, device=device)
        bias_grad = torch.zeros(out_cols, dtype=torch.float32, device=device)
        rc = lib.nnueft_sparse_bwd_atomic(
            feature_indices.data_ptr(), grad_output.data_ptr(), weight_grad.data_ptr(), bias_grad.data_ptr(),
            B, K, num_rows, out_cols, _stream_ptr(device),
        )
        _native.check(rc, "nnueft_sparse_bwd_atomic")
    return weight_grad, bias_grad


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

        output = torch.empty(
            feature_indices.shape[0], weight.shape[1], dtype=torch.float32, device=feature_indices.device
        )
        with torch.cuda.device(weight.device):
            _launch_sparse_fwd(feature_indices, weight, bias, output)
        return output

    @staticmethod
    def backward(ctx, grad_output):
        assert not ctx.needs_input_grad[0]
        grad_output = grad_output.contiguous()
        feature_indices, weight, _bias = ctx.saved_tensors
        with torch.cuda.device(weight.device):
            weight_grad, bias_grad = _launch_sparse_bwd(
                feature_indices, grad_output, weight.shape[0], ctx.backward_mode
            )
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
