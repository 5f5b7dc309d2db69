"""Host-side mirror of the reference interface: dispatch, errors, the device-agnostic path (CPU only)."""
import numpy as np
import pytest
import torch

import nnueft
from _cases import double_case, sparse_case
from nnueft.double_ft_functions import double_feature_transform
from nnueft.sparse_linear_functions import SparseLinearFunction, _torch_sparse_linear
from nnueft import quantized


def test_public_names_of_the_reference_package():
    # model/modules/feature_transformer/__init__.py:6-11 (ComposedFeatureTransformer stays the caller's)
    for name in ("FusedDoubleFtFunction", "SparseLinearFunction", "double_feature_transform"):
        assert hasattr(nnueft, name)
    from nnueft import fused_ft_functions, sparse_linear_functions

    assert isinstance(sparse_linear_functions._HAS_CUPY_KERNELS, bool)
    assert isinstance(fused_ft_functions._HAS_CUPY_KERNELS, bool)
    assert fused_ft_functions.BACKWARD_TILE_SIZE >= 1


def test_sparse_cpu_matches_dense_emulation_like_the_reference_test(oracle_cpu):
    # tests/test_feature_transformer.py:35-78 on the CPU device
    torch.manual_seed(0)
    w0 = torch.rand(10, 128, requires_grad=True)
    b0 = torch.rand(128, requires_grad=True)
    idx = (torch.rand(16, 32) * 10).to(torch.int32)
    out = SparseLinearFunction.apply(idx, w0, b0)
    dense = torch.zeros(16, 10)
    for i in range(16):
        for j in range(32):
            dense[i, idx[i, j]] += 1.0
    w1 = w0.detach().clone().requires_grad_()
    b1 = b0.detach().clone().requires_grad_()
    ref = torch.mm(dense, w1) + b1
    assert torch.max(torch.abs(out - ref)) < 1e-4
    out.sum().backward()
    ref.sum().backward()
    assert torch.max(torch.abs(w0.grad - w1.grad)) < 1e-4
    assert torch.max(torch.abs(b0.grad - b1.grad)) < 1e-4
    assert np.array_equal(out.detach().numpy(), oracle_cpu.sparse_fwd(idx.numpy(), w0.detach().numpy(), b0.detach().numpy()))


def test_backend_errors_match_the_reference():
    c = sparse_case(1, 4, 16, 10, 8)
    idx, W, b = torch.from_numpy(c["idx"]), torch.from_numpy(c["W"]), torch.from_numpy(c["bias"])
    with pytest.raises(ValueError):
        SparseLinearFunction.apply(idx, W, b, backend="nope")
    with pytest.raises(RuntimeError):
        SparseLinearFunction.apply(idx, W, b, backend="sparse")      # CPU tensors
    assert torch.equal(SparseLinearFunction.apply(idx, W, b, backend="torch"), _torch_sparse_linear(idx, W, b))
    assert torch.equal(SparseLinearFunction.apply(idx, W, b), _torch_sparse_linear(idx, W, b))

    d = double_case(2, 4, 16, 20, 8)
    args = [torch.from_numpy(d[k]) for k in ("us", "them", "widx", "bidx", "psqt_idx", "W", "bias")]
    with pytest.raises(ValueError):
        double_feature_transform(*args, 1.0, 16, "nope")
    for backend in ("fused", "sparse"):
        with pytest.raises(RuntimeError):
            double_feature_transform(*args, 1.0, 16, backend)     # CPU tensors
    with pytest.raises(AssertionError):
        double_feature_transform(*args, 1.0, 15, "torch")          # odd l1_size
    a = double_feature_transform(*args, 1.0, 16, "torch")
    b2 = double_feature_transform(*args, 1.0, 16)                   # auto on CPU tensors = torch
    for x, y in zip(a, b2):
        assert torch.equal(x, y)


def test_torch_backend_equals_oracle(oracle_cpu):
    d = double_case(3, 33, 64, 200)
    args = [torch.from_numpy(d[k]) for k in ("us", "them", "widx", "bidx", "psqt_idx", "W", "bias")]
    l0, wp, bp = double_feature_transform(*args, d["max_act"], 64, "torch")
    r = oracle_cpu.double_fwd(d["us"], d["them"], d["widx"], d["bidx"], d["psqt_idx"], d["W"], d["bias"], d["max_act"], 64)
    assert np.array_equal(l0.numpy(), r[0]) and np.array_equal(wp.numpy(), r[1]) and np.array_equal(bp.numpy(), r[2])


def test_backward_mode_switch():
    assert nnueft.get_backward_mode() in ("atomic", "deterministic")
    old = nnueft.get_backward_mode()
    nnueft.set_backward_mode("deterministic")
    assert nnueft.get_backward_mode() == "deterministic"
    with pytest.raises(ValueError):
        nnueft.set_backward_mode("fast")
    nnueft.set_backward_mode(old)


def test_quantize_helpers_follow_quantize_py():
    # model/quantize.py:66-73 and :98-107
    assert quantized.FT_QUANTIZED_ONE == 256 and quantized.FT_QUANTIZED_MAX == 255
    assert (255 * 255) >> quantized.L0_SHIFT == 127
    assert quantized.PSQT_SCALE == 9600.0
    W = torch.tensor([[0.5, -0.25, 1.0 / 9600.0, 0.0], [1.0 / 256.0, 127.0, 0.1, -0.1]])
    b = torch.tensor([0.25, -1.0, 0.0, 0.0])
    w16, b16, p32 = quantized.quantize_feature_transformer(W, b, 2)
    assert w16.tolist() == [[128, -64], [1, 32512]] and w16.dtype == torch.int16
    assert b16.tolist() == [64, -256]
    assert p32.tolist() == [[1, 0], [960, -960]] and p32.dtype == torch.int32
    with pytest.raises(RuntimeError, match="out of bounds"):
        quantized.quantize_feature_transformer(torch.tensor([[128.0, 0.0]]), torch.zeros(2), 1)   # 128*256 > 32767
