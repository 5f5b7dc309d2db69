"""Quantized (int16) feature transformer forward, as the engine evaluates an exported net.

The reference holds no code for this step (it runs inside the chess engine); the tensors are what
QuantizationManager.quantize_feature_transformer_{weights,bias} produce (model/quantize.py:175-204)
and the arithmetic is the one described in docs/nnue.md:1014-1069 and :2097-2134 with the constants
of model/quantize.py:58-73 (one = 256, clip at 255, product >> 9).
"""
import torch

from . import _native
from .sparse_linear_functions import _stream_ptr

FT_QUANTIZED_ONE = 256        # model/quantize.py:66
FT_QUANTIZED_MAX = 255        # model/quantize.py:67
L0_SHIFT = 9                  # inference_l0_division_factor = 512, model/quantize.py:72
PSQT_SCALE = 600.0 * 16.0     # nnue2score * weight_scale_out, model/quantize.py:107


def _safe_round_to(value: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    """round, then convert; raises when a value does not fit the symmetric range (model/quantize.py:18-34)."""
    limit = torch.iinfo(dtype).max
    rounded = value.round()
    bad = int(((rounded < -limit) | (rounded > limit)).sum().item())
    if bad > 0:
        raise RuntimeError(
            f"Found {bad} out of bounds values when converting to target dtype {dtype}. "
            f"Min: {rounded.min().item()}, max: {rounded.max().item()}."
        )
    return rounded.to(dtype)


def quantize_feature_transformer(weight: torch.Tensor, bias: torch.Tensor, l1_size: int):
    """float [R, L1+n_psqt] table and [L1+n_psqt] bias -> (int16 [R,L1], int16 [L1], int32 [R,n_psqt])."""
    w16 = _safe_round_to(weight[:, :l1_size] * float(FT_QUANTIZED_ONE), torch.int16).contiguous()
    b16 = _safe_round_to(bias[:l1_size] * float(FT_QUANTIZED_ONE), torch.int16).contiguous()
    p32 = _safe_round_to(weight[:, l1_size:] * PSQT_SCALE, torch.int32).contiguous()
    return w16, b16, p32


def ft_int16_forward(white_indices, black_indices, stm, w16, b16, psqt32, psqt_indices,
                     clip_max: int = FT_QUANTIZED_MAX, shift: int = L0_SHIFT, table_block_rows: int = 0,
                     use_workspace: bool = True):
    """Returns (u8 [B, L1] with the side to move's half first, int32 [B] psqt difference / 2).

    stm: uint8 [B], 0 = white to move, 1 = black to move.
    table_block_rows: rows per king bucket of the table (scheduling hint); 0 picks 704 for the
    22528-row exported table and 768 otherwise.
    """
    assert white_indices.is_cuda, "the quantized path has a GPU implementation only"
    assert white_indices.dtype == torch.int32 and black_indices.dtype == torch.int32
    assert white_indices.shape == black_indices.shape and white_indices.ndim == 2
    assert stm.dtype == torch.uint8 and stm.ndim == 1
    assert w16.dtype == torch.int16 and b16.dtype == torch.int16 and psqt32.dtype == torch.int32
    assert psqt_indices.dtype == torch.int64 and psqt_indices.ndim == 1
    assert w16.ndim == 2 and b16.ndim == 1 and w16.shape[1] == b16.shape[0]
    assert psqt32.ndim == 2 and psqt32.shape[0] == w16.shape[0]
    assert w16.shape[1] % 2 == 0
    assert (clip_max * clip_max) >> shift <= 255
    for t in (white_indices, black_indices, stm, w16, b16, psqt32, psqt_indices):
        assert t.is_contiguous() and t.device == white_indices.device
    B, K = white_indices.shape
    assert stm.shape[0] == B and psqt_indices.shape[0] == B
    R, L1 = w16.shape
    device = white_indices.device
    out = torch.empty(B, L1, dtype=torch.uint8, device=device)
    psqt = torch.empty(B, dtype=torch.int32, device=device)
    lib = _native.load()
    if table_block_rows == 0 and R == 22528:
        table_block_rows = 704
    nbytes = lib.nnueft_int16_workspace_bytes(B, K, R, L1, table_block_rows) if (use_workspace and B > 0) else 0
    ws = torch.empty(max(nbytes, 1), dtype=torch.uint8, device=device)
    with torch.cuda.device(device):
        rc = lib.nnueft_ft_int16_fwd(
            white_indices.data_ptr(), black_indices.data_ptr(), stm.data_ptr(), w16.data_ptr(), b16.data_ptr(),
            psqt32.data_ptr(), psqt_indices.data_ptr(), out.data_ptr(), psqt.data_ptr(),
            B, K, R, L1, psqt32.shape[1], int(clip_max), int(shift), int(table_block_rows),
            ws.data_ptr() if nbytes else None, nbytes, _stream_ptr(device),
        )
    _native.check(rc, "nnueft_ft_int16_fwd")
    return out, psqt


def quantize_layer_stacks(layer_stacks, quantization=None):
    """LayerStacks (nnueft.model) -> the six integer tensors nnueft_stack_int8_fwd takes: int8 weights and
    int32 biases at the scales of QuantizationManager.quantize_fc_layer (model/quantize.py:218-236), the
    factorised first layer folded in.  Raises when a value does not fit."""
    q = quantization or layer_stacks.quantization
    d = q.weight_scales_dict
    w1, b1 = layer_stacks.l1._params()
    out = []
    for (w, b), key in (((w1, b1), "ls_l1"), ((layer_stacks.l2.linear.weight, layer_stacks.l2.linear.bias), "ls_l2"),
                        ((layer_stacks.output.linear.weight, layer_stacks.output.linear.bias), "ls_output")):
        out.append(_safe_round_to(w.detach() * d[f"{key}_weight"], torch.int8).contiguous())
        out.append(_safe_round_to(b.detach() * d[f"{key}_bias"], torch.int32).contiguous())
    return tuple(out)


def stack_int8_forward(x_u8, bucket, w1, b1, w2, b2, wo, bo, lin_shift1=7, sqr_shift1=21, lin_shift2=6,
                       sqr_shift2=19, act_max=127, out_mult=9600, out_den=32768):
    """int32 [B]: the stack output at scale out_mult (9600 = nnue2score * 16) for u8 inputs [B, L1]."""
    assert x_u8.is_cuda and x_u8.dtype == torch.uint8 and x_u8.ndim == 2 and x_u8.is_contiguous()
    assert bucket.dtype == torch.int64 and bucket.shape == (x_u8.shape[0],)
    for w, b in ((w1, b1), (w2, b2), (wo, bo)):
        assert w.dtype == torch.int8 and b.dtype == torch.int32 and w.is_contiguous() and b.is_contiguous()
        assert w.device == x_u8.device and b.device == x_u8.device
    B, L1 = x_u8.shape
    count = bo.shape[0]
    L2, L3 = w1.shape[0] // count, w2.shape[0] // count
    assert w1.shape == (count * L2, L1) and w2.shape == (count * L3, 2 * L2) and wo.shape == (count, 2 * L2 + 2 * L3)
    out = torch.empty(B, dtype=torch.int32, device=x_u8.device)
    lib = _native.load()
    with torch.cuda.device(x_u8.device):
        rc = lib.nnueft_stack_int8_fwd(
            x_u8.data_ptr(), bucket.data_ptr(), w1.data_ptr(), b1.data_ptr(), w2.data_ptr(), b2.data_ptr(),
            wo.data_ptr(), bo.data_ptr(), out.data_ptr(), B, L1, L2, L3, count, lin_shift1, sqr_shift1, lin_shift2,
            sqr_shift2, act_max, out_mult, out_den, _stream_ptr(x_u8.device),
        )
    _native.check(rc, "nnueft_stack_int8_fwd")
    return out
