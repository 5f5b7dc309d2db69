"""The callers of the feature transformer, restated for the full-model step (BASELINE config 4).

These are the modules that sit directly above the operator in the reference; they are written
against the same public names so that code using the reference's classes reads the same:

  QuantizationConfig, QuantizationManager   model/quantize.py:58-113 (constants), :36-56 (fake quantization)
  HalfKav2Hm                                model/modules/features/halfka_v2_hm.py:39-170
  ComposedFeatureTransformer                model/modules/feature_transformer/composed_feature_transformer.py:12-151
  StackedLinear, FactorizedStackedLinear    model/modules/stacked_linear.py
  LayerStacks                               model/modules/layer_stacks.py:11-84
  NNUEModel                                 model/model.py:9-133
  sf_loss                                   model/nnue.py:39-70 (calculate_sf_loss; tablebase remap :19-36)

What differs from the reference: on the GPU the table-side work of the feature transformer (real +
virtual weights, fake quantization of both column groups, concatenation; five or more passes over a
300 MB table in torch ops) is one HIP kernel, nnueft_table_merge, and the gradient of the virtual
weights is one more, nnueft_table_virtual_grad.  Values are bit-identical to the torch ops.
The dense layer stacks stay torch (small GEMMs through hipBLASLt).
"""
import math
from dataclasses import dataclass, field

import torch
import torch.nn.functional as F
from torch import nn

from . import _native, _ops
from . import halfka_v2_hm as hk
from .double_ft_functions import double_feature_transform
from .fused_ft_functions import FusedDoubleFtFunction
from .sparse_linear_functions import _stream_ptr

FAKE_QUANTIZE_EPS = 1e-5


# ------------------------------------------------------------------------------------------ quantization

@dataclass
class QuantizationConfig:
    nnue2score: float = 600.0
    weight_scale_l1: float = 128.0
    weight_scale_l2: float = 64.0
    weight_scale_l_out: float = 128
    weight_scale_out: float = 16.0
    weight_quantized_max_hidden: float = 127.0
    ft_quantized_one: float = 256.0
    ft_quantized_max: float = 255.0
    hidden_quantized_one: float = 128.0
    hidden_quantized_max: float = 127.0
    inference_l0_division_factor: float = 512.0
    inference_sqr_crelu_division_factor: float = 128.0


def _ste(hard: torch.Tensor, value: torch.Tensor) -> torch.Tensor:
    """Forward value `hard`, gradient of the identity (straight-through estimator)."""
    return hard.detach() + (value - value.detach())


class QuantizationManager:
    def __init__(self, config: QuantizationConfig):
        c = self.config = config
        self.nnue2score = c.nnue2score
        self.weight_scale_hidden = [c.weight_scale_l1, c.weight_scale_l2, c.weight_scale_l_out]
        self.weight_scale_out = c.weight_scale_out
        self.hidden_quantized_one = c.hidden_quantized_one
        self.ft_quantized_one = c.ft_quantized_one
        self.max_hidden_weight = [c.weight_quantized_max_hidden / s for s in self.weight_scale_hidden]
        self.l0_correction_factor = c.ft_quantized_one ** 2 / c.inference_l0_division_factor / c.hidden_quantized_one
        self.sqr_crelu_correction_factor = c.hidden_quantized_one / c.inference_sqr_crelu_division_factor
        self.max_ft_activation = c.ft_quantized_max / c.ft_quantized_one
        self.max_hidden_activation = c.hidden_quantized_max / c.hidden_quantized_one
        one = c.hidden_quantized_one
        self.weight_scales_dict = {
            "ft_weight": c.ft_quantized_one,
            "ft_bias": c.ft_quantized_one,
            "ft_psqt_weight": c.nnue2score * c.weight_scale_out,
            "ls_l1_weight": c.weight_scale_l1,
            "ls_l1_bias": c.weight_scale_l1 * one,
            "ls_l2_weight": c.weight_scale_l2,
            "ls_l2_bias": c.weight_scale_l2 * one,
            "ls_output_weight": c.weight_scale_l_out,
            "ls_output_bias": c.weight_scale_l_out * one,
        }

    def clip_ft_act(self, x):
        return torch.clamp(x, 0.0, self.max_ft_activation)

    def clip_ls_act(self, x):
        return torch.clamp(x, 0, self.max_hidden_activation)

    def fake_quantize_weights(self, tensor, key: str):
        scale = self.weight_scales_dict[key]
        return _ste(tensor.mul(scale).round().div(scale), tensor)

    def _fake_quantize_acts(self, x):
        scale = self.config.hidden_quantized_one
        return _ste(x.mul(scale).add(FAKE_QUANTIZE_EPS).floor().div(scale), x)

    fake_quantize_ft_act = _fake_quantize_acts
    fake_quantize_ls_act = _fake_quantize_acts

    def fake_quantize_skip_act(self, x):
        return x

    def output_quantization(self):
        """(den, mult) of fake_quantize_output."""
        mult = int(self.config.nnue2score * self.config.weight_scale_out)
        den = int(self.config.hidden_quantized_one * self.config.weight_scale_l_out * 2.0)
        return den, mult

    def fake_quantize_output(self, x):
        den, mult = self.output_quantization()
        q = torch.div(torch.round(x * den).to(torch.int64) * mult, den, rounding_mode="trunc")
        return _ste(q.to(x.dtype) / float(mult), x)


# ------------------------------------------------------------------------------------------ feature block

def _export_row_map():
    """For every row of the 22528-row exported table, the row of the 24576-row training table it comes
    from: ten piece-type blocks copied, the king block taken from the opposing-king rows except on the
    bucket's own king square, which comes from the own-king row (halfka_v2_hm.py:104-135)."""
    inverse_bucket = {int(b): sq for sq, b in enumerate(hk.KING_BUCKETS) if b >= 0}
    src = torch.empty(hk.NUM_INPUTS_EXPORT, dtype=torch.long)
    for b in range(hk.NUM_BUCKETS):
        s0, d0 = b * hk.NUM_PLANES, b * 704
        src[d0:d0 + 640] = torch.arange(s0, s0 + 640)
        src[d0 + 640:d0 + 704] = torch.arange(s0 + 704, s0 + 768)
        ksq = inverse_bucket[b]
        src[d0 + 640 + ksq] = s0 + 640 + ksq
    return src


class HalfKav2Hm(nn.Module):
    HASH = 0x7F234CB8
    FEATURE_NAME = "HalfKAv2_hm^"
    INPUT_FEATURE_NAME = "HalfKAv2_hm"
    MAX_ACTIVE_FEATURES = hk.MAX_ACTIVE_FEATURES
    NUM_PLANES = hk.NUM_PLANES
    NUM_BUCKETS = hk.NUM_BUCKETS
    NUM_INPUTS = hk.NUM_INPUTS
    NUM_INPUTS_VIRTUAL = hk.NUM_PLANES
    NUM_REAL_FEATURES = hk.NUM_INPUTS_EXPORT

    def __init__(self, num_outputs: int):
        super().__init__()
        self.num_outputs = num_outputs
        self.weight = nn.Parameter(torch.empty(self.NUM_INPUTS, num_outputs))
        self.virtual_weight = nn.Parameter(torch.zeros(self.NUM_INPUTS_VIRTUAL, num_outputs))
        sigma = math.sqrt(1 / self.NUM_INPUTS)
        with torch.no_grad():
            self.weight.uniform_(-sigma, sigma)

    def merged_weight(self):
        return self.weight + self.virtual_weight.repeat(self.NUM_BUCKETS, 1)

    @torch.no_grad()
    def zero_virtual_weights(self):
        self.virtual_weight.zero_()

    @torch.no_grad()
    def coalesce(self):
        self.weight.add_(self.virtual_weight.repeat(self.NUM_BUCKETS, 1))
        self.zero_virtual_weights()

    @staticmethod
    def halfka_psqts():
        """Initial PSQT value of every table row: +value for an own piece, -value for an opposing one."""
        values = {hk.PAWN: 126, hk.KNIGHT: 781, hk.BISHOP: 825, hk.ROOK: 1276, hk.QUEEN: 2538}
        out = [0] * hk.NUM_INPUTS
        for ksq in range(64):
            for sq in range(64):
                for pt, val in values.items():
                    out[hk.feature_index(hk.WHITE, ksq, sq, pt, hk.WHITE)] = val
                    out[hk.feature_index(hk.WHITE, ksq, sq, pt, hk.BLACK)] = -val
        return out

    @torch.no_grad()
    def init_weights(self, num_psqt_buckets: int, nnue2score: float):
        self.zero_virtual_weights()
        col = torch.tensor(self.halfka_psqts(), dtype=self.weight.dtype, device=self.weight.device) / nnue2score
        l1 = self.num_outputs - num_psqt_buckets
        self.weight[:, l1:] = col[:, None]

    @torch.no_grad()
    def get_export_weights(self):
        merged = self.merged_weight()
        return merged[_export_row_map().to(merged.device)]

    @torch.no_grad()
    def load_export_weights(self, export_weight):
        src = _export_row_map().to(export_weight.device)
        full = export_weight.new_zeros(self.NUM_INPUTS, export_weight.shape[1])
        full[src] = export_weight
        self.weight.data.copy_(full)
        self.zero_virtual_weights()

    def clip_weights(self, quantization):
        pass


def get_feature_cls(name: str):
    if name in ("HalfKAv2_hm", "HalfKAv2_hm^"):
        return [HalfKav2Hm]
    raise ValueError(f"feature set {name} is not part of this build (HalfKAv2_hm only)")


# ------------------------------------------------------------------------------------------ FT module

def _launch_table_merge(weight, virtual, l1_size, scale_ft, scale_psqt, quantize):
    return _ops.launch("table_merge", weight, virtual, int(l1_size), float(scale_ft), float(scale_psqt), bool(quantize))


def _launch_table_virtual_grad(grad, vrows):
    return _ops.launch("table_virtual_grad", grad, int(vrows))


class _TableMerge(torch.autograd.Function):
    """merged = q(weight + virtual[row % 768]) in one pass; STE gradient: weight gets the incoming
    gradient itself, virtual its sum over the table blocks.  The launches are torch custom ops
    (nnueft/_ops.py), so a compiled graph keeps them inside."""

    @staticmethod
    def forward(ctx, weight, virtual, l1_size, scale_ft, scale_psqt, quantize):
        ctx.vrows = None if virtual is None else virtual.shape[0]
        return _launch_table_merge(weight, virtual, l1_size, scale_ft, scale_psqt, quantize)

    @staticmethod
    def backward(ctx, grad):
        grad = grad.contiguous()
        gv = None
        if ctx.vrows is not None and ctx.needs_input_grad[1]:
            gv = _launch_table_virtual_grad(grad, ctx.vrows)
        return grad, gv, None, None, None, None


def _table_merge(weight, virtual, l1_size, scale_ft, scale_psqt, quantize):
    return _TableMerge.apply(weight, virtual, l1_size, scale_ft, scale_psqt, quantize)


# FOLD_TABLE_MERGE: whether ComposedFeatureTransformer lets the forward kernel merge real and virtual weights on
# their way into LDS (no merged table in memory, no merge pass) where the library can; False keeps the separate
# pass.  Both give the same bits.
FOLD_TABLE_MERGE = True


@torch.compiler.assume_constant_result
def _virtual_fits(B: int, K: int, R: int, l1_size: int, n_psqt: int, vrows: int, device_index: int) -> bool:
    """Whether the library can merge the virtual weights inside its forward for these sizes on that device: a
    host-side question about shapes and the device, so a traced graph takes the answer as a constant."""
    if not (FOLD_TABLE_MERGE and _native.available()) or B <= 0:
        return False
    with torch.cuda.device(device_index):
        return _native.load().nnueft_double_fwd_virtual_fits(B, K, R, l1_size, n_psqt, vrows) == 1


def _virtual_forward_fits(white_indices, weight, virtual, l1_size) -> bool:
    if not weight.is_cuda:
        return False
    B, K = white_indices.shape
    R, cols = weight.shape
    index = weight.device.index if weight.device.index is not None else torch.cuda.current_device()
    return _virtual_fits(int(B), int(K), int(R), int(l1_size), int(cols - l1_size), int(virtual.shape[0]), int(index))


def _launch_double_fwd_virtual(us, them, white_indices, black_indices, psqt_indices, weight, virtual, bias,
                               max_ft_activation, l1_size, scale_ft, scale_psqt, quantize, act_grid):
    act = act_grid if act_grid is not None else (1.0, 0.0, 1.0)
    return _ops.launch("double_fwd_virtual", us, them, white_indices, black_indices, psqt_indices, weight, virtual, bias,
                       float(max_ft_activation), int(l1_size), float(scale_ft), float(scale_psqt), bool(quantize),
                       act_grid is not None, float(act[0]), float(act[1]), float(act[2]))


class _FusedDoubleFtVirtual(torch.autograd.Function):
    """FusedDoubleFtFunction over the table q(weight + virtual[row % 768]) without that table ever being
    written: the forward kernel merges while it fills its LDS tiles.  The backward is FusedDoubleFtFunction's
    (it never reads the table); the merge's straight-through gradient hands its weight gradient to `weight`
    as it is and to `virtual` summed over the table blocks."""

    @staticmethod
    def forward(ctx, us, them, white_indices, black_indices, psqt_indices, weight, virtual, bias, max_ft_activation,
                l1_size, scale_ft, scale_psqt, quantize, act_grid):
        from . import sparse_linear_functions as _slf

        ctx.act_grid = None if act_grid is None else tuple(float(v) for v in act_grid)
        ctx.max_ft_activation = float(max_ft_activation)
        ctx.l1_size = int(l1_size)
        ctx.backward_mode = _slf.get_backward_mode()
        ctx.sort_placement = _slf.get_sort_placement()
        ctx.shape = tuple(weight.shape)
        ctx.vrows = virtual.shape[0]
        for t in (us, them, white_indices, black_indices, psqt_indices, weight, virtual, bias):
            assert t.is_cuda and t.is_contiguous() and t.device == weight.device
        assert weight.dtype == torch.float32 and virtual.dtype == torch.float32 and bias.dtype == torch.float32
        assert virtual.shape[1] == weight.shape[1] == bias.shape[0]
        l0_, wpsqt, bpsqt, row_sums = _launch_double_fwd_virtual(
            us, them, white_indices, black_indices, psqt_indices, weight, virtual, bias, ctx.max_ft_activation,
            ctx.l1_size, scale_ft, scale_psqt, quantize, ctx.act_grid)
        ctx.save_for_backward(us, them, white_indices, black_indices, psqt_indices, bias, row_sums)
        return l0_, wpsqt, bpsqt

    @staticmethod
    def backward(ctx, grad_l0, grad_wpsqt, grad_bpsqt):

        us, them, white_indices, black_indices, psqt_indices, bias, row_sums = ctx.saved_tensors
        if ctx.act_grid is not None and ctx.act_grid[2] != 1.0:
            grad_l0 = grad_l0 * ctx.act_grid[2]
        second_stream = ctx.sort_placement != "inline" and not torch.compiler.is_compiling()
        grad_weight, grad_bias = _ops.launch(
            "double_bwd", us, them, white_indices, black_indices, psqt_indices, bias, ctx.max_ft_activation,
            grad_l0, grad_wpsqt, grad_bpsqt, row_sums, ctx.shape[0], ctx.l1_size, ctx.shape[1], ctx.backward_mode,
            None, second_stream)
        grad_virtual = _launch_table_virtual_grad(grad_weight, ctx.vrows) if ctx.needs_input_grad[6] else None
        return (None, None, None, None, None, grad_weight, grad_virtual, grad_bias, None, None, None, None, None, None)


def _launch_act_fake_quantize(x, scale, post_mul):
    return _ops.launch("act_fake_quantize", x, float(scale), float(FAKE_QUANTIZE_EPS), float(post_mul))


class _ActFakeQuantize(torch.autograd.Function):
    """(floor(x * scale + eps) / scale) * post_mul in one pass; the straight-through estimator leaves
    the gradient as it comes, times post_mul."""

    @staticmethod
    def forward(ctx, x, scale, post_mul):
        ctx.post_mul = float(post_mul)
        return _launch_act_fake_quantize(x.contiguous(), scale, post_mul)

    @staticmethod
    def backward(ctx, grad):
        return (grad if ctx.post_mul == 1.0 else grad * ctx.post_mul), None, None


def _fused_tail_applies(x) -> bool:
    return x.is_cuda and x.dtype == torch.float32


@torch.compiler.disable(recursive=False)
def _launch_sqr_crelu(x, want_skip, scale, c, m, fq):
    lib = _native.load()
    B, n = x.shape
    y = torch.empty(B, 2 * n, dtype=x.dtype, device=x.device)
    skip = torch.empty(B, 1, dtype=x.dtype, device=x.device) if want_skip else None
    if B:
        with torch.cuda.device(x.device):
            rc = lib.nnueft_sqr_crelu_fwd(x.data_ptr(), y.data_ptr(), skip.data_ptr() if want_skip else None, B, n,
                                          float(scale), float(FAKE_QUANTIZE_EPS), float(c), float(m), int(fq),
                                          _stream_ptr(x.device))
        _native.check(rc, "nnueft_sqr_crelu_fwd")
    return y, skip


@torch.compiler.disable(recursive=False)
def _launch_sqr_crelu_bwd(x, gy, gskip, scale, c, m, fq):
    lib = _native.load()
    B, n = x.shape
    gx = torch.empty_like(x)
    if B:
        with torch.cuda.device(x.device):
            rc = lib.nnueft_sqr_crelu_bwd(x.data_ptr(), gy.data_ptr(), None if gskip is None else gskip.data_ptr(),
                                          gx.data_ptr(), B, n, float(scale), float(FAKE_QUANTIZE_EPS), float(c),
                                          float(m), int(fq), _stream_ptr(x.device))
        _native.check(rc, "nnueft_sqr_crelu_bwd")
    return gx


class _SqrCrelu(torch.autograd.Function):
    """clamp(cat[fq(x^2) * c, fq(x)], 0, m) and, on request, the skip value x[:, -2] - x[:, -1], as one
    kernel; fq is straight-through."""

    @staticmethod
    def forward(ctx, x, want_skip, scale, c, m, fq):
        x = x.contiguous()
        ctx.save_for_backward(x)
        ctx.args = (float(scale), float(c), float(m), bool(fq))
        ctx.want_skip = bool(want_skip)
        return _launch_sqr_crelu(x, want_skip, scale, c, m, fq)

    @staticmethod
    def backward(ctx, gy, gskip):
        (x,) = ctx.saved_tensors
        if gy is None:
            gy = torch.zeros(x.shape[0], 2 * x.shape[1], dtype=x.dtype, device=x.device)
        gskip = gskip.contiguous() if (ctx.want_skip and gskip is not None) else None
        return _launch_sqr_crelu_bwd(x, gy.contiguous(), gskip, *ctx.args), None, None, None, None, None


@torch.compiler.disable(recursive=False)
def _launch_stack_output(lin, skip, wpsqt, bpsqt, us, den, mult, fq):
    lib = _native.load()
    B = lin.shape[0]
    net = torch.empty_like(lin)
    if B:
        with torch.cuda.device(lin.device):
            rc = lib.nnueft_stack_output_fwd(lin.data_ptr(), skip.data_ptr(), wpsqt.data_ptr(), bpsqt.data_ptr(),
                                             us.data_ptr(), net.data_ptr(), B, int(den), int(mult), int(fq),
                                             _stream_ptr(lin.device))
        _native.check(rc, "nnueft_stack_output_fwd")
    return net


@torch.compiler.disable(recursive=False)
def _launch_stack_output_bwd(g, us):
    lib = _native.load()
    gw, gb = torch.empty_like(g), torch.empty_like(g)
    if g.shape[0]:
        with torch.cuda.device(g.device):
            rc = lib.nnueft_stack_output_bwd(g.data_ptr(), us.data_ptr(), gw.data_ptr(), gb.data_ptr(), g.shape[0],
                                             _stream_ptr(g.device))
        _native.check(rc, "nnueft_stack_output_bwd")
    return gw, gb


class _StackOutput(torch.autograd.Function):
    """fq_out(lin + skip) + (wpsqt - bpsqt) * (us - 0.5) as one kernel; fq_out is straight-through."""

    @staticmethod
    def forward(ctx, lin, skip, wpsqt, bpsqt, us, den, mult, fq):
        lin, skip, wpsqt, bpsqt, us = (t.contiguous() for t in (lin, skip, wpsqt, bpsqt, us))
        ctx.save_for_backward(us)
        return _launch_stack_output(lin, skip, wpsqt, bpsqt, us, den, mult, fq)

    @staticmethod
    def backward(ctx, g):
        (us,) = ctx.saved_tensors
        g = g.contiguous()
        gw, gb = _launch_stack_output_bwd(g, us)
        return g, g, gw, gb, None, None, None, None


@torch.compiler.disable(recursive=False)
def _launch_sf_loss(scorenet, score, outcome, p, actual_lambda):
    lib = _native.load()
    B = scorenet.shape[0]
    terms = torch.empty(3, B, dtype=torch.float32, device=scorenet.device)
    sums = torch.empty(2, dtype=torch.float32, device=scorenet.device)
    loss = torch.empty((), dtype=torch.float32, device=scorenet.device)
    with torch.cuda.device(scorenet.device):
        rc = lib.nnueft_sf_loss_fwd(scorenet.data_ptr(), score.data_ptr(), outcome.data_ptr(), terms.data_ptr(),
                                    sums.data_ptr(), loss.data_ptr(), B, p.in_offset, p.in_scaling, p.out_offset,
                                    p.out_scaling, p.pow_exp, p.qp_asymmetry, p.w1, p.w2, p.tb_remap_base,
                                    p.tb_remap_scale, p.tb_remap_decay, float(actual_lambda),
                                    _stream_ptr(scorenet.device))
    _native.check(rc, "nnueft_sf_loss_fwd")
    return terms, sums, loss


@torch.compiler.disable(recursive=False)
def _launch_sf_loss_bwd(terms, sums, grad_loss, shape):
    lib = _native.load()
    B = terms.shape[1]
    g = torch.empty(shape, dtype=torch.float32, device=terms.device)
    with torch.cuda.device(terms.device):
        rc = lib.nnueft_sf_loss_bwd(terms.data_ptr(), sums.data_ptr(), grad_loss.data_ptr(), g.data_ptr(), B,
                                    _stream_ptr(terms.device))
    _native.check(rc, "nnueft_sf_loss_bwd")
    return g


class _SfLoss(torch.autograd.Function):
    """sf_loss as two launches forward (per-position terms, fixed-order sums) and one backward."""

    @staticmethod
    def forward(ctx, scorenet, score, outcome, p, actual_lambda):
        scorenet = scorenet.contiguous()
        terms, sums, loss = _launch_sf_loss(scorenet, score.contiguous(), outcome.contiguous(), p, actual_lambda)
        ctx.save_for_backward(terms, sums)
        ctx.shape = scorenet.shape
        return loss

    @staticmethod
    def backward(ctx, grad_loss):
        terms, sums = ctx.saved_tensors
        grad_loss = grad_loss.contiguous().to(torch.float32)
        return _launch_sf_loss_bwd(terms, sums, grad_loss, ctx.shape), None, None, None, None


class ComposedFeatureTransformer(nn.Module):
    def __init__(self, feature_classes, l1_size: int, num_psqt_buckets: int, quantization: QuantizationManager):
        super().__init__()
        if l1_size % 2 != 0:
            raise ValueError(f"l1_size must be even, got {l1_size}.")
        self.l1_size = l1_size
        self.num_psqt_buckets = num_psqt_buckets
        self.num_outputs = l1_size + num_psqt_buckets
        self.features = nn.ModuleList([cls(self.num_outputs) for cls in feature_classes])
        self.bias = nn.Parameter(torch.empty(self.num_outputs))
        # moves with the module, stays out of the state dict (checkpoints are the reference's)
        self.register_buffer("psqt_bias_zeros", torch.zeros(num_psqt_buckets), persistent=False)
        self.NUM_INPUTS = sum(f.NUM_INPUTS for f in self.features)
        self.MAX_ACTIVE_FEATURES = sum(f.MAX_ACTIVE_FEATURES for f in self.features)
        self.NUM_REAL_FEATURES = sum(f.NUM_REAL_FEATURES for f in self.features)
        self.FEATURE_NAME = "+".join(f.FEATURE_NAME for f in self.features)
        self.INPUT_FEATURE_NAME = "+".join(f.INPUT_FEATURE_NAME for f in self.features)
        h = 0
        for f in self.features:
            h = (((h << 1) | (h >> 31)) & 0xFFFFFFFF) ^ f.HASH
        self.HASH = h
        self.quantization = quantization
        sigma = math.sqrt(1 / self.NUM_INPUTS)
        with torch.no_grad():
            self.bias.uniform_(-sigma, sigma)

    def merged_weight_and_bias(self, fake_quantize_weights: bool = False):
        q = self.quantization
        only = self.features[0] if len(self.features) == 1 else None
        if only is not None and isinstance(only, HalfKav2Hm) and only.weight.is_cuda and _native.available():
            merged = _table_merge(only.weight, only.virtual_weight, self.l1_size,
                                  q.weight_scales_dict["ft_weight"], q.weight_scales_dict["ft_psqt_weight"],
                                  fake_quantize_weights)
        else:
            merged = torch.cat([f.merged_weight() for f in self.features], dim=0)
            if fake_quantize_weights:
                merged = torch.cat([q.fake_quantize_weights(merged[:, :self.l1_size], "ft_weight"),
                                    q.fake_quantize_weights(merged[:, self.l1_size:], "ft_psqt_weight")], dim=1)
        return merged, self._merged_bias(fake_quantize_weights)

    @torch.no_grad()
    def coalesce(self):
        for f in self.features:
            f.coalesce()

    @torch.no_grad()
    def zero_virtual_weights(self):
        for f in self.features:
            f.zero_virtual_weights()

    @torch.no_grad()
    def init_weights(self):
        for f in self.features:
            f.init_weights(self.num_psqt_buckets, self.quantization.nnue2score)
        self.bias[self.l1_size:] = 0.0

    @torch.no_grad()
    def get_export_weights(self):
        return torch.cat([f.get_export_weights() for f in self.features], dim=0)

    @torch.no_grad()
    def load_export_weights(self, export_weight):
        at = 0
        for f in self.features:
            f.load_export_weights(export_weight[at:at + f.NUM_REAL_FEATURES])
            at += f.NUM_REAL_FEATURES

    def clip_weights(self, quantization):
        for f in self.features:
            f.clip_weights(quantization)

    def _merged_bias(self, fake_quantize_weights: bool):
        q = self.quantization
        b = self.bias[:self.l1_size]
        if fake_quantize_weights:
            if b.is_cuda and b.dtype == torch.float32 and _native.available():
                # one launch instead of the five elementwise ops of fake_quantize_weights (same bits)
                s = q.weight_scales_dict["ft_bias"]
                b = _table_merge(b.view(1, -1), None, self.l1_size, s, s, True).view(-1)
            else:
                b = q.fake_quantize_weights(b, "ft_bias")
        # the PSQT part of the bias is held at zero
        return torch.cat([b, self.psqt_bias_zeros.to(b.dtype)], dim=0)

    def forward(self, us, them, white_indices, black_indices, psqt_indices, fake_quantize_acts: bool,
                fake_quantize_weights: bool, backend: str = "auto"):
        q = self.quantization
        only = self.features[0] if len(self.features) == 1 else None
        if (only is not None and isinstance(only, HalfKav2Hm) and backend in ("auto", "fused")
                and all(t.is_cuda for t in (us, them, white_indices, black_indices, psqt_indices, self.bias))
                and white_indices.dtype == torch.int32 and white_indices.dim() == 2
                and _virtual_forward_fits(white_indices, only.weight, only.virtual_weight, self.l1_size)):
            # real + virtual weights (and their grid) merged inside the forward kernel: no pass over the table
            act_grid = (q.hidden_quantized_one, FAKE_QUANTIZE_EPS, q.l0_correction_factor) if fake_quantize_acts else None
            l0_, wpsqt, bpsqt = _FusedDoubleFtVirtual.apply(
                us, them, white_indices, black_indices, psqt_indices, only.weight, only.virtual_weight,
                self._merged_bias(fake_quantize_weights), q.max_ft_activation, self.l1_size,
                q.weight_scales_dict["ft_weight"], q.weight_scales_dict["ft_psqt_weight"], fake_quantize_weights,
                act_grid)
            if not fake_quantize_acts and q.l0_correction_factor != 1.0:
                l0_ = l0_ * q.l0_correction_factor
            return l0_, wpsqt, bpsqt
        merged, bias = self.merged_weight_and_bias(fake_quantize_weights)
        if (fake_quantize_acts and backend in ("auto", "fused") and merged.is_cuda and _native.available()
                and all(t.is_cuda for t in (us, them, white_indices, black_indices, psqt_indices, bias))):
            # the activation grid and the correction factor inside the kernel that writes l0
            return FusedDoubleFtFunction.apply(
                us, them, white_indices, black_indices, psqt_indices, merged, bias, q.max_ft_activation,
                self.l1_size, (q.hidden_quantized_one, FAKE_QUANTIZE_EPS, q.l0_correction_factor))
        l0_, wpsqt, bpsqt = double_feature_transform(us, them, white_indices, black_indices, psqt_indices, merged,
                                                     bias, self.quantization.max_ft_activation, self.l1_size, backend)
        if fake_quantize_acts and l0_.is_cuda and l0_.dtype == torch.float32 and _native.available():
            # activation grid and correction factor in one pass over [B, L1]
            return _ActFakeQuantize.apply(l0_, q.hidden_quantized_one, q.l0_correction_factor), wpsqt, bpsqt
        if fake_quantize_acts:
            l0_ = q.fake_quantize_ft_act(l0_)
        if q.l0_correction_factor != 1.0:     # x * 1.0 is x, and so is its gradient
            l0_ = l0_ * q.l0_correction_factor
        return l0_, wpsqt, bpsqt


# ------------------------------------------------------------------------------------------ layer stacks

@torch.compiler.disable(recursive=False)
def bucket_grouping(bucket, count):
    """The positions of a batch grouped by bucket, as the bucketed linear kernels read them: an opaque
    byte tensor to hand to every StackedLinear of the stack (they share `bucket`)."""
    lib = _native.load()
    bucket = bucket.flatten().contiguous()
    B = bucket.shape[0]
    nbytes = lib.nnueft_bucket_linear_workspace_bytes(B, count)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=bucket.device)
    with torch.cuda.device(bucket.device):
        rc = lib.nnueft_bucket_linear_group(bucket.data_ptr(), B, count, ws.data_ptr(), nbytes,
                                            _stream_ptr(bucket.device))
    _native.check(rc, "nnueft_bucket_linear_group")
    return ws


@torch.compiler.disable(recursive=False)
def _launch_bucket_linear_fwd(x, bucket, weight, bias, out_features, count, ws):
    lib = _native.load()
    B, n_in = x.shape
    y = torch.empty(B, out_features, dtype=torch.float32, device=x.device)
    with torch.cuda.device(x.device):
        rc = lib.nnueft_bucket_linear_fwd(x.data_ptr(), bucket.data_ptr(), weight.data_ptr(), bias.data_ptr(),
                                          y.data_ptr(), B, n_in, out_features, count, ws.data_ptr(), ws.numel(), 1,
                                          _stream_ptr(x.device))
    _native.check(rc, "nnueft_bucket_linear_fwd")
    return y


@torch.compiler.disable(recursive=False)
def _launch_bucket_linear_bwd(x, bucket, weight, gy, out_features, count, need_gx, ws):
    lib = _native.load()
    B, n_in = x.shape
    gx = torch.empty_like(x) if need_gx else None
    gw = torch.empty_like(weight)
    gb = torch.empty(count * out_features, dtype=torch.float32, device=x.device)
    with torch.cuda.device(x.device):
        # ws still holds the grouping of the positions the forward call made (a few bytes per position)
        rc = lib.nnueft_bucket_linear_bwd(x.data_ptr(), bucket.data_ptr(), weight.data_ptr(), gy.data_ptr(),
                                          gx.data_ptr() if need_gx else None, gw.data_ptr(), gb.data_ptr(), B, n_in,
                                          out_features, count, ws.data_ptr(), ws.numel(), 1, _stream_ptr(x.device))
    _native.check(rc, "nnueft_bucket_linear_bwd")
    return gx, gw, gb


class _BucketLinear(torch.autograd.Function):
    """y[b] = bias[bucket[b]] + weight[bucket[b]] x[b]: every position meets the block of its own
    bucket only (the wide layer followed by a selection computes the other blocks to drop them)."""

    @staticmethod
    def forward(ctx, x, bucket, weight, bias, out_features, count, grouping):
        x, weight, bias = x.contiguous(), weight.contiguous(), bias.contiguous()
        bucket = bucket.flatten().contiguous()
        ws = grouping if grouping is not None else bucket_grouping(bucket, count)
        ctx.save_for_backward(x, bucket, weight, ws)
        ctx.shape = (out_features, count)
        return _launch_bucket_linear_fwd(x, bucket, weight, bias, out_features, count, ws)

    @staticmethod
    def backward(ctx, gy):
        x, bucket, weight, ws = ctx.saved_tensors
        out_features, count = ctx.shape
        gx, gw, gb = _launch_bucket_linear_bwd(x, bucket, weight, gy.contiguous(), out_features, count,
                                               ctx.needs_input_grad[0], ws)
        return gx, None, gw, gb, None, None, None


def _bucket_linear_applies(x, in_features, out_features, count):
    # every layer of the stacks qualifies at the usual sizes (in = 3072, 64, 128)
    return (x.is_cuda and x.dtype == torch.float32 and in_features >= 32 and in_features % 32 == 0
            and out_features <= 32 and count <= 64 and _native.available())


class StackedLinear(nn.Module):
    """`count` linear layers of the same shape evaluated as one wide layer; each position picks the
    output block of its bucket."""

    def __init__(self, in_features, out_features, count, quantization=None, layer_key=None):
        super().__init__()
        self.in_features, self.out_features, self.count = in_features, out_features, count
        self.linear = nn.Linear(in_features, out_features * count)
        self.quantization, self.layer_key = quantization, layer_key
        with torch.no_grad():   # every bucket starts from the same layer
            self.linear.weight.copy_(self.linear.weight[:out_features].repeat(count, 1))
            self.linear.bias.copy_(self.linear.bias[:out_features].repeat(count))

    def _params(self):
        return self.linear.weight, self.linear.bias

    def _shared(self):
        """(weight, bias) of a layer added to every bucket's block, or (None, None)."""
        return None, None

    def _params_one_pass(self, fake_quantize_weights: bool):
        """_params() and the two fake_quantize_weights calls as one kernel per tensor (the table merge:
        q(W + V[row % rows of V]), straight-through gradient, the shared layer's gradient summed over the
        buckets); the values are those of the torch ops, bit for bit."""
        sw, sb = self._shared()
        weight, bias = self.linear.weight, self.linear.bias
        if not fake_quantize_weights and sw is None:
            return weight, bias
        q = self.quantization
        ws = q.weight_scales_dict[f"{self.layer_key}_weight"] if fake_quantize_weights else 1.0
        bs = q.weight_scales_dict[f"{self.layer_key}_bias"] if fake_quantize_weights else 1.0
        weight = _table_merge(weight, sw, weight.shape[1], ws, ws, fake_quantize_weights)
        bias = _table_merge(bias.view(-1, 1), None if sb is None else sb.view(-1, 1), 1, bs, bs,
                            fake_quantize_weights).view(-1)
        return weight, bias

    def forward(self, x, ls_indices, fake_quantize_weights: bool = False, grouping=None):
        """grouping: bucket_grouping(ls_indices, count) when several layers share ls_indices (optional)."""
        if fake_quantize_weights and (self.quantization is None or self.layer_key is None):
            raise RuntimeError("self.quantization and self.layer_key are required to use fake quantize weights.")
        w = self.linear.weight
        if w.is_cuda and w.dtype == torch.float32 and w.is_contiguous():
            weight, bias = self._params_one_pass(fake_quantize_weights)
        else:
            weight, bias = self._params()
            if fake_quantize_weights:
                weight = self.quantization.fake_quantize_weights(weight, f"{self.layer_key}_weight")
                bias = self.quantization.fake_quantize_weights(bias, f"{self.layer_key}_bias")
        if _bucket_linear_applies(x, self.in_features, self.out_features, self.count):
            return _BucketLinear.apply(x, ls_indices, weight, bias, self.out_features, self.count, grouping)
        wide = F.linear(x, weight, bias).reshape(-1, self.out_features)
        pick = ls_indices.flatten() + torch.arange(0, ls_indices.shape[0] * self.count, self.count, device=x.device)
        return wide[pick]

    @torch.no_grad()
    def at_index(self, index: int):
        layer = nn.Linear(self.in_features, self.out_features)
        weight, bias = self._params()
        lo, hi = index * self.out_features, (index + 1) * self.out_features
        layer.weight.copy_(weight[lo:hi])
        layer.bias.copy_(bias[lo:hi])
        return layer


class FactorizedStackedLinear(StackedLinear):
    """StackedLinear plus one layer shared by all buckets (added to each of them)."""

    def __init__(self, in_features, out_features, count, quantization, layer_key):
        super().__init__(in_features, out_features, count, quantization, layer_key)
        self.factorized_linear = nn.Linear(in_features, out_features)
        self.zero_virtual_weights()

    def _params(self):
        return (self.linear.weight + self.factorized_linear.weight.repeat(self.count, 1),
                self.linear.bias + self.factorized_linear.bias.repeat(self.count))

    def _shared(self):
        return self.factorized_linear.weight, self.factorized_linear.bias

    @torch.no_grad()
    def zero_virtual_weights(self):
        self.factorized_linear.weight.zero_()
        self.factorized_linear.bias.zero_()

    @torch.no_grad()
    def coalesce_weights(self):
        self.linear.weight.add_(self.factorized_linear.weight.repeat(self.count, 1))
        self.linear.bias.add_(self.factorized_linear.bias.repeat(self.count))
        self.zero_virtual_weights()


@dataclass
class ModelConfig:
    L1: int = 1024
    L2: int = 32
    L3: int = 32
    quantize_config: QuantizationConfig = field(default_factory=QuantizationConfig)


class LayerStacks(nn.Module):
    def __init__(self, count: int, config, quantization: QuantizationManager):
        super().__init__()
        self.count, self.L1, self.L2, self.L3 = count, config.L1, config.L2, config.L3
        self.quantization = quantization
        self.l1 = FactorizedStackedLinear(self.L1, self.L2, count, quantization, "ls_l1")
        self.l2 = StackedLinear(self.L2 * 2, self.L3, count, quantization, "ls_l2")
        self.output = StackedLinear(self.L2 * 2 + self.L3 * 2, 1, count, quantization, "ls_output")
        with torch.no_grad():
            self.output.linear.bias.zero_()

    def _sqr_and_linear(self, x, fake_quantize_acts):
        q = self.quantization
        sqr = torch.pow(x, 2.0)
        if fake_quantize_acts:
            sqr = q.fake_quantize_ls_act(sqr)
            x = q.fake_quantize_ls_act(x)
        return q.clip_ls_act(torch.cat([sqr * q.sqr_crelu_correction_factor, x], dim=1))

    def _sqr_crelu(self, x, fake_quantize_acts, want_skip=False):
        """_sqr_and_linear (and the skip value) as one kernel on the GPU."""
        q = self.quantization
        if _fused_tail_applies(x):
            return _SqrCrelu.apply(x, want_skip, q.hidden_quantized_one, q.sqr_crelu_correction_factor,
                                   q.max_hidden_activation, fake_quantize_acts)
        skip = x[:, -2].view(-1, 1) - x[:, -1].view(-1, 1) if want_skip else None
        return self._sqr_and_linear(x, fake_quantize_acts), skip

    def forward_parts(self, x, ls_indices, fake_quantize_acts: bool = True, fake_quantize_weights: bool = True):
        """(output layer's result, skip value), both [B, 1], before they are added and quantized."""
        # the three layers pick blocks by the same indices: group the positions once
        grouping = None
        if _bucket_linear_applies(x, self.l1.in_features, self.l1.out_features, self.count):
            grouping = bucket_grouping(ls_indices, self.count)
        l1c = self.l1(x, ls_indices, fake_quantize_weights, grouping)
        l1x, skip = self._sqr_crelu(l1c, fake_quantize_acts, want_skip=True)
        l2x, _ = self._sqr_crelu(self.l2(l1x, ls_indices, fake_quantize_weights, grouping), fake_quantize_acts)
        out = self.output(torch.cat([l1x, l2x], dim=1), ls_indices, fake_quantize_weights, grouping)
        assert out.shape[1] == 1
        return out, skip

    def forward(self, x, ls_indices, fake_quantize_acts: bool = True, fake_quantize_weights: bool = True):
        q = self.quantization
        out, skip = self.forward_parts(x, ls_indices, fake_quantize_acts, fake_quantize_weights)
        if fake_quantize_acts:
            skip = q.fake_quantize_skip_act(skip)
        out = out + skip
        if fake_quantize_acts:
            out = q.fake_quantize_output(out)
        return out

    @torch.no_grad()
    def zero_virtual_weights(self):
        self.l1.zero_virtual_weights()


# ------------------------------------------------------------------------------------------ model + loss

class NNUEModel(nn.Module):
    def __init__(self, feature_name: str, config: ModelConfig, num_psqt_buckets: int = 8, num_ls_buckets: int = 8):
        super().__init__()
        self.L1, self.L2, self.L3 = config.L1, config.L2, config.L3
        self.quantization = QuantizationManager(config.quantize_config)
        self.num_psqt_buckets, self.num_ls_buckets = num_psqt_buckets, num_ls_buckets
        self.input = ComposedFeatureTransformer(get_feature_cls(feature_name), self.L1, num_psqt_buckets,
                                                self.quantization)
        self.layer_stacks = LayerStacks(num_ls_buckets, config, self.quantization)
        self.input.init_weights()

    def calculate_buckets(self, piece_count):
        psqt_indices = (piece_count - 1) // 4
        return psqt_indices, psqt_indices

    def forward_ft(self, us, them, white_indices, black_indices, psqt_indices, fake_quantize_acts,
                   fake_quantize_weights):
        return self.input(us, them, white_indices, black_indices, psqt_indices, fake_quantize_acts,
                          fake_quantize_weights)

    # Nearly every step of this forward is a launch of libnnueft already; traced by dynamo each of them is a
    # graph break with nothing left between the breaks to fuse, and the guards cost more than they buy
    # (3.2 ms against 2.3 ms per training step at L1=3072).  torch.compile(model) therefore runs it as it is.
    @torch.compiler.disable
    def forward(self, us, them, white_indices, black_indices, piece_count, fake_quantize_acts: bool = True,
                fake_quantize_weights: bool = True):
        psqt_indices, ls_indices = self.calculate_buckets(piece_count)
        l0_, wpsqt, bpsqt = self.forward_ft(us, them, white_indices, black_indices, psqt_indices,
                                            fake_quantize_acts, fake_quantize_weights)
        # the PSQT term is the perspective average with the sign of the side to move
        if _fused_tail_applies(l0_):
            lin, skip = self.layer_stacks.forward_parts(l0_, ls_indices, fake_quantize_acts, fake_quantize_weights)
            den, mult = self.quantization.output_quantization()
            return _StackOutput.apply(lin, skip, wpsqt, bpsqt, us, den, mult, fake_quantize_acts)
        return self.layer_stacks(l0_, ls_indices, fake_quantize_acts, fake_quantize_weights) + (wpsqt - bpsqt) * (us - 0.5)

    def weight_clipping_config(self):
        """The layer-stack weights and the range the quantization scheme leaves them
        (QuantizationManager.generate_weight_clipping_config, model/quantize.py:150-172)."""
        ls, m = self.layer_stacks, self.quantization.max_hidden_weight
        return [
            {"params": [ls.l1.linear.weight], "min_weight": -m[0], "max_weight": m[0],
             "virtual_params": ls.l1.factorized_linear.weight},
            {"params": [ls.l2.linear.weight], "min_weight": -m[1], "max_weight": m[1]},
            {"params": [ls.output.linear.weight], "min_weight": -m[2], "max_weight": m[2]},
        ]

    @torch.no_grad()
    def clip_weights(self, include_input: bool):
        """Clamp the layer-stack weights to what their int8 image can hold (model/model.py:42-72; the
        reference's trainer calls it after every batch, trainer/callbacks.py:70-85).  Where a layer has
        shared (factorised) weights, the sum of the two is what gets exported, so the bounds of the real
        weights move by the shared ones."""
        if include_input:
            self.input.clip_weights(self.quantization)
        for group in self.weight_clipping_config():
            lo, hi = group["min_weight"], group["max_weight"]
            for p in group["params"]:
                if "virtual_params" in group:
                    v = group["virtual_params"]
                    spread = v.repeat(p.shape[0] // v.shape[0], p.shape[1] // v.shape[1])
                    p.data.copy_(torch.minimum(torch.maximum(p.data, lo - spread), hi - spread))
                else:
                    p.data.clamp_(lo, hi)

    @torch.no_grad()
    def zero_virtual_weights(self):
        self.input.zero_virtual_weights()
        self.layer_stacks.zero_virtual_weights()


@dataclass
class LossParams:
    in_offset: float = 270
    out_offset: float = 270
    in_scaling: float = 340
    out_scaling: float = 380
    pow_exp: float = 2.5
    qp_asymmetry: float = 0.0
    w1: float = 0.0
    w2: float = 0.5
    tb_remap_base: float = 4000.0
    tb_remap_scale: float = 4000.0
    tb_remap_decay: float = 0.85


def remap_tablebase_score(score, base: float, scale: float, decay: float):
    mate_score, max_mate_ply = 32000, 245
    magnitude = score.abs()
    plies = (mate_score - magnitude).clamp(min=0)
    remapped = base + (decay ** plies) * scale
    return torch.where(magnitude >= mate_score - max_mate_ply, torch.where(score < 0, -remapped, remapped), score)


def sf_loss(scorenet, score, outcome, p: LossParams, actual_lambda):
    """Win-rate-model loss; `scorenet` is the net output times nnue2score (model/nnue.py:39-70)."""
    # the fused kernels take one lambda for the batch, as a host number, and device pointers for the rest; a
    # per-sample lambda tensor (the reference's jittered schedule, model/lambda_utils.py:69-83) or tensors that
    # live elsewhere go through the torch formula below
    if _fused_tail_applies(scorenet) and isinstance(actual_lambda, (int, float)) \
            and score.is_cuda and outcome.is_cuda and score.device == scorenet.device == outcome.device \
            and score.dtype == torch.float32 and outcome.dtype == torch.float32 \
            and scorenet.numel() > 0 and score.shape == scorenet.shape == outcome.shape:
        return _SfLoss.apply(scorenet, score, outcome, p, float(actual_lambda))
    score = remap_tablebase_score(score, p.tb_remap_base, p.tb_remap_scale, p.tb_remap_decay)

    def win_rate(x, offset, scaling):
        return 0.5 * (1.0 + ((x - offset) / scaling).sigmoid() - ((-x - offset) / scaling).sigmoid())

    qf = win_rate(scorenet, p.in_offset, p.in_scaling)
    pf = win_rate(score, p.out_offset, p.out_scaling)
    pt = pf * actual_lambda + outcome * (1.0 - actual_lambda)
    loss = torch.pow(torch.abs(pt - qf), p.pow_exp)
    if p.qp_asymmetry != 0.0:
        loss = loss * ((qf > pt) * p.qp_asymmetry + 1)
    weights = 1 + (2.0 ** p.w1 - 1) * torch.pow((pf - 0.5) ** 2 * pf * (1 - pf), p.w2)
    return (loss * weights).sum() / weights.sum()


def optimizer_param_groups(model: "NNUEModel", lr: float = 8.75e-4, ft_weight_decay: float = 0.0,
                           dense_weight_decay: float = 0.0, factorized_weight_decay: float = 0.0):
    """The ten parameter groups the reference hands its optimizer (model/nnue.py:120-177): feature
    transformer weights / biases, then weight and bias of every layer of the stacks, biases never decayed."""
    def named(module, biases):
        return [p for n, p in module.named_parameters() if ("bias" in n) == biases and p.requires_grad]

    ls = model.layer_stacks
    groups = [
        (named(model.input, False), ft_weight_decay), (named(model.input, True), 0.0),
        ([ls.l1.factorized_linear.weight], factorized_weight_decay), ([ls.l1.factorized_linear.bias], 0.0),
        ([ls.l1.linear.weight], dense_weight_decay), ([ls.l1.linear.bias], 0.0),
        ([ls.l2.linear.weight], dense_weight_decay), ([ls.l2.linear.bias], 0.0),
        ([ls.output.linear.weight], dense_weight_decay), ([ls.output.linear.bias], 0.0),
    ]
    return [{"params": params, "lr": lr, "weight_decay": wd} for params, wd in groups]
