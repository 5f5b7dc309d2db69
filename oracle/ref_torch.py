"""The reference's CPU path, restated with the same torch library calls.

TEST INFRASTRUCTURE: used as a checker and as the timed CPU baseline.

  sparse_linear             follows model/modules/feature_transformer/sparse_linear_functions.py:16-50
  double_feature_transform  follows model/modules/feature_transformer/double_ft_functions.py:53-80
Backward is torch autograd, as in the reference.
"""
import torch
import torch.nn.functional as F


def sparse_linear(feature_indices, weight, bias):
    batch, max_active = feature_indices.shape
    keep = feature_indices >= 0
    flat = feature_indices.clamp(min=0).long().reshape(-1)
    psw = keep.to(weight.dtype).reshape(-1)
    offsets = torch.arange(0, batch * max_active, max_active, device=feature_indices.device)
    summed = F.embedding_bag(flat, weight, offsets, mode="sum", per_sample_weights=psw)
    return summed + bias


def double_feature_transform(us, them, white_indices, black_indices, psqt_indices, weight, bias,
                             max_ft_activation, l1_size):
    assert l1_size % 2 == 0
    wp = sparse_linear(white_indices, weight, bias)
    bp = sparse_linear(black_indices, weight, bias)
    w, wpsqt = torch.split(wp, l1_size, dim=1)
    b, bpsqt = torch.split(bp, l1_size, dim=1)
    sel = psqt_indices.unsqueeze(dim=1)
    wpsqt = wpsqt.gather(1, sel)
    bpsqt = bpsqt.gather(1, sel)
    x = (us * torch.cat([w, b], dim=1)) + (them * torch.cat([b, w], dim=1))
    x = torch.clamp(x, 0.0, max_ft_activation)
    q = torch.split(x, l1_size // 2, dim=1)
    l0 = torch.cat([q[0] * q[1], q[2] * q[3]], dim=1)
    return l0, wpsqt, bpsqt
