"""Loader hand-off on the GPU: one staged copy and one kernel give the tensors the CPU path gives; the
pinned ring is reused correctly; the prefetcher feeds the feature transformer from its own stream."""
import numpy as np
import pytest
import torch

import nnueft
from nnueft.batch_handoff import DevicePrefetcher, _ring
from nnueft.double_ft_functions import double_feature_transform
from test_handoff_cpu import check, make_batch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.mark.parametrize("B", [1, 7, 1000, 16384])
def test_get_tensors_gpu(B):
    sb, want = make_batch(B, 20 + B)
    out = sb.get_tensors(DEV, use_pinned_memory=True)
    torch.cuda.synchronize()
    assert all(t.is_cuda for t in out)
    assert out[2].data_ptr() % 256 == 0 and out[3].data_ptr() % 128 == 0      # the index lists stay aligned
    check(out, want, B)
    cpu = sb.get_tensors("cpu")
    for a, b in zip(out, cpu):
        assert torch.equal(a.cpu(), b)


def test_staging_ring_is_reused_without_mixing_batches():
    made = [make_batch(200 + 37 * (i % 5), 500 + i) for i in range(25)]
    outs = [sb.get_tensors(DEV) for sb, _ in made]       # all copies enqueued before any is checked
    ring = _ring(torch.device(DEV))
    assert sum(b is not None for b in ring._bufs) == ring.depth
    torch.cuda.synchronize()
    for out, (sb, want) in zip(outs, made):
        check(out, want, sb.size)


def test_prefetcher_feeds_the_feature_transformer():
    L1, R = 64, 24576
    g = torch.Generator().manual_seed(3)
    W = (torch.randn(R, L1 + 8, generator=g) * 0.05).to(DEV)
    bias = torch.randn(L1 + 8, generator=g).to(DEV)
    made = [make_batch(300 + i, 700 + i) for i in range(12)]
    pf = DevicePrefetcher((sb for sb, _ in made), DEV, depth=3)
    n = 0
    for out, (sb, want) in zip(pf, made):
        us, them, white, black, outcome, score, piece_count = out
        psqt = (piece_count - 1) // 4
        l0, wp, bp = double_feature_transform(us, them, white, black, psqt, W, bias, 255 / 256, L1, "fused")
        t = [torch.from_numpy(want[k]).to(DEV) for k in ("us", "them", "white", "black")]
        psqt2 = torch.from_numpy(((want["pc"] - 1) // 4).astype(np.int64)).to(DEV)
        l0b, wpb, bpb = double_feature_transform(*t, psqt2, W, bias, 255 / 256, L1, "fused")
        assert torch.equal(l0, l0b) and torch.equal(wp, wpb) and torch.equal(bp, bpb)
        check(out, want, sb.size)
        n += 1
    assert n == 12
    pf.close()
