"""nnueft_double_fwd_noalloc (the entry point that allocates nothing: its scratch memory is a fixed array
inside the library) against nnueft_double_fwd on the same inputs, through the C ABI: bit-equal outputs on
two calls in a row, the second with a smaller input, so what the first call left in the shared scratch
array must not leak into the second."""
import numpy as np
import pytest
import torch

from nnueft import _native
from nnueft import halfka_v2_hm as hk

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _inputs(B, L1, seed):
    us, them, white, black, pc = hk.synthetic_batch(B, seed, game_like=bool(seed & 1))
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(DEV)
    g = torch.Generator().manual_seed(seed)
    W = (torch.randn(hk.NUM_INPUTS, L1 + 8, generator=g) * 0.02).to(DEV)
    bias = (torch.randn(L1 + 8, generator=g) * 0.02).to(DEV)
    return [t(us), t(them), t(white), t(black), t((pc - 1) // 4), W, bias]


def _outputs(B, L1):
    return [torch.full(s, float("nan"), device=DEV) for s in ((B, L1), (B,), (B,), (2, B, L1))]


def test_noalloc_forward_equals_the_workspace_forward_on_two_calls_in_a_row():
    lib = _native.load()
    st = torch.cuda.current_stream().cuda_stream
    K, R, n_psqt = 32, hk.NUM_INPUTS, 8
    # everything is allocated before the first call; the calls themselves must not need the allocator
    cases = [(6000, 1024, 71), (1500, 1024, 72)]
    prepared = []
    for B, L1, seed in cases:
        nbytes = lib.nnueft_fwd_workspace_bytes(B, K, R, L1, n_psqt)
        assert 0 < nbytes <= 2 << 20
        prepared.append((B, L1, _inputs(B, L1, seed), _outputs(B, L1), _outputs(B, L1),
                         torch.empty(nbytes, dtype=torch.uint8, device=DEV), nbytes))
    torch.cuda.synchronize()
    for B, L1, inp, got, want, ws, nbytes in prepared:
        head = [x.data_ptr() for x in inp] + [255.0 / 256.0]
        before = torch.cuda.memory_allocated()
        _native.check(lib.nnueft_double_fwd_noalloc(*head, *[x.data_ptr() for x in got], B, K, R, L1, n_psqt, st),
                      "nnueft_double_fwd_noalloc")
        assert torch.cuda.memory_allocated() == before
        _native.check(lib.nnueft_double_fwd(*head, *[x.data_ptr() for x in want], B, K, R, L1, n_psqt, ws.data_ptr(),
                                            nbytes, st), "nnueft_double_fwd")
        torch.cuda.synchronize()
        for a, b in zip(got, want):
            assert not torch.isnan(a).any()
            assert torch.equal(a, b)


def test_noalloc_forward_rejects_sizes_beyond_its_scratch():
    lib = _native.load()
    x = torch.zeros(64, device=DEV)
    p = x.data_ptr()
    st = torch.cuda.current_stream().cuda_stream
    B = 1 << 19
    assert lib.nnueft_fwd_workspace_bytes(B, 32, hk.NUM_INPUTS, 1024, 8) > 2 << 20
    rc = lib.nnueft_double_fwd_noalloc(p, p, p, p, p, p, p, 1.0, p, p, p, p, B, 32, hk.NUM_INPUTS, 1024, 8, st)
    assert rc == -4
    assert b"scratch" in lib.nnueft_error_string(rc)
