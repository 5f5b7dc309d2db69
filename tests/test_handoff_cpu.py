"""Loader hand-off on the CPU: SparseBatch.get_tensors against the arrays the batch was made from, against
the reference's own C++ encoder where oracle/_ref holds it, and the prefetcher's queue logic."""
import ctypes
import json
import os

import numpy as np
import pytest
import torch

from nnueft import halfka_v2_hm as hk
from nnueft.batch_handoff import DevicePrefetcher, SparseBatch
from oracle import loader_ref

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "halfka_fens.json")


def make_batch(B, seed, K=32):
    rng = np.random.default_rng(seed)
    us, them, white, black, pc = hk.synthetic_batch(B, seed)
    outcome = rng.choice(np.array([0.0, 0.5, 1.0], dtype=np.float32), size=B)
    score = rng.normal(0, 300, size=B).astype(np.float32)
    sb = SparseBatch.from_arrays(hk.NUM_INPUTS, us.reshape(B), outcome, score, white, black, pc)
    return sb, dict(us=us, them=them, white=white, black=black, outcome=outcome, score=score, pc=pc)


def check(tensors, want, B, K=32):
    us, them, white, black, outcome, score, piece_count = tensors
    for t in (us, them, outcome, score):
        assert t.dtype == torch.float32 and tuple(t.shape) == (B, 1)
    assert white.dtype == torch.int32 and black.dtype == torch.int32 and tuple(white.shape) == (B, K)
    assert piece_count.dtype == torch.int64 and tuple(piece_count.shape) == (B,)
    assert np.array_equal(us.cpu().numpy(), want["us"].reshape(B, 1))
    assert np.array_equal(them.cpu().numpy(), (np.float32(1.0) - want["us"]).reshape(B, 1))
    assert np.array_equal(white.cpu().numpy(), want["white"]) and np.array_equal(black.cpu().numpy(), want["black"])
    assert np.array_equal(outcome.cpu().numpy().reshape(B), want["outcome"])
    assert np.array_equal(score.cpu().numpy().reshape(B), want["score"])
    assert np.array_equal(piece_count.cpu().numpy(), want["pc"].astype(np.int64))


@pytest.mark.parametrize("B", [1, 7, 1000])
def test_get_tensors_cpu(B):
    sb, want = make_batch(B, 10 + B)
    assert sb.size == B and sb.max_active_features == 32
    assert sb.num_active_white_features == int((want["white"] >= 0).sum())
    out = sb.get_tensors("cpu")
    check(out, want, B)
    # nothing aliases the loader's memory
    sb._keep[0][:] = -5.0
    sb._keep[1][:] = -7
    check(out, want, B)


def test_struct_layout_matches_the_reference_declaration():
    # data_loader/_native.py:33-46 on a 64-bit ABI: 2 ints, 3 pointers, 3 ints (+pad), 3 pointers
    assert [f[0] for f in SparseBatch._fields_] == [
        "num_inputs", "size", "is_white", "outcome", "score", "num_active_white_features",
        "num_active_black_features", "max_active_features", "white", "black", "piece_count"]
    assert SparseBatch.is_white.offset == 8 and SparseBatch.num_active_white_features.offset == 32
    assert SparseBatch.white.offset == 48 and ctypes.sizeof(SparseBatch) == 72


@pytest.mark.skipif(not loader_ref.available(), reason="oracle/_ref loader not built (needs the reference sources)")
def test_batch_from_the_reference_encoder():
    """A batch made by the reference's C++ (compiled under oracle/_ref) read through this struct."""
    fens = json.load(open(GOLDEN))["fens"]
    lib = ctypes.CDLL(loader_ref.LIB_PATH)
    lib.get_sparse_batch_from_fens.restype = ctypes.POINTER(SparseBatch)
    lib.get_sparse_batch_from_fens.argtypes = [ctypes.c_char_p, ctypes.c_int, ctypes.POINTER(ctypes.c_char_p),
                                               ctypes.POINTER(ctypes.c_int), ctypes.POINTER(ctypes.c_int),
                                               ctypes.POINTER(ctypes.c_int)]
    lib.destroy_sparse_batch.argtypes = [ctypes.POINTER(SparseBatch)]
    n = len(fens)
    arr = (ctypes.c_char_p * n)(*[f.encode() for f in fens])
    scores = (ctypes.c_int * n)(*range(n))
    plies = (ctypes.c_int * n)(*([0] * n))
    results = (ctypes.c_int * n)(*[(i % 3) - 1 for i in range(n)])
    ptr = lib.get_sparse_batch_from_fens(b"HalfKAv2_hm", n, arr, scores, plies, results)
    assert ptr
    us, them, white, black, outcome, score, piece_count = ptr.contents.get_tensors("cpu")
    lib.destroy_sparse_batch(ptr)
    ref = loader_ref.encode_fens(fens)
    assert np.array_equal(white.numpy(), ref["white"]) and np.array_equal(black.numpy(), ref["black"])
    assert np.array_equal(us.numpy().reshape(n), ref["is_white"])
    assert np.array_equal(piece_count.numpy(), ref["piece_count"].astype(np.int64))
    assert np.array_equal(score.numpy().reshape(n), np.arange(n, dtype=np.float32))
    assert np.array_equal(outcome.numpy().reshape(n), np.array([((i % 3) - 1 + 1) / 2 for i in range(n)], np.float32))


def test_prefetcher_on_cpu_keeps_order_and_releases():
    made = [make_batch(50 + i, 300 + i) for i in range(6)]
    released = []
    pf = DevicePrefetcher((sb for sb, _ in made), "cpu", depth=2, release=lambda b: released.append(b.size))
    got = list(pf)
    assert len(got) == 6 and released == [50 + i for i in range(6)]
    for out, (sb, want) in zip(got, made):
        check(out, want, sb.size)
    with pytest.raises(StopIteration):
        next(pf)
    pf.close()


def test_prefetcher_hands_over_worker_errors():
    def source():
        yield make_batch(5, 1)[0]
        raise OSError("file went away")

    pf = DevicePrefetcher(source(), "cpu", depth=2)
    next(pf)
    with pytest.raises(OSError, match="file went away"):
        next(pf)
    pf.close()


def test_prefetcher_accepts_tuples_of_tensors():
    items = [(torch.full((3,), float(i)), torch.arange(4) + i) for i in range(4)]
    got = list(DevicePrefetcher(iter(items), "cpu"))
    assert all(torch.equal(a[0], b[0]) and torch.equal(a[1], b[1]) for a, b in zip(got, items))
