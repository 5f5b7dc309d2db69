"""ctypes front end of oracle/_ref/libtraining_data_loader_ref.so: the reference's own C++ batch encoder
(data_loader/cpp/training_data_loader.cpp), compiled from the reference sources by oracle/Makefile.

TEST INFRASTRUCTURE.  Used to check nnueft.halfka_v2_hm against the real encoder on FEN strings.
The struct layout is the one data_loader/_native.py:33-46 declares.
"""
import ctypes
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "_ref", "libtraining_data_loader_ref.so")


class _SparseBatch(ctypes.Structure):
    _fields_ = [
        ("num_inputs", ctypes.c_int),
        ("size", ctypes.c_int),
        ("is_white", ctypes.POINTER(ctypes.c_float)),
        ("outcome", ctypes.POINTER(ctypes.c_float)),
        ("score", ctypes.POINTER(ctypes.c_float)),
        ("num_active_white_features", ctypes.c_int),
        ("num_active_black_features", ctypes.c_int),
        ("max_active_features", ctypes.c_int),
        ("white", ctypes.POINTER(ctypes.c_int)),
        ("black", ctypes.POINTER(ctypes.c_int)),
        ("piece_count", ctypes.POINTER(ctypes.c_int)),
    ]


def available() -> bool:
    return os.path.exists(LIB_PATH)


def encode_fens(fens, feature_set="HalfKAv2_hm"):
    """-> dict(num_inputs, max_active, is_white f32[B], white int32[B,K], black int32[B,K], piece_count int32[B])."""
    lib = ctypes.CDLL(LIB_PATH)
    lib.get_sparse_batch_from_fens.restype = ctypes.POINTER(_SparseBatch)
    lib.get_sparse_batch_from_fens.argtypes = [
        ctypes.c_char_p, ctypes.c_int, ctypes.POINTER(ctypes.c_char_p),
        ctypes.POINTER(ctypes.c_int), ctypes.POINTER(ctypes.c_int), ctypes.POINTER(ctypes.c_int),
    ]
    lib.destroy_sparse_batch.argtypes = [ctypes.POINTER(_SparseBatch)]
    n = len(fens)
    arr = (ctypes.c_char_p * n)(*[f.encode() for f in fens])
    zeros = (ctypes.c_int * n)(*([0] * n))
    ptr = lib.get_sparse_batch_from_fens(feature_set.encode(), n, arr, zeros, zeros, zeros)
    if not ptr:
        raise RuntimeError(f"the reference loader does not know feature set {feature_set}")
    sb = ptr.contents
    K = sb.max_active_features
    out = dict(
        num_inputs=int(sb.num_inputs), max_active=int(K),
        is_white=np.ctypeslib.as_array(sb.is_white, shape=(n,)).copy(),
        white=np.ctypeslib.as_array(sb.white, shape=(n, K)).copy(),
        black=np.ctypeslib.as_array(sb.black, shape=(n, K)).copy(),
        piece_count=np.ctypeslib.as_array(sb.piece_count, shape=(n,)).copy(),
    )
    lib.destroy_sparse_batch(ptr)
    return out
