"""The C-ABI library loads and exports what include/nnueft.h declares (no GPU, no compute calls)."""
import ctypes
import os
import re

import pytest

from nnueft import _native

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "nnueft.h")


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(nnueft_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_expected_entry_points():
    syms = declared_symbols()
    for name in ("nnueft_sparse_fwd", "nnueft_sparse_bwd_atomic", "nnueft_sparse_bwd_det", "nnueft_double_fwd",
                 "nnueft_double_bwd_atomic", "nnueft_double_bwd_det", "nnueft_det_workspace_bytes",
                 "nnueft_ft_int16_fwd", "nnueft_version", "nnueft_error_string", "nnueft_bias_tile"):
        assert name in syms


def test_library_exports_every_declared_symbol():
    assert os.path.exists(_native.LIB_PATH), "libnnueft.so is not built (python -c 'import __graft_entry__ as g; g.build()')"
    lib = ctypes.CDLL(_native.LIB_PATH)
    for name in declared_symbols():
        assert hasattr(lib, name), f"{name} is declared in nnueft.h but not exported"


def test_binding_covers_every_declared_symbol():
    assert sorted(_native.PROTOTYPES) == declared_symbols()
    assert _native.available()


def test_host_only_entry_points():
    lib = _native.load()
    assert lib.nnueft_version() == 2
    assert lib.nnueft_bias_tile() == 32
    # the constants of the deterministic order are the oracle's
    from oracle import cpu as oracle_cpu

    assert lib.nnueft_bias_tile() == oracle_cpu.bias_tile()
    assert lib.nnueft_row_split() == oracle_cpu.row_split()
    for B in (1, 127, 2048, 2049, 5000, 16384, 16385, 65536, 1000003):
        assert lib.nnueft_row_window(B) == oracle_cpu.row_window(B)
    assert lib.nnueft_row_window(0) == 0
    assert lib.nnueft_error_string(0) == b"success"
    for code in (-1, -2, -3, -4):
        assert lib.nnueft_error_string(code).startswith(b"nnueft:")
    # workspace size: monotone, 256-byte granular, zero for nonsense
    a = lib.nnueft_det_workspace_bytes(16384, 32, 24576, 3080, 2, 512)
    b = lib.nnueft_det_workspace_bytes(16384, 32, 24576, 3080, 1, 512)
    strict = lib.nnueft_det_workspace_bytes(16384, 32, 24576, 3080, 2, 0)
    assert a > b > 0 and a % 256 == 0 and b % 256 == 0
    assert a > strict >= 2 * 16384 * 3080 * 4   # holds the two upstream rows of every position; no window sums
    # window sums are kept for 384 split rows at most, however many rows a lower threshold could split
    assert lib.nnueft_det_workspace_bytes(16384, 32, 24576, 3080, 2, 256) == a
    assert lib.nnueft_det_workspace_bytes(16384, 32, 24576, 3080, 2, 1) == a
    assert a - strict <= 384 * 2 * 16 * 3080 * 4 + 4096 and a <= 600 * 1000 * 1000
    # a small batch cannot split that many rows: 2 * 64 * 32 slots over a threshold of 512 make 7 rows at most
    # (against a threshold that no row can reach: no window sums at all)
    small = lib.nnueft_det_workspace_bytes(64, 32, 24576, 3080, 2, 512) - lib.nnueft_det_workspace_bytes(64, 32, 24576, 3080, 2, 2 * 64 * 32)
    assert 0 < small <= 7 * 2 * 1 * 3080 * 4 + 4096
    # the strict order keeps the tables of its reduction out of LDS tiles beside the sorted lists: a chunk table, and
    # per chunk of 624 pairs its inverted lists (65 KB at most) and the facts of its chains
    tables = strict - lib.nnueft_det_workspace_bytes(16384, 32, 24576, 3080, 2, 2 * 16384 * 32)
    assert 0 < tables <= 13 * 1000 * 1000
    assert lib.nnueft_det_workspace_bytes(0, 32, 10, 8, 1, 512) == 0
    assert lib.nnueft_det_workspace_bytes(4, 32, 10, 8, 3, 512) == 0
    assert lib.nnueft_det_workspace_bytes(4, 32, 10, 8, 1, -1) == 0


def test_check_raises_with_the_library_message():
    with pytest.raises(RuntimeError, match="invalid argument"):
        _native.check(-1, "unit test")
    _native.check(0, "unit test")
