"""Writes tests/golden/halfka_fens.json: FEN strings and the index lists the REFERENCE's C++ encoder
(oracle/_ref, built from the reference sources by oracle/Makefile) produces for them.

Run here, where the reference checkout exists:  python tests/golden/make_halfka_golden.py
The fixture is data (inputs and expected outputs); the GPU box only reads the JSON.
"""
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "nnue-pytorch_amd"))

from nnueft import halfka_v2_hm as hk  # noqa: E402
from oracle import loader_ref  # noqa: E402

HAND_WRITTEN = [
    "rnbqkbnr/pppppppp/8/8/8/8/PPPPPPPP/RNBQKBNR w KQkq - 0 1",
    "r1bq1rk1/pp2ppbp/2np1np1/8/3NP3/2N1BP2/PPPQ2PP/R3KB1R w KQ - 3 9",
    "8/8/4k3/8/8/3K4/8/8 w - - 0 1",
    "8/5k2/8/8/8/8/2K5/8 b - - 0 1",
    "k7/8/8/8/8/8/8/K7 w - - 0 1",
    "7k/8/8/8/8/8/8/7K b - - 0 1",
    "4k3/8/8/8/8/8/8/R3K2R w KQ - 0 1",
    "2r3k1/5ppp/p3p3/1p6/3P4/P3PQ2/1q3PPP/5RK1 b - - 0 25",
]


def playable(squares, types, colors):
    """Keep positions the reference's FEN parser and move generator are happy with: no pawns on the
    first or last rank, kings not adjacent."""
    sq = {int(s): (int(t), int(c)) for s, t, c in zip(squares, types, colors) if s >= 0}
    kings = [s for s, (t, _) in sq.items() if t == hk.KING]
    (a, b) = kings
    if max(abs(a % 8 - b % 8), abs(a // 8 - b // 8)) <= 1:
        return False
    return all(not (t == hk.PAWN and (s // 8 in (0, 7))) for s, (t, _) in sq.items())


def main():
    fens = list(HAND_WRITTEN)
    squares, types, colors = hk.random_positions(400, seed=2024)
    rng = np.random.default_rng(5)
    for i in range(squares.shape[0]):
        if playable(squares[i], types[i], colors[i]):
            fens.append(hk.to_fen(squares[i], types[i], colors[i], white_to_move=bool(rng.integers(0, 2))))
        if len(fens) >= 72:
            break
    enc = loader_ref.encode_fens(fens, "HalfKAv2_hm")
    doc = {
        "source": "reference C++ encoder, get_sparse_batch_from_fens('HalfKAv2_hm') "
                  "(data_loader/cpp/training_data_loader_abi.cpp:12-33, training_data_loader.cpp:20-73,487-544)",
        "num_inputs": enc["num_inputs"],
        "max_active": enc["max_active"],
        "fens": fens,
        "is_white": enc["is_white"].astype(int).tolist(),
        "white": enc["white"].tolist(),
        "black": enc["black"].tolist(),
        "piece_count": enc["piece_count"].tolist(),
    }
    with open(os.path.join(HERE, "halfka_fens.json"), "w") as f:
        json.dump(doc, f, separators=(",", ":"))
    print(f"wrote {len(fens)} positions, num_inputs={enc['num_inputs']}")


if __name__ == "__main__":
    main()
