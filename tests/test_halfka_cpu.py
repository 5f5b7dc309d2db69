"""HalfKAv2_hm index scheme: golden vectors from the reference's C++ encoder, hand-derived known
answers, structural properties, and (where oracle/_ref is built) the live reference encoder."""
import json
import os

import numpy as np
import pytest

from nnueft import halfka_v2_hm as hk
from oracle import loader_ref

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "halfka_fens.json")
LETTER = {"p": hk.PAWN, "n": hk.KNIGHT, "b": hk.BISHOP, "r": hk.ROOK, "q": hk.QUEEN, "k": hk.KING}


def parse_fen(fen):
    board = fen.split()[0]
    squares, types, colors = [], [], []
    for rank_from_top, row in enumerate(board.split("/")):
        file = 0
        for ch in row:
            if ch.isdigit():
                file += int(ch)
            else:
                squares.append((7 - rank_from_top) * 8 + file)
                types.append(LETTER[ch.lower()])
                colors.append(hk.WHITE if ch.isupper() else hk.BLACK)
                file += 1
    pad = 32 - len(squares)
    return squares + [-1] * pad, types + [-1] * pad, colors + [-1] * pad


def encode_fens(fens, fold_kings=False):
    sq, ty, co = zip(*[parse_fen(f) for f in fens])
    return hk.encode_batch(np.array(sq), np.array(ty), np.array(co), fold_kings=fold_kings)


def test_golden_vectors_from_the_reference_encoder():
    doc = json.load(open(GOLDEN))
    assert doc["num_inputs"] == hk.NUM_INPUTS == 24576 and doc["max_active"] == hk.MAX_ACTIVE_FEATURES == 32
    white, black, pc = encode_fens(doc["fens"])
    assert np.array_equal(white, np.array(doc["white"], np.int32))
    assert np.array_equal(black, np.array(doc["black"], np.int32))
    assert np.array_equal(pc, np.array(doc["piece_count"], np.int32))
    assert len(doc["fens"]) >= 64


@pytest.mark.skipif(not loader_ref.available(), reason="oracle/_ref not built (needs the reference checkout)")
def test_live_reference_encoder_on_fresh_positions():
    squares, types, colors = hk.random_positions(600, seed=77)
    keep = []
    for i in range(600):
        sq = {int(s): int(t) for s, t in zip(squares[i], types[i]) if s >= 0}
        kings = [s for s, t in sq.items() if t == hk.KING]
        far = max(abs(kings[0] % 8 - kings[1] % 8), abs(kings[0] // 8 - kings[1] // 8)) > 1
        if far and all(not (t == hk.PAWN and s // 8 in (0, 7)) for s, t in sq.items()):
            keep.append(i)
    keep = keep[:200]
    fens = [hk.to_fen(squares[i], types[i], colors[i], white_to_move=bool(i & 1)) for i in keep]
    ref = loader_ref.encode_fens(fens)
    white, black, pc = hk.encode_batch(squares[keep], types[keep], colors[keep])
    assert np.array_equal(white, ref["white"]) and np.array_equal(black, ref["black"])
    assert np.array_equal(pc, ref["piece_count"])
    assert ref["is_white"].tolist() == [float(i & 1) for i in keep]


def test_known_answers_by_hand():
    # largest index: bucket 31, opposing king (p_idx 11), oriented square 63
    assert 63 + 64 * 11 + 768 * 31 == hk.NUM_INPUTS - 1 == 24575
    # white king e1 (sq 4), white point of view: file e is not < e, no mirror; bucket KingBuckets[4] = 31;
    # own king: p_idx = 2*5 + 0 = 10
    assert hk.feature_index(hk.WHITE, 4, 4, hk.KING, hk.WHITE) == 4 + 64 * 10 + 768 * 31
    # white king a1 (sq 0): mirrored to h1 (sq 7), bucket KingBuckets[7] = 28; a white pawn on a2 (sq 8) -> h2 (sq 15)
    assert hk.feature_index(hk.WHITE, 0, 0, hk.KING, hk.WHITE) == 7 + 64 * 10 + 768 * 28
    assert hk.feature_index(hk.WHITE, 0, 8, hk.PAWN, hk.WHITE) == 15 + 64 * 0 + 768 * 28
    # black point of view, black king e8 (sq 60): vertical flip -> e1, bucket 31; a white queen on d1 (sq 3)
    # is an opposing queen (p_idx 9) on d8 (sq 59) after the flip
    assert hk.feature_index(hk.BLACK, 60, 3, hk.QUEEN, hk.WHITE) == 59 + 64 * 9 + 768 * 31
    # black king h8 (sq 63): flip -> h1 (sq 7): file h, no mirror, bucket 28
    assert hk.feature_index(hk.BLACK, 63, 63, hk.KING, hk.BLACK) == 7 + 64 * 10 + 768 * 28
    # exported numbering: both kings in block 10, 704 rows per bucket
    assert hk.feature_index(hk.WHITE, 4, 60, hk.KING, hk.BLACK, fold_kings=True) == 60 + 64 * 10 + 704 * 31
    assert 63 + 64 * 10 + 704 * 31 == hk.NUM_INPUTS_EXPORT - 1 == 22527
    assert sorted(set(hk.KING_BUCKETS.tolist()) - {-1}) == list(range(32))


def test_batch_encoder_agrees_with_scalar_formula():
    squares, types, colors = hk.random_positions(64, seed=3)
    for fold in (False, True):
        white, black, pc = hk.encode_batch(squares, types, colors, fold_kings=fold)
        for i in range(64):
            pieces = sorted((int(s), int(t), int(c)) for s, t, c in zip(squares[i], types[i], colors[i]) if s >= 0)
            wk = next(s for s, t, c in pieces if t == hk.KING and c == hk.WHITE)
            bk = next(s for s, t, c in pieces if t == hk.KING and c == hk.BLACK)
            want_w = [hk.feature_index(hk.WHITE, wk, s, t, c, fold) for s, t, c in pieces]
            want_b = [hk.feature_index(hk.BLACK, bk, s, t, c, fold) for s, t, c in pieces]
            n = len(pieces)
            assert white[i, :n].tolist() == want_w and black[i, :n].tolist() == want_b
            assert (white[i, n:] == -1).all() and (black[i, n:] == -1).all()
            assert pc[i] == n


def test_structural_properties():
    B = 2000
    squares, types, colors = hk.random_positions(B, seed=11)
    white, black, pc = hk.encode_batch(squares, types, colors)
    n = (squares >= 0).sum(1)
    assert (pc == n).all() and n.min() >= 4 and n.max() <= 32
    assert ((white >= 0).sum(1) == n).all() and ((black >= 0).sum(1) == n).all()
    assert white.max() < hk.NUM_INPUTS and black.max() < hk.NUM_INPUTS
    for lists in (white, black):
        for i in range(0, B, 97):
            v = lists[i][lists[i] >= 0]
            assert len(set(v.tolist())) == len(v)                 # distinct inside a list
            assert len(set((v // 768).tolist())) == 1             # one king bucket per list
    # colour swap + vertical flip of the board swaps the two lists (as sets: the order follows squares)
    fs = np.where(squares >= 0, squares ^ 56, -1)
    fc = np.where(colors >= 0, 1 - colors, -1)
    w2, b2, _ = hk.encode_batch(fs, types, fc)
    assert np.array_equal(np.sort(w2, axis=1), np.sort(black, axis=1))
    assert np.array_equal(np.sort(b2, axis=1), np.sort(white, axis=1))
    # the exported numbering stays below 22528
    wf, bf, _ = hk.encode_batch(squares, types, colors, fold_kings=True)
    assert wf.max() < hk.NUM_INPUTS_EXPORT and bf.max() < hk.NUM_INPUTS_EXPORT


def test_synthetic_batch_tuple():
    us, them, white, black, pc = hk.synthetic_batch(512, seed=5)
    assert us.shape == (512, 1) and us.dtype == np.float32 and set(np.unique(us)) <= {0.0, 1.0}
    assert np.array_equal(them, 1.0 - us)
    assert white.shape == black.shape == (512, 32) and white.dtype == np.int32
    assert pc.dtype == np.int64 and pc.min() >= 4 and pc.max() <= 32
    again = hk.synthetic_batch(512, seed=5)
    assert all(np.array_equal(a, b) for a, b in zip((us, them, white, black, pc), again))
    assert 16.0 < pc.mean() < 20.0     # 2 kings + U{2..30}: mean 18


def test_game_like_positions_are_well_formed_and_concentrated():
    B = 8192
    squares, types, colors = hk.game_like_positions(B, seed=9)
    again = hk.game_like_positions(B, seed=9)
    assert all(np.array_equal(a, b) for a, b in zip((squares, types, colors), again))
    used = squares >= 0
    assert ((types >= 0) == used).all() and ((colors >= 0) == used).all()
    for i in range(0, B, 97):
        sq = squares[i][used[i]]
        assert len(set(sq.tolist())) == len(sq)                 # one piece per square
    assert ((types == hk.KING) & (colors == hk.WHITE)).sum(1).tolist() == [1] * B
    assert ((types == hk.KING) & (colors == hk.BLACK)).sum(1).tolist() == [1] * B
    white, black, pc = hk.encode_batch(squares, types, colors)
    assert pc.min() >= 2 and pc.max() <= 32 and 14.0 < pc.mean() < 20.0
    # what makes these positions a different workload from the uniform ones: one king bucket holds
    # more than a fifth of the batch, and the rows named by more than 512 slots hold a third of all slots
    bucket = np.bincount(white[:, 0] // hk.NUM_PLANES, minlength=hk.NUM_BUCKETS)
    assert bucket.max() > 0.2 * B
    rows = np.bincount(np.concatenate([white[white >= 0], black[black >= 0]]), minlength=hk.NUM_INPUTS)
    assert rows[rows > 512].sum() > rows.sum() / 3
    us, them, w2, b2, pc2 = hk.synthetic_batch(B, seed=9, game_like=True)
    assert np.array_equal(w2, white) and np.array_equal(b2, black)


@pytest.mark.skipif(not loader_ref.available(), reason="oracle/_ref not built (needs the reference checkout)")
def test_live_reference_encoder_on_game_like_positions():
    squares, types, colors = hk.game_like_positions(400, seed=78)
    keep = []
    for i in range(400):
        sq = {int(s): int(t) for s, t in zip(squares[i], types[i]) if s >= 0}
        kings = [s for s, t in sq.items() if t == hk.KING]
        far = max(abs(kings[0] % 8 - kings[1] % 8), abs(kings[0] // 8 - kings[1] // 8)) > 1
        if far and all(not (t == hk.PAWN and s // 8 in (0, 7)) for s, t in sq.items()):
            keep.append(i)
    assert len(keep) > 200
    fens = [hk.to_fen(squares[i], types[i], colors[i], white_to_move=bool(i & 1)) for i in keep]
    ref = loader_ref.encode_fens(fens)
    white, black, pc = hk.encode_batch(squares[keep], types[keep], colors[keep])
    assert np.array_equal(white, ref["white"]) and np.array_equal(black, ref["black"])
