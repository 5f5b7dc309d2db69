"""HalfKAv2_hm feature indices and seeded synthetic batches.

The index scheme is the one of the reference's batch encoder,
data_loader/cpp/training_data_loader.cpp:20-73 (== model/modules/features/halfka_v2_hm.py:8-36):
    flip  = (56 if the point of view is black) ^ (7 if that side's king is on files a-d)
    p_idx = 2 * piece_type + (piece colour != point of view),   pawn = 0 ... king = 5
    index = (sq ^ flip) + 64 * p_idx + 768 * KingBuckets[ksq ^ flip]
One index per piece (both kings included) in ascending square order, then -1 up to 32 slots
(training_data_loader.cpp:516-519).  Squares are a1 = 0, b1 = 1, ... h8 = 63.

`fold_kings=True` gives the 11-piece-type numbering of exported nets (22528 rows): own and
opposing king share block 10 and a king bucket spans 704 rows
(model/modules/features/halfka_v2_hm.py:104-135).
"""
import numpy as np

NUM_SQ = 64
NUM_PT = 12
NUM_PLANES = NUM_SQ * NUM_PT          # 768
NUM_BUCKETS = 32
NUM_INPUTS = NUM_PLANES * NUM_BUCKETS  # 24576
NUM_INPUTS_EXPORT = 704 * NUM_BUCKETS  # 22528
MAX_ACTIVE_FEATURES = 32

PAWN, KNIGHT, BISHOP, ROOK, QUEEN, KING = range(6)
WHITE, BLACK = 0, 1

# fmt: off
KING_BUCKETS = np.array([
    -1, -1, -1, -1, 31, 30, 29, 28,
    -1, -1, -1, -1, 27, 26, 25, 24,
    -1, -1, -1, -1, 23, 22, 21, 20,
    -1, -1, -1, -1, 19, 18, 17, 16,
    -1, -1, -1, -1, 15, 14, 13, 12,
    -1, -1, -1, -1, 11, 10,  9,  8,
    -1, -1, -1, -1,  7,  6,  5,  4,
    -1, -1, -1, -1,  3,  2,  1,  0,
], dtype=np.int32)
# fmt: on


def feature_index(pov: int, ksq: int, sq: int, piece_type: int, piece_color: int, fold_kings: bool = False) -> int:
    """Index of one piece seen from `pov` whose king stands on `ksq`."""
    flip = (56 if pov == BLACK else 0) ^ (7 if (ksq % 8) < 4 else 0)
    p_idx = 2 * piece_type + (1 if piece_color != pov else 0)
    planes = NUM_PLANES
    if fold_kings:
        p_idx = min(p_idx, 10)
        planes = 704
    return (sq ^ flip) + NUM_SQ * p_idx + planes * int(KING_BUCKETS[ksq ^ flip])


def encode_batch(squares, types, colors, fold_kings: bool = False):
    """Vectorised encoder.

    squares, types, colors: int arrays [B, 32]; unused slots have squares < 0.  Each position must
    hold exactly one king per colour.  Returns (white int32 [B,32], black int32 [B,32],
    piece_count int32 [B]); lists are in ascending square order and padded with -1.
    """
    squares = np.asarray(squares, dtype=np.int64)
    types = np.asarray(types, dtype=np.int64)
    colors = np.asarray(colors, dtype=np.int64)
    B, S = squares.shape
    present = squares >= 0
    # ascending square order, empty slots last
    order = np.argsort(np.where(present, squares, 1 << 20), axis=1, kind="stable")
    squares = np.take_along_axis(squares, order, 1)
    types = np.take_along_axis(types, order, 1)
    colors = np.take_along_axis(colors, order, 1)
    present = squares >= 0
    out = []
    for pov in (WHITE, BLACK):
        is_king = present & (types == KING) & (colors == pov)
        assert (is_king.sum(1) == 1).all(), "each side needs exactly one king"
        ksq = (squares * is_king).sum(1)
        flip = (56 if pov == BLACK else 0) ^ np.where((ksq % 8) < 4, 7, 0)
        p_idx = 2 * types + (colors != pov)
        planes = NUM_PLANES
        if fold_kings:
            p_idx = np.minimum(p_idx, 10)
            planes = 704
        bucket = KING_BUCKETS[ksq ^ flip].astype(np.int64)
        idx = (squares ^ flip[:, None]) + NUM_SQ * p_idx + planes * bucket[:, None]
        out.append(np.where(present, idx, -1).astype(np.int32)[:, :MAX_ACTIVE_FEATURES])
    return out[0], out[1], present.sum(1).astype(np.int32)


def random_positions(batch_size: int, seed: int, min_other: int = 2, max_other: int = 30,
                     castled_kings: float = 0.0):
    """Seeded synthetic positions: two kings on distinct squares plus U{min_other..max_other} other
    pieces with uniform type (pawn..queen) and colour on distinct non-king squares.

    castled_kings: fraction of positions whose kings stand on g1 / g8 (as in most game positions),
    which concentrates the batch on one king bucket per perspective; 0 keeps the kings uniform.

    Returns (squares, types, colors) int32 [B, 32] with -1 in unused slots; slot 0 is the white
    king, slot 1 the black king.
    """
    rng = np.random.default_rng(seed)
    B = batch_size
    keys = rng.random((B, 64))
    if castled_kings > 0.0:
        fixed = rng.random(B) < castled_kings
        keys[fixed, 6] = -2.0     # g1 sorts first: white king
        keys[fixed, 62] = -1.0    # g8 second: black king
    perm = np.argsort(keys, axis=1)[:, :32].astype(np.int32)
    n_other = rng.integers(min_other, max_other + 1, size=B)
    slot = np.arange(32)[None, :]
    used = slot < (2 + n_other)[:, None]
    types = rng.integers(PAWN, QUEEN + 1, size=(B, 32)).astype(np.int32)
    colors = rng.integers(0, 2, size=(B, 32)).astype(np.int32)
    types[:, 0] = KING
    types[:, 1] = KING
    colors[:, 0] = WHITE
    colors[:, 1] = BLACK
    squares = np.where(used, perm, -1).astype(np.int32)
    types = np.where(used, types, -1).astype(np.int32)
    colors = np.where(used, colors, -1).astype(np.int32)
    return squares, types, colors


def game_like_positions(batch_size: int, seed: int):
    """Seeded synthetic positions with the piece placement statistics of real game positions.

    game_like_stats.npz (written by tests/golden/make_game_like_stats.py from the reference's sample data) holds,
    per piece kind and square, how often it occurs from white's point of view with white's king
    mirrored onto files e-h: one table for each of white's three most common king buckets, one for
    the rest.  A position draws its class, the kings from their rows of the class's table, and
    every other (kind, square) independently with its frequency, one piece per square.  Most
    kings end up on their castled squares and most pawns near their home ranks, so one or two
    king buckets hold a large part of a batch and a few hundred table rows half of all slots,
    which uniform positions (random_positions) do not show.

    Returns (squares, types, colors) like random_positions.
    """
    import os

    stats = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "game_like_stats.npz"))
    freq, share = stats["freq"].astype(np.float64), stats["share"].astype(np.float64)
    rng = np.random.default_rng(seed)
    B = batch_size
    cls = rng.choice(len(share), size=B, p=share / share.sum())
    squares = np.full((B, 32), -1, np.int32)
    types = np.full((B, 32), -1, np.int32)
    colors = np.full((B, 32), -1, np.int32)
    for c in range(len(share)):
        rows = np.nonzero(cls == c)[0]
        n = len(rows)
        if n == 0:
            continue
        pk = freq[c, 10:12] / freq[c, 10:12].sum(1, keepdims=True)
        wk = rng.choice(64, size=n, p=pk[0])
        bk = rng.choice(64, size=n, p=pk[1])
        clash = wk == bk
        while clash.any():
            bk[clash] = rng.choice(64, size=int(clash.sum()), p=pk[1])
            clash = wk == bk
        # race between the ten other kinds on every square: kind k claims it when u_k < freq_k,
        # the smallest u_k / freq_k wins
        ratio = rng.random((n, 10, 64)) / np.maximum(freq[c, :10], 1e-12)[None]
        kind = ratio.argmin(1)
        taken = ratio.min(1) < 1.0
        sq = np.arange(64)[None, :]
        taken &= (sq != wk[:, None]) & (sq != bk[:, None])
        taken &= np.cumsum(taken, axis=1) <= 30    # at most 30 others (a surplus is rare)
        squares[rows, 0], types[rows, 0], colors[rows, 0] = wk, KING, WHITE
        squares[rows, 1], types[rows, 1], colors[rows, 1] = bk, KING, BLACK
        slot = 1 + np.cumsum(taken, axis=1)
        b_i, s_i = np.nonzero(taken)
        squares[rows[b_i], slot[b_i, s_i]] = s_i
        types[rows[b_i], slot[b_i, s_i]] = kind[b_i, s_i] // 2
        colors[rows[b_i], slot[b_i, s_i]] = kind[b_i, s_i] % 2
    return squares, types, colors


def synthetic_batch(batch_size: int, seed: int, fold_kings: bool = False, castled_kings: float = 0.0,
                    game_like: bool = False):
    """The batch tuple the loader hands the model (data_loader/_native.py:48-96), from seeded
    synthetic positions (random_positions, or game_like_positions when `game_like`): us f32 [B,1]
    ~ Bernoulli(1/2), them = 1 - us, white/black int32 [B,32], piece_count int64 [B].  numpy arrays."""
    if game_like:
        squares, types, colors = game_like_positions(batch_size, seed)
    else:
        squares, types, colors = random_positions(batch_size, seed, castled_kings=castled_kings)
    white, black, pc = encode_batch(squares, types, colors, fold_kings=fold_kings)
    rng = np.random.default_rng(seed + 7919)
    us = rng.integers(0, 2, size=(batch_size, 1)).astype(np.float32)
    them = (1.0 - us).astype(np.float32)
    return us, them, white, black, pc.astype(np.int64)


_PIECE_LETTERS = "pnbrqk"


def to_fen(squares, types, colors, white_to_move: bool = True) -> str:
    """FEN of one position (no castling rights, no en-passant square)."""
    board = {}
    for sq, t, c in zip(squares, types, colors):
        if sq >= 0:
            ch = _PIECE_LETTERS[int(t)]
            board[int(sq)] = ch.upper() if int(c) == WHITE else ch
    ranks = []
    for rank in range(7, -1, -1):
        row, empty = "", 0
        for file in range(8):
            ch = board.get(rank * 8 + file)
            if ch is None:
                empty += 1
            else:
                if empty:
                    row += str(empty)
                    empty = 0
                row += ch
        if empty:
            row += str(empty)
        ranks.append(row)
    return "/".join(ranks) + (" w" if white_to_move else " b") + " - - 0 1"
