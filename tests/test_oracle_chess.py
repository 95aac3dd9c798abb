"""Pins the chess/encoder checker (oracle/chess.c) against the known answers
the reference's own tests hold: perft counts (src/chess/board_test.cc:127-183,
Chess960 table :187-2126), repetition cases (src/chess/position_test.cc:60-154)
and the ten encoder cases (src/neural/encoder_test.cc:27-532)."""
import hashlib
import json
import os

import numpy as np
import pytest

from oracle import chess as oc

ALL = (1 << 64) - 1
GOLDEN = os.path.join(os.path.dirname(__file__), "golden")


@pytest.mark.parametrize("fen,counts", [
    (oc.STARTPOS_FEN, [20, 400, 8902, 197281]),
    ("r3k2r/p1ppqpb1/bn2pnp1/3PN3/1p2P3/2N2Q1p/PPPBBPPP/R3K2R w KQkq - 1 1", [48, 2039, 97862, 4085603]),
    ("8/2p5/3p4/KP5r/1R3p1k/8/4P1P1/8 w - - 1 1", [14, 191, 2812, 43238, 674624]),
    ("r2q1rk1/pP1p2pp/Q4n2/bbp1p3/Np6/1B3NBn/pPPP1PPP/R3K2R b KQ - 0 1", [6, 264, 9467, 422333]),
    ("rnbq1k1r/pp1Pbppp/2p5/8/2B5/8/PPP1NnPP/RNBQK2R w KQ - 1 8", [44, 1486, 62379, 2103487]),
    ("r4rk1/1pp1qppp/p1np1n2/2b1p1B1/2B1P1b1/P1NP1N2/1PP1QPPP/R4RK1 w - - 0 10", [46, 2079, 89890, 3894594]),
])
def test_perft_known_answers(fen, counts):
    for d, c in enumerate(counts, 1):
        assert oc.perft(fen, d) == c, (fen, d)


def test_perft_chess960():
    rows = json.load(open(os.path.join(GOLDEN, "chess960_perft.json")))
    assert len(rows) >= 10
    for row in rows:
        for d in range(3):
            assert oc.perft(row["fen"], d + 1) == row["perft"][d], (row["fen"], d + 1)


def test_fen_edge_cases():
    # board_test.cc:30-66 and :2223-2229
    with pytest.raises(ValueError):
        oc.perft("nqrbkrnr/bnnbnbnn/8/8/8/8/NNNBPNBN/QNRPKPQQ w - - 0 1", 1)
    for bad in ["rnbqkbnr/ppppppppp/8/8/8/8/PPPPPPPP/RNBQKBNR w KQkq - 0 1",
                "rnbqkbnr/pppppppp/8/8/8/8/PPPPPPPP/RNBQKBNR/8 w KQkq - 0 1",
                "rnbqkbnr/pppppppp/8/8/8/8/PPPPPPPP/RNBQKBNR g KQkq - 0 1",
                "rnbqkbnr/ppp2ppp/4p3/3pP3/8/8/PPPP1PPP/RNBQKBNR w KQkq i6 0 3",
                "rnbqkbnr/ppp2ppp/4p3/3pP3/8/8/PPPP1PPP/RNBQKBNR w KQkq A6 0 3"]:
        with pytest.raises(ValueError):
            oc.perft(bad, 1)
    h = oc.History("   k/1R//K   w   ")
    assert h.position(0).rule50 == 0


def test_knight_promotion_clears_en_passant_and_queen_move_is_not_en_passant():
    # board_test.cc:2232-2253
    h = oc.History("Q3b3/2P2pnk/3R3p/p7/1pp1p3/PnP1P2P/2B2PP1/5RK1 w - - 1 31")
    h.append_uci("c7c8")
    assert h.position(-1).pawns & ~0x00FFFFFFFFFFFF00 == 0
    h = oc.History("1Qnkr3/1p1b4/p2P2p1/P1q5/1NP3pP/1KN5/8/3R4 b - - 0 32")
    h.append_uci("b7b5")
    m = h.parse_move("b8c7")
    assert (m & 0x7000) != 0x2000
    h.append(m)
    assert [oc.move_to_uci(x, h.black_to_move()) for x in h.legal_moves()] == ["c5c7"]


REP_FEN = "3b4/rp1r1k2/8/1RP2p1p/p1KP4/P3P2P/5P2/1R2B3 b - - 2 30"
REP_MOVES = ["f7f8", "f2f4", "d7h7", "c4d3", "h7d7", "d3c4"]


def _hist(fen, moves):
    h = oc.History(fen)
    for m in moves:
        h.append_uci(m)
    return h


def test_repetitions():
    assert _hist(REP_FEN, REP_MOVES).position(-1).repetitions == 1
    # With a legal en passant in the first position the boards differ.
    h = _hist("3b4/rp1r1k2/8/1RP2p1p/p1KP2p1/P3P2P/5P2/1R2B3 b - - 2 30", REP_MOVES)
    assert h.position(-1).repetitions == 0
    assert _hist(REP_FEN, REP_MOVES).did_repeat_since_last_zeroing_move()
    assert _hist(REP_FEN, REP_MOVES + ["d7e7"]).did_repeat_since_last_zeroing_move()
    assert _hist(REP_FEN, REP_MOVES + ["d7e7", "c4b4"]).did_repeat_since_last_zeroing_move()
    assert not _hist(REP_FEN, REP_MOVES + ["d7e7", "c4b4", "h5h4"]).did_repeat_since_last_zeroing_move()


def _check_startpos_common(m, v):
    assert m[0] == sum(1 << (8 + i) for i in range(8)) and v[0] == 1.0
    assert m[1] == (1 << 1) | (1 << 6)
    assert m[2] == (1 << 2) | (1 << 5)
    assert m[3] == 1 | (1 << 7)
    assert m[4] == 1 << 3
    assert m[5] == 1 << 4
    assert m[11] == 1 << (8 * 7 + 4)
    assert all(int(x) == 0 for x in m[13:104])
    assert m[109] == ALL and v[109] == 0.0
    assert m[110] == 0
    assert m[111] == ALL and v[111] == 1.0


def test_encode_startpos_formats_1_2_3():
    h = oc.History()
    m, v, _ = h.encode(oc.INPUT_CLASSICAL_112_PLANE, 8, oc.FILL_NO)
    m = [int(x) for x in m]
    _check_startpos_common(m, v)
    assert m[104:108] == [ALL] * 4 and m[108] == 0
    for fmt in (oc.INPUT_112_WITH_CASTLING_PLANE, oc.INPUT_112_WITH_CANONICALIZATION):
        m, v, _ = h.encode(fmt, 8, oc.FILL_NO)
        m = [int(x) for x in m]
        _check_startpos_common(m, v)
        assert m[104] == 1 | (1 << 56)
        assert m[105] == (1 << 7) | (1 << 63)
        assert m[106] == 0 and m[107] == 0 and m[108] == 0


def test_encode_fifty_move_counter():
    h = oc.History()
    h.append_uci("g1f3")
    m, v, _ = h.encode(oc.INPUT_CLASSICAL_112_PLANE, 8, oc.FILL_NO)
    assert int(m[108]) == ALL and int(m[109]) == ALL and v[109] == 1.0
    h.append_uci("g8f6")
    m, v, _ = h.encode(oc.INPUT_CLASSICAL_112_PLANE, 8, oc.FILL_NO)
    assert int(m[108]) == 0 and int(m[109]) == ALL and v[109] == 2.0
    h = oc.History()
    h.append_uci("g1f3")
    m, v, _ = h.encode(oc.INPUT_112_WITH_CANONICALIZATION, 8, oc.FILL_NO)
    assert int(m[108]) == 0 and int(m[109]) == ALL
    h.append_uci("g8f6")
    m, v, _ = h.encode(oc.INPUT_112_WITH_CANONICALIZATION, 8, oc.FILL_NO)
    assert int(m[108]) == 0 and int(m[109]) == ALL and v[109] == 2.0


def test_encode_endgames_and_transforms():
    h = oc.History("3r4/4k3/8/1K6/8/8/8/8 w - - 0 1")
    m, _, t = h.encode(oc.INPUT_CLASSICAL_112_PLANE, 8, oc.FILL_NO)
    assert t == 0 and int(m[5]) == 1 << 33 and int(m[11]) == 1 << 52
    m, _, t = h.encode(oc.INPUT_112_WITH_CANONICALIZATION, 8, oc.FILL_NO)
    assert t == oc.FLIP_TRANSFORM | oc.MIRROR_TRANSFORM | oc.TRANSPOSE_TRANSFORM
    assert int(m[5]) == 1 << 12 and int(m[11]) == 1 << 38
    h = oc.History("3r4/4k3/2K5/8/8/8/8/8 w - - 0 1")
    m, _, t = h.encode(oc.INPUT_112_WITH_CANONICALIZATION, 8, oc.FILL_NO)
    assert t == oc.FLIP_TRANSFORM | oc.MIRROR_TRANSFORM
    assert int(m[5]) == 1 << 21 and int(m[11]) == 1 << 11


def test_encode_en_passant_format3():
    h = oc.History()
    for mv in ["e2e4", "g7g6", "e4e5", "f7f5"]:
        h.append_uci(mv)
    m, _, _ = h.encode(oc.INPUT_112_WITH_CANONICALIZATION, 8, oc.FILL_NO)
    assert int(m[108]) == 1 << 61
    assert all(int(x) == 0 for x in m[13:104])
    h.append_uci("g1f3")
    m, _, _ = h.encode(oc.INPUT_112_WITH_CANONICALIZATION, 8, oc.FILL_NO)
    assert int(m[108]) == 0
    assert all(int(x) == 0 for x in m[13:104])
    h.append_uci("g8f5")  # the reference test plays this (illegal but accepted) move
    m, _, _ = h.encode(oc.INPUT_112_WITH_CANONICALIZATION, 8, oc.FILL_NO)
    for i in range(7):
        for j in range(13):
            x = int(m[13 + i * 13 + j])
            if i == 0 and j < 12:
                assert x != 0
            else:
                assert x == 0


def test_encode_early_game_flip_format3():
    h = oc.History()
    for mv in ["e2e4", "e7e5", "e1e2", "e8e7", "e2d3"]:
        h.append_uci(mv)
    m, _, t = h.encode(oc.INPUT_112_WITH_CANONICALIZATION, 8, oc.FILL_NO)
    assert t == 0 and int(m[5]) == 1 << 12 and int(m[11]) == 1 << 43
    h.append_uci("e7e6")
    m, _, t = h.encode(oc.INPUT_112_WITH_CANONICALIZATION, 8, oc.FILL_NO)
    assert t == oc.FLIP_TRANSFORM and int(m[5]) == 1 << 20 and int(m[11]) == 1 << 43


def test_move_table_hash_and_index_properties():
    strs = oc.move_strs()
    assert len(strs) == 1858 and len(set(strs)) == 1858
    # SHA-256 of the reference's kMoveStrs joined by newlines (encoder.cc:339-572).
    assert hashlib.sha256("\n".join(strs).encode()).hexdigest() == \
        "4a901f49851725496e39e34648dd58f240950fa6b72a0bbf6b2816b9af767cc7"
    # Every legal move of random positions maps to a distinct index whose move
    # string is the move itself seen from the mover's side.
    pos = oc.random_positions(64, seed=7)
    for lg in pos["legal"]:
        assert len(set(lg.tolist())) == len(lg) and lg.min() >= 0 and lg.max() < 1858


def test_encoder_invariants_on_random_playouts():
    pos = oc.random_positions(200, seed=123)
    masks, values = pos["masks"], pos["values"]
    assert (masks[:, 111] == np.uint64(ALL)).all()
    assert (masks[:, 110] == 0).all()
    assert (values[:, :109] == 1.0).all()
    for i in range(200):
        m = [int(x) for x in masks[i]]
        ours = 0
        for p in range(6):
            assert ours & m[p] == 0
            ours |= m[p]
        theirs = 0
        for p in range(6, 12):
            assert (ours | theirs) & m[p] == 0
            theirs |= m[p]
        assert bin(m[5]).count("1") == 1 and bin(m[11]).count("1") == 1
        plies = len(pos["uci"][i].split())
        assert (m[108] == ALL) == (plies % 2 == 1)
        assert 0 <= values[i, 109] <= plies


def test_colour_flip_symmetry():
    """Encoding is from the mover's view: a position with black to move encodes
    like its colour-swapped, rank-mirrored twin with white to move (except the
    side-to-move plane 108)."""
    fen_b = "r1bqkbnr/pppp1ppp/2n5/4p3/4P3/5N2/PPPP1PPP/RNBQKB1R b KQkq - 2 2"
    fen_w = "rnbqkb1r/pppp1ppp/5n2/4p3/4P3/2N5/PPPP1PPP/R1BQKBNR w KQkq - 2 2"
    mb, vb, _ = oc.History(fen_b).encode(fill=oc.FILL_NO)
    mw, vw, _ = oc.History(fen_w).encode(fill=oc.FILL_NO)
    idx = [i for i in range(112) if i != 108]
    assert (mb[idx] == mw[idx]).all() and (vb == vw).all()
    assert int(mb[108]) == ALL and int(mw[108]) == 0
