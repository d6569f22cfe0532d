"""The CPU rules engine that makes synthetic positions and legal-move masks.

Pinned by the published perft node counts the reference's own environment tests hold
(reference tests/test_env.py:42-69) -- an external oracle -- and by the structural
invariants of the position format (reference docs/reference/spec.md:108-116).
"""
import numpy as np
import pytest

from brokefish_amd import positions

START = "rnbqkbnr/pppppppp/8/8/8/8/PPPPPPPP/RNBQKBNR w KQkq - 0 1"
PERFT = [
    (START, [20, 400, 8902, 197281]),
    ("r3k2r/p1ppqpb1/bn2pnp1/3PN3/1p2P3/2N2Q1p/PPPBBPPP/R3K2R w KQkq - 0 1", [48, 2039, 97862]),
    ("8/2p5/3p4/KP5r/1R3p1k/8/4P1P1/8 w - - 0 1", [14, 191, 2812, 43238]),
    ("r3k2r/Pppp1ppp/1b3nbN/nP6/BBP1P3/q4N2/Pp1P2PP/R2Q1RK1 w kq - 0 1", [6, 264, 9467]),
    ("rnbq1k1r/pp1Pbppp/2p5/8/2B5/8/PPP1NnPP/RNBQK2R w KQ - 1 8", [44, 1486, 62379]),
    ("r4rk1/1pp1qppp/p1np1n2/2b1p1B1/2B1P1b1/P1NP1N2/1PP1QPPP/R4RK1 w - - 0 10", [46, 2079, 89890]),
]
DEEP = [(START, 5, 4865609), (PERFT[1][0], 4, 4085603), (PERFT[2][0], 5, 674624),
        (PERFT[3][0], 4, 422333), (PERFT[4][0], 4, 2103487), (PERFT[5][0], 4, 3894594)]


@pytest.mark.parametrize("fen,counts", PERFT)
def test_perft_matches_published_counts(fen, counts):
    board, control = positions.from_fen(fen)
    assert [positions.perft(board, control, d + 1) for d in range(len(counts))] == counts


@pytest.mark.parametrize("fen,depth,count", DEEP)
def test_perft_one_ply_deeper(fen, depth, count):
    board, control = positions.from_fen(fen)
    assert positions.perft(board, control, depth) == count


def test_start_position_words():
    board, control = positions.from_fen(START)
    assert control == 1
    assert board[15] == (5 << 6) | 4 and board[31] == (1 << 10) | (5 << 6) | 60
    assert list(board[:8]) == list(range(8, 16))


def test_fen_special_bits_and_promoted_material():
    # no castling rights: kings and rooks carry the special ("has moved") bit
    board, control = positions.from_fen("r3k2r/8/8/8/8/8/8/R3K2R b - - 12 40")
    assert control == -13
    for slot in (12, 13, 15, 28, 29, 31):
        assert board[slot] & 0x200
    # three white queens: two live in pawn slots with type bits overwritten
    board, _ = positions.from_fen("4k3/8/8/8/8/8/8/QQQ1K3 w - - 0 1")
    assert (board[14] >> 6) & 7 == 4
    assert sorted(((w >> 6) & 7) for w in board[:8] if not w & 0x800) == [4, 4]
    # en passant target: the pawn that just double-pushed carries the flag
    board, _ = positions.from_fen("rnbqkbnr/pppp1ppp/8/8/4pP2/8/PPPPP1PP/RNBQKBNR b KQkq f3 0 3")
    flagged = [w for w in board if not w & 0x800 and (w >> 6) & 7 == 0 and w & 0x200]
    assert len(flagged) == 1 and flagged[0] & 63 == 29


def test_playouts_keep_the_format_invariants():
    b, c, r, m = positions.random_positions_np(512, plies=120, seed=5)
    alive = (b & 0x800) == 0
    assert alive[:, 15].all() and alive[:, 31].all()                 # kings never captured
    assert ((b[:, 15] >> 6) & 7 == 5).all() and ((b[:, 31] >> 6) & 7 == 5).all()
    assert (b[~alive] == 0x800).all()                                # dead slots are wiped
    assert (b >> 12 == 0).all()
    assert (((b >> 10) & 1)[:, :16][alive[:, :16]] == 0).all()       # colour follows the slot half
    assert (((b >> 10) & 1)[:, 16:][alive[:, 16:]] == 1).all()
    for i in range(b.shape[0]):                                      # no two live pieces share a square
        sq = (b[i] & 63)[alive[i]]
        assert len(set(sq.tolist())) == len(sq)
    pawn_flag = alive & (((b >> 6) & 7) == 0) & ((b & 0x200) != 0)
    assert (pawn_flag.sum(1) <= 1).all()                             # at most one en-passant target
    assert (c != 0).all() and (r == np.arange(512) % 3).all()
    # the mask belongs to the side to move and never targets an own piece
    stm_black = c < 0
    own = ((b >> 10) & 1) == stm_black[:, None]
    assert (m[~(own & alive)] == 0).all()
    assert ((c != 0) & (np.abs(c.astype(np.int32)) <= 121)).all()
    assert len(set(np.abs(c.astype(np.int32)).tolist())) > 10        # a spread of clocks


def test_playouts_are_seeded_and_batch_independent():
    a = positions.random_positions_np(64, plies=60, seed=9)
    b = positions.random_positions_np(64, plies=60, seed=9)
    for x, y in zip(a, b):
        assert (x == y).all()
    c = positions.random_positions_np(16, plies=60, seed=9, first_game=48)
    for x, y in zip(a, c):
        assert (x[48:] == y).all()
    d = positions.random_positions_np(64, plies=60, seed=10)
    assert (a[0] != d[0]).any()


def test_mask_agrees_with_movegen_and_step():
    b, c, r, m = positions.random_positions_np(128, plies=80, seed=2)
    m2, chk = positions.movegen(b, c)
    assert (m == m2).all()
    # zero plies is the initial position with its 20 legal moves
    b0, c0, _, m0 = positions.random_positions_np(4, plies=0, seed=1)
    assert (c0 == 1).all() and all(int(np.unpackbits(m0[i].view(np.uint8)).sum()) == 20 for i in range(4))


# --------------------------------------------------------------------------- #
# The reference's own edge-case positions (tests/edge_positions.py), against what the rules of
# chess fix for them.  The device twin of this test is tests/test_edge_positions_gpu.py.
# --------------------------------------------------------------------------- #

def _edge_masks():
    import edge_positions as ep
    boards, control = ep.boards_of()
    mask, check = positions.movegen(boards, control)
    by = {n: i for i, n in enumerate(ep.NAMES)}
    return ep, boards, control, mask, check, by


def check_edge_position_facts(ep, boards, control, mask, check, by):
    """Facts chess fixes for the edge-case positions, given any generator's masks."""
    sq = ep.square
    count = lambda n: sum(bin(int(w)).count("1") for w in mask[by[n]])
    mv = lambda n: ep.moves_of(boards[by[n]], mask[by[n]])
    assert count("max-mobility") == 218 and count("startpos") == 20
    # nine white queens: one in the queen's slot, eight living in pawn slots
    b = boards[by["max-mobility"]]
    assert sum(1 for w in b[:16] if not w & 0x800 and (w >> 6) & 7 == 4) == 9
    assert sum(1 for w in b[:8] if not w & 0x800 and (w >> 6) & 7 == 4) == 8
    assert int(((boards[by["bare-kings-and-a-rook"]] & 0x800) == 0).sum()) == 3
    # mate (the fool's mate: in check, no move) and stalemate (not in check, no move): all-zero masks
    assert check[by["check-by-queen"]] and not mask[by["check-by-queen"]].any()
    assert not check[by["stalemate-queen"]] and not mask[by["stalemate-queen"]].any()
    assert mv("single-reply-rook") == {(sq("g8"), sq("h8"))}
    assert not check[by["white-queen-on-h4-black-to-move"]] and count("white-queen-on-h4-black-to-move") == 25
    # castling: both ways when free, none out of check, without rights or through a piece
    e1, e8 = sq("e1"), sq("e8")
    assert {(e1, sq("g1")), (e1, sq("c1"))} <= mv("castle-both-white")
    assert {(e8, sq("g8")), (e8, sq("c8"))} <= mv("castle-both-black")
    for n, k, tg in (("castle-white-in-check", e1, ("g1", "c1")), ("castle-black-in-check", e8, ("g8", "c8")),
                     ("castle-rights-lost", e1, ("g1", "c1"))):
        assert not {(k, sq(t)) for t in tg} & mv(n), n
    assert check[by["castle-white-in-check"]] and check[by["castle-black-in-check"]]
    blocked = mv("castle-blocked")
    assert (e1, sq("c1")) in blocked and (e1, sq("g1")) not in blocked       # the knight stands on g1
    # en passant: taken when it is legal (also as the answer to the pawn's check, and by either
    # neighbour), absent when it would open the rank between queen and king
    assert (sq("d4"), sq("e3")) in mv("en-passant-plain")
    assert {(sq("d4"), sq("e3")), (sq("f4"), sq("e3"))} <= mv("en-passant-two-capturers")
    assert (sq("d4"), sq("e3")) not in mv("en-passant-pinned") and (sq("d4"), sq("d3")) in mv("en-passant-pinned")
    assert check[by["en-passant-out-of-check"]] and (sq("e4"), sq("d3")) in mv("en-passant-out-of-check")
    # promotions by push and by capture; the pinned pawn may not move; checks restrict the replies
    assert (sq("a7"), sq("a8")) in mv("promotion-by-push")
    assert not any(f == sq("d2") for f, _ in mv("pinned-pawn"))
    assert check[by["check-by-bishop"]] and 0 < count("check-by-bishop") < 10
    assert check[by["promotion-race"]] and count("promotion-race") == 2             # the b2 pawn gives check
    # the fifty-move clock is carried in the control word: magnitude = clock + 1
    assert control[by["fifty-move-100"]] == 101 and control[by["fifty-move-99"]] == 100
    # four legal replies, each the only bit of its word and each bit 62: the words sum to 2**64
    words = [int(w) for w in mask[by["mask-words-sum-to-2-pow-64"]] if w]
    assert words == [1 << 62] * 4 and sum(words) == 1 << 64


def test_reference_edge_case_positions_on_the_cpu_generator():
    check_edge_position_facts(*_edge_masks())
