"""The edge-case positions the reference keeps for its own evaluator and rules tests, as data.

ADVERSARIAL: reference brokefish/nn/validate.py:81-87 (positions no random playout produces: 218
legal moves -- the edge cap and the widest softmax, nine queens living in pawn slots; almost every
slot dead; a promotion race).  SPECIAL: reference scripts/dump_cuda_testset.py:87-127 (rules that
random play reaches rarely or never: castling through check, the pinned en-passant capture, mate
and stalemate, the fifty-move boundary, and the position whose four mask words sum to 2**64).
Only the FEN strings are taken over; they are inputs, and the names given to them here say what
the rules of chess make of each (of the three positions the reference files under "mate and
stalemate", one is a stalemate, one leaves a single reply and one is an ordinary position; the
mate of that list's "check" group is the fool's mate).
"""
import numpy as np

from brokefish_amd import positions

ADVERSARIAL = (
    ("max-mobility", "R6R/3Q4/1Q4Q1/4Q3/2Q4Q/Q4Q2/pp1Q4/kBNN1KB1 w - - 0 1"),
    ("bare-kings-and-a-rook", "4k3/8/8/8/8/8/8/4K2R w K - 0 1"),
    ("promotion-race", "8/PPPPPPPP/8/8/8/8/pppppppp/K6k w - - 0 1"),
    ("startpos", "rnbqkbnr/pppppppp/8/8/8/8/PPPPPPPP/RNBQKBNR w KQkq - 0 1"),
    ("endgame-kq-vs-k", "8/8/8/4k3/8/8/4KQ2/8 w - - 0 1"),
)

SPECIAL = (
    ("castle-both-white", "r3k2r/pppppppp/8/8/8/8/PPPPPPPP/R3K2R w KQkq - 0 1"),
    ("castle-both-black", "r3k2r/pppppppp/8/8/8/8/PPPPPPPP/R3K2R b KQkq - 0 1"),
    ("castle-white-in-check", "r3k2r/8/8/8/8/4r3/8/R3K2R w KQkq - 0 1"),
    ("castle-black-in-check", "r3k2r/8/5N2/8/8/8/8/R3K2R b KQkq - 0 1"),
    ("castle-rights-lost", "r3k2r/pppppppp/8/8/8/8/PPPPPPPP/R3K2R w - - 0 1"),
    ("castle-blocked", "rn2k2r/8/8/8/8/8/8/R3K1NR w KQkq - 0 1"),
    ("en-passant-plain", "rnbqkbnr/ppp1pppp/8/8/3pP3/8/PPPP1PPP/RNBQKBNR b KQkq e3 0 3"),
    ("en-passant-two-capturers", "rnbqkbnr/ppp1p1pp/8/8/3pPp2/8/PPPP1PPP/RNBQKBNR b KQkq e3 0 4"),
    ("en-passant-pinned", "8/8/8/8/k2pP2Q/8/8/4K3 b - e3 0 1"),
    ("en-passant-out-of-check", "8/8/8/2k5/3Pp3/8/8/4K3 b - d3 0 1"),
    ("promotion-by-push", "8/P7/8/8/8/8/p7/K6k w - - 0 1"),
    ("promotion-by-capture", "1n6/P7/8/8/8/8/p6K/1N5k b - - 0 1"),
    ("check-by-queen", "rnb1kbnr/pppp1ppp/8/4p3/6Pq/5P2/PPPPP2P/RNBQKBNR w KQkq - 1 3"),
    ("check-by-bishop", "rnbqk1nr/pppp1ppp/8/4p3/1b6/3P4/PPP1PPPP/RNBQKBNR w KQkq - 2 3"),
    ("pinned-pawn", "4k3/8/8/8/1b6/8/3P4/4K3 w - - 0 1"),
    ("white-queen-on-h4-black-to-move", "rnb1kbnr/pppp1ppp/8/4p3/6PQ/5P2/PPPPP2P/RNB1KBNR b KQkq - 0 3"),
    ("stalemate-queen", "7k/5Q2/6K1/8/8/8/8/8 b - - 0 1"),
    ("single-reply-rook", "6k1/5R2/6K1/8/8/8/8/8 b - - 0 1"),
    ("bare-kings", "8/8/8/3k4/8/3K4/8/8 w - - 0 1"),
    ("two-pawns", "8/2p5/8/8/8/8/6P1/K6k w - - 0 1"),
    ("fifty-move-100", "8/8/8/3k4/8/8/4Q3/4K3 w - - 100 1"),
    ("fifty-move-99", "8/8/8/3k4/8/8/4Q3/4K3 w - - 99 1"),
    ("bishops-same-colour", "8/8/8/3k4/8/8/8/B1B1K3 w - - 0 1"),
    ("bishops-opposite-colour", "8/8/8/3k4/8/8/8/BB2K3 w - - 0 1"),
    ("mask-words-sum-to-2-pow-64", "1r1r2Rk/pp5p/4b2n/1P5P/n1Ppp3/R4P1p/1B1KP3/8 b - - 1 1"),
)

ALL = ADVERSARIAL + SPECIAL
NAMES = [n for n, _ in ALL]


def boards_of(entries=ALL):
    """(boards uint16 [n,32], control int16 [n]) of the listed positions."""
    bc = [positions.from_fen(f) for _, f in entries]
    return np.stack([b for b, _ in bc]), np.array([c for _, c in bc], np.int16)


def square(name: str) -> int:
    return (ord(name[0]) - ord("a")) + 8 * (int(name[1]) - 1)


def moves_of(board, mask):
    """{(from square, to square)} of one position's mask words."""
    out = set()
    for p in range(32):
        w, m = int(board[p]), int(mask[p])
        for s in range(64):
            if (m >> s) & 1:
                out.add((w & 63, s))
    return out
