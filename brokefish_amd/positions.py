"""Synthetic positions for tests and benchmarks: seeded uniformly random legal playouts.

Wraps the CPU rules engine in ``csrc/chessgen.c`` (built by ``brokefish_amd._build``).
Mirrors what the reference's position fixture does (tests/boards.py:23-72): each game
walks uniformly random legal moves from the start, a game with no legal move stays where
it is, ``rep = i mod 3``, and optionally a queen is stamped into pawn slot 3 of every
seventh board so a promoted piece in a pawn slot is always present.
"""
from __future__ import annotations

import ctypes as C
import os

import numpy as np
import torch

from . import _build

_lib = None


def lib():
    global _lib
    if _lib is None:
        path = _build.CHESSGEN_LIB
        if not os.path.exists(path):
            _build.build_chessgen()
        L = C.CDLL(path)
        L.bf_chess_perft.restype = C.c_uint64
        L.bf_chess_perft.argtypes = [C.c_void_p, C.c_int16, C.c_int]
        L.bf_chess_from_fen.restype = C.c_int
        L.bf_chess_from_fen.argtypes = [C.c_char_p, C.c_void_p, C.c_void_p]
        L.bf_chess_initial.argtypes = [C.c_void_p, C.c_void_p]
        L.bf_chess_movegen.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_void_p]
        L.bf_chess_step.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int]
        L.bf_chess_random_playouts.argtypes = [C.c_int, C.c_int, C.c_uint64, C.c_uint64,
                                               C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]
        _lib = L
    return _lib


def from_fen(fen: str):
    """FEN -> (board [32] uint16, control int)."""
    b = np.zeros(32, np.uint16)
    c = np.zeros(1, np.int16)
    rc = lib().bf_chess_from_fen(fen.encode(), b.ctypes.data, c.ctypes.data)
    if rc:
        raise ValueError(f"bad FEN ({rc}): {fen!r}")
    return b, int(c[0])


def perft(board: np.ndarray, control: int, depth: int) -> int:
    b = np.ascontiguousarray(board, dtype=np.uint16)
    return int(lib().bf_chess_perft(b.ctypes.data, int(control), int(depth)))


def movegen(boards: np.ndarray, control: np.ndarray):
    """(mask [n,32] uint64, in_check [n] uint8) for uint16 boards [n,32], int16 control [n]."""
    b = np.ascontiguousarray(boards, dtype=np.uint16)
    c = np.ascontiguousarray(control, dtype=np.int16)
    n = b.shape[0]
    mask = np.zeros((n, 32), np.uint64)
    chk = np.zeros(n, np.uint8)
    lib().bf_chess_movegen(b.ctypes.data, c.ctypes.data, n, mask.ctypes.data, chk.ctypes.data)
    return mask, chk


def step(boards: np.ndarray, control: np.ndarray, move: np.ndarray, promo: np.ndarray):
    """Apply ``move[i] = slot * 64 + target`` (promotion type ``promo[i]``: 0 N, 1 B, 2 R, 3 Q) to
    position i; returns new (boards uint16 [n,32], control int16 [n])."""
    b = np.array(boards, dtype=np.uint16, copy=True)
    c = np.array(control, dtype=np.int16, copy=True)
    mv = np.ascontiguousarray(move, dtype=np.int16)
    pr = np.ascontiguousarray(promo, dtype=np.uint8)
    lib().bf_chess_step(b.ctypes.data, c.ctypes.data, mv.ctypes.data, pr.ctypes.data, b.shape[0])
    return b, c


def random_positions_np(n: int, plies: int = 120, seed: int = 0, first_game: int = 0,
                        stamp_queen: bool = False):
    """numpy version: boards uint16 [n,32], control int16 [n], rep uint8 [n], mask uint64 [n,32].

    Game i plays U{0..plies} random legal moves.  The result for game i depends only on
    (seed, first_game + i), not on the batch it is generated in.
    """
    boards = np.zeros((n, 32), np.uint16)
    control = np.zeros(n, np.int16)
    rep = np.zeros(n, np.uint8)
    mask = np.zeros((n, 32), np.uint64)
    lib().bf_chess_random_playouts(n, plies, seed, first_game, boards.ctypes.data,
                                   control.ctypes.data, rep.ctypes.data, mask.ctypes.data)
    if stamp_queen:
        idx = np.arange(n) % 7 == 0
        live = (boards[:, 3] & 0x800) == 0
        sel = idx & live
        boards[sel, 3] = (boards[sel, 3] & ~np.uint16(7 << 6)) | np.uint16(4 << 6)
        mask, _ = movegen(boards, control)
    return boards, control, rep, mask


def random_positions(n: int, plies: int = 120, seed: int = 0, device="cpu", stamp_queen: bool = False,
                     with_mask: bool = True):
    """torch version with the evaluator's dtypes: boards int16 [n,32], control int16 [n],
    rep uint8 [n], mask int64 [n,32] (uint64 bit patterns)."""
    b, c, r, m = random_positions_np(n, plies, seed, 0, stamp_queen)
    out = (torch.from_numpy(b.view(np.int16)).to(device), torch.from_numpy(c).to(device),
           torch.from_numpy(r).to(device))
    if with_mask:
        out = out + (torch.from_numpy(m.view(np.int64)).to(device),)
    return out
