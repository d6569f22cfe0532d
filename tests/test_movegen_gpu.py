"""Device move generation against the CPU generator (which the published perft counts pin,
tests/test_positions.py): legal-move words and in-check flags must be bit-identical.

Positions: everything reachable within two plies (three for the sparse end-game position) of the
six perft positions the reference's environment tests use (reference tests/test_env.py:42-69 --
chosen for castling through and out of check, en-passant pins, promotions with capture, double
checks), every promotion type included, plus 20,000 random playouts of up to 200 plies.
"""
import numpy as np
import pytest
import torch

from brokefish_amd import positions
from test_positions import PERFT

pytestmark = pytest.mark.gpu


def _frontier(fen, plies):
    b, c = positions.from_fen(fen)
    boards, control = b[None].copy(), np.array([c], np.int16)
    seen_b, seen_c = [boards], [control]
    for _ in range(plies):
        mask, _ = positions.movegen(boards, control)
        src, mv, pr = [], [], []
        for i in range(boards.shape[0]):
            last = 0 if control[i] < 0 else 7
            for p in range(32):
                w, m = int(boards[i, p]), int(mask[i, p])
                pawn = not (w & 0x800) and ((w >> 6) & 7) == 0
                while m:
                    s = (m & -m).bit_length() - 1
                    m &= m - 1
                    for k in (range(4) if pawn and s // 8 == last else (3,)):
                        src.append(i); mv.append(p * 64 + s); pr.append(k)
        if not src:
            break
        boards, control = positions.step(boards[src], control[src], np.array(mv), np.array(pr))
        seen_b.append(boards); seen_c.append(control)
    return np.concatenate(seen_b), np.concatenate(seen_c)


def _compare(boards, control):
    from brokefish_amd.hip_impl import movegen
    want_m, want_c = positions.movegen(boards, control)
    bt = torch.from_numpy(np.ascontiguousarray(boards).view(np.int16)).cuda()
    ct = torch.from_numpy(np.ascontiguousarray(control)).cuda()
    got_m, got_c = movegen(bt, ct)
    gm = got_m.cpu().numpy().view(np.uint64)
    bad = np.nonzero((gm != want_m).any(1))[0]
    assert bad.size == 0, (bad[:5], boards[bad[0]].tolist(), int(control[bad[0]]),
                           [hex(int(x)) for x in gm[bad[0]]], [hex(int(x)) for x in want_m[bad[0]]])
    assert (got_c.cpu().numpy() == (want_c != 0)).all()
    return want_m, want_c


@pytest.mark.parametrize("idx", range(len(PERFT)))
def test_every_position_near_the_perft_suite(idx):
    fen, counts = PERFT[idx]
    boards, control = _frontier(fen, 3 if idx == 2 else 2)
    assert boards.shape[0] >= 1 + counts[0] + counts[1]
    want_m, want_c = _compare(boards, control)
    # the frontier reproduces the published counts (a promoting move counts once per piece type)
    from oracle import expand as ox
    edges = [len(ox.candidates(boards[i], int(control[i]), want_m[i])) for i in range(1 + counts[0])]
    assert edges[0] == counts[0] and sum(edges[1:]) == counts[1]
    assert want_c.sum() > 0 or idx == 0


def test_twenty_thousand_random_playouts():
    b, c, r, m = positions.random_positions_np(20000, plies=200, seed=77, stamp_queen=True)
    want_m, want_c = _compare(b, c)
    assert (want_m == m).all()                                   # the generator's own mask, re-derived
    assert want_c.mean() > 0.02                                  # checks do occur in the sample
    # and it chains: evaluator + expansion from a mask that never left the device
    from brokefish_amd import encoder_impl
    from brokefish_amd.net import BrokefishNet
    torch.manual_seed(0)
    model = encoder_impl("hip")(BrokefishNet().eval(), int8=True)
    bt, ct, rt = (torch.from_numpy(np.ascontiguousarray(x[:500])).cuda() for x in (b.view(np.int16), c, r))
    mt = torch.from_numpy(m[:500].view(np.int64)).cuda()
    dev = model.forward_expand(bt, ct, rt)                       # mask generated on the device
    host = model.forward_expand(bt, ct, rt, mt)
    assert torch.equal(dev["mask"], mt)
    for k in ("edge_move", "edge_prior", "n_edges", "count"):
        assert torch.equal(dev[k], host[k]), k
