"""The search's expand step behind the evaluator (docs/reference/search.md:616-636).

CPU part: pins ``oracle/expand.py`` by what the reference's own ``Search._expand`` wrote for 38
positions (tests/golden/reference_vectors_expand.npz), by hand-built positions, by the properties
the reference's own tests assert (tests/test_search.py:317-372) and by brute-force definitions on
small cases.
GPU part (marked): the HIP kernel against that checker through the C-ABI -- move codes, edge
counts and candidate counts exactly; priors to fp16 rounding of the exact value (tolerance
6e-4 relative + 6e-8: half an fp16 ulp plus the fp32 evaluation error); the kept set under
truncation exactly wherever the checker's margin between the last kept and the first dropped
log-prior exceeds 1e-5 (closer than that, fp32 and float64 may order two candidates differently).
"""
import numpy as np
import pytest
import torch

from brokefish_amd import positions
from oracle import expand as ox

PROMOTION = "8/P7/8/8/8/8/8/K6k w - - 0 1"          # reference tests/test_search.py:39


def _logits(n, seed, scale=2.0):
    g = np.random.default_rng(seed)
    return (g.standard_normal((n, 32, 64)) * scale).astype(np.float32), \
           g.standard_normal((n, 32, 4)).astype(np.float32), np.tanh(g.standard_normal(n)).astype(np.float32)


def test_canonical_order_and_promotion_fan_out_on_a_hand_built_position():
    board = np.full(32, 0x800, np.uint16)                      # everything dead ...
    board[3] = (0 << 6) | 54                                   # white pawn on g7
    board[2] = (4 << 6) | 51                                   # a promoted queen in pawn slot 2, on d7
    board[8] = (1 << 6) | 1                                    # white knight on b1
    board[15] = (5 << 6) | 4
    board[31] = (1 << 10) | (5 << 6) | 60
    mask = np.zeros(32, np.uint64)
    mask[3] = (1 << 62) | (1 << 63)                            # g8, and a capture on h8: both promote
    mask[2] = (1 << 59) | (1 << 43)                            # the queen to d8 (last rank, NOT a promotion) and d6
    mask[8] = (1 << 16) | (1 << 18)
    want = [(2 * 64 + 43, 0), (2 * 64 + 59, 0)] + [(3 * 64 + 62, k) for k in range(4)] + \
           [(3 * 64 + 63, k) for k in range(4)] + [(8 * 64 + 16, 0), (8 * 64 + 18, 0)]
    assert ox.candidates(board, 1, mask) == want
    # black to move: the last rank is rank 1; a white pawn's bit on rank 8 is then no promotion
    bb = board.copy()
    bb[19] = (1 << 10) | (0 << 6) | 9                          # black pawn on b2
    mb = np.zeros(32, np.uint64)
    mb[19] = (1 << 0) | (1 << 1)
    mb[3] = 1 << 62
    assert ox.candidates(bb, -5, mb) == [(3 * 64 + 62, 0)] + [(19 * 64 + 0, k) for k in range(4)] + \
        [(19 * 64 + 1, k) for k in range(4)]
    # a dead slot never promotes, whatever its (wiped) type bits say
    dead = board.copy()
    dead[3] = 0x800
    assert ox.candidates(dead, 1, mask)[2] == (3 * 64 + 62, 0)


def test_reference_test_properties_on_the_promotion_position():
    b, c = positions.from_fen(PROMOTION)
    mask, _ = positions.movegen(b[None], np.array([c], np.int16))
    bits = int(sum(bin(int(w)).count("1") for w in mask[0]))
    pol, pro, val = _logits(1, 0)
    out = ox.expand(pol, pro, val, mask, b[None], np.array([c]), 96)
    ne = int(out["n_edges"][0])
    labels = out["edge_move"][0, :ne].astype(np.int64) & 0xFFFF
    moves, promos = labels & ((1 << ox.MOVE_BITS) - 1), labels >> ox.MOVE_BITS
    pairs = list(zip(moves.tolist(), promos.tolist()))
    assert sorted(pairs) == pairs                               # ascending slot, square, then N B R Q
    assert sum(1 for m in set(moves.tolist()) if moves.tolist().count(m) == 4) == 1
    assert ne == bits + 3 == out["count"][0]
    assert abs(out["edge_prior"][0, :ne].sum() - 1.0) < 1e-12 and (out["edge_prior"][0, ne:] == 0).all()
    group = np.nonzero(moves == moves[promos == 3][0])[0]
    share = out["edge_prior"][0, group] / out["edge_prior"][0, group].sum()
    want = np.exp(pro[0, moves[group[0]] // 64].astype(np.float64))
    assert np.allclose(share, want / want.sum(), atol=1e-12)    # P(type | piece) splits the move's mass
    # ... and the move's total mass is what its policy logit alone would get
    z = np.exp(pol[0].astype(np.float64))
    legal = np.array([[(int(mask[0, p]) >> s) & 1 for s in range(64)] for p in range(32)], bool)
    mv = int(moves[group[0]])
    assert np.isclose(out["edge_prior"][0, group].sum(), z[mv // 64, mv % 64] / z[legal].sum(), atol=1e-12)
    assert np.isclose(out["node_value"][0], (val[0] + 1) / 2)


def test_start_position_has_twenty_edges_in_order():
    b, c = positions.from_fen("rnbqkbnr/pppppppp/8/8/8/8/PPPPPPPP/RNBQKBNR w KQkq - 0 1")
    mask, _ = positions.movegen(b[None], np.array([c], np.int16))
    pol, pro, val = _logits(1, 1)
    out = ox.expand(pol, pro, val, mask, b[None], np.array([c]), 96)
    assert out["n_edges"][0] == 20 and out["dropped"][0] == 0
    mv = out["edge_move"][0, :20].tolist()
    assert mv == sorted(mv) and all(m < 2048 for m in mv)


def test_truncation_keeps_the_largest_with_ties_by_order_brute_force():
    b, c, r, m = positions.random_positions_np(40, plies=60, seed=3)
    pol, pro, val = _logits(40, 2)
    pol = np.round(pol)                                        # many exact ties
    for E in (1, 4, 7):
        out = ox.expand(pol, pro, val, m, b, c, E)
        for i in range(40):
            cand = ox.candidates(b[i], int(c[i]), m[i])
            if not cand:
                continue
            x = pro[i].astype(np.float64) - pro[i].max(-1, keepdims=True)
            lp = x - np.log(np.exp(x).sum(-1, keepdims=True))
            four = {mv for mv, k in cand if k == 3}
            logit = [float(pol[i, mv // 64, mv % 64]) + (float(lp[mv // 64, k]) if mv in four else 0.0) for mv, k in cand]
            # definition: sort by (-logit, index), take E, report in index order
            best = sorted(sorted(range(len(cand)), key=lambda j: (-logit[j], j))[:E])
            want = [cand[j][0] | (cand[j][1] << 11) for j in best]
            ne = int(out["n_edges"][i])
            assert ne == min(E, len(cand)) and out["count"][i] == len(cand)
            assert (out["edge_move"][i, :ne].astype(np.int64) & 0xFFFF).tolist() == want
            before = np.exp(np.array(logit, np.float64) - max(logit))
            before /= before.sum()
            assert np.isclose(out["dropped"][i], 1.0 - before[best].sum(), atol=1e-12)
            assert abs(out["edge_prior"][i, :ne].sum() - 1.0) < 1e-12
            if len(cand) > E:
                assert out["dropped"][i] > 0                    # reference tests/test_search.py:371


# --------------------------------------------------------------------------- #
# What the reference's own Search._expand wrote (tests/golden/reference_vectors_expand.npz, made by
# `python tests/golden/make_golden.py expand`: brokefish/search/torch_impl.py:962-1033 run on the
# eight golden positions and the reference's edge-case positions with formula logits, E = 96 and 16)
# --------------------------------------------------------------------------- #

def _reference_expand_case():
    import os
    import sys
    here = os.path.dirname(os.path.abspath(__file__))
    sys.path.insert(0, os.path.join(here, "golden"))
    import make_golden as mg
    import edge_positions as ep
    g = np.load(os.path.join(here, "golden", "reference_vectors_expand.npz"))
    gb, gc, _ = mg.positions()
    fb, fc = ep.boards_of()
    boards = np.concatenate([gb.numpy().view(np.uint16), fb])
    control = np.concatenate([gc.numpy(), fc])
    pol, pro, val = [t.numpy() for t in mg.expand_logits(boards.shape[0])]
    return g, boards, control, pol, pro, val, ep


def _well_formed(boards):
    """No two live slots on one square (three of the eight hand-built golden positions keep a
    bishop under the castled rook: fine for the evaluator they were made for, which reads slots,
    but not a chess position, and generators may differ on them)."""
    ok = np.ones(boards.shape[0], bool)
    for i, b in enumerate(boards):
        sq = [int(w) & 63 for w in b if not int(w) & 0x800]
        ok[i] = len(sq) == len(set(sq))
    return ok


def test_position_words_and_legal_moves_equal_the_references_on_its_edge_cases():
    # the reference's own from_fen and movegen (brokefish/env/torch_impl.py:781, :254) on the
    # same FEN strings and on the eight golden positions
    g, boards, control, *_ , ep = _reference_expand_case()
    n_fen = len(ep.ALL)
    assert (boards[-n_fen:].view(np.int16) == g["fen_boards"]).all() and (control[-n_fen:] == g["fen_control"]).all()
    mask, check = positions.movegen(boards, control)
    ok = _well_formed(boards)
    assert ok.sum() == boards.shape[0] - 3 and ok[-n_fen:].all()
    assert (mask.view(np.int64)[ok] == g["mask"][ok]).all()
    assert ((check != 0)[ok] == g["in_check"][ok]).all()


@pytest.mark.parametrize("E", [96, 16])
def test_checker_reproduces_the_references_expand(E):
    g, boards, control, pol, pro, val, ep = _reference_expand_case()
    out = ox.expand(pol, pro, val, g["mask"], boards, control, E)
    assert (out["count"] == g[f"count_E{E}"]).all() and (out["n_edges"] == g[f"n_edges_E{E}"]).all()
    assert out["count"].max() == 218 and (out["count"] > E).sum() >= (1 if E == 96 else 20)
    assert (out["edge_move"] == g[f"edge_move_E{E}"]).all()          # no near-tie at the cut in these vectors
    assert out["margin"].min() > 1e-4
    ref = g[f"edge_prior_E{E}"].astype(np.float64)                   # fp16 of the reference's fp32 softmax
    assert (np.abs(out["edge_prior"] - ref) <= 5e-4 * out["edge_prior"] + 6e-8).all()
    assert np.abs(out["dropped"] - g[f"dropped_E{E}"]).max() < 2e-6
    assert np.abs(out["node_value"] - g[f"node_value_E{E}"].astype(np.float64)).max() <= 2.5e-4


# --------------------------------------------------------------------------- #
# GPU
# --------------------------------------------------------------------------- #

def _check(got, want, n, E, exact_rows=None):
    ne = got["n_edges"].cpu().numpy()
    assert (ne == want["n_edges"]).all() and (got["count"].cpu().numpy() == want["count"]).all()
    em, ep = got["edge_move"].cpu().numpy(), got["edge_prior"].float().cpu().numpy().astype(np.float64)
    rows = range(n) if exact_rows is None else exact_rows
    for i in rows:
        assert (em[i] == want["edge_move"][i]).all(), i
        w = want["edge_prior"][i]
        assert (np.abs(ep[i] - w) <= 6e-4 * w + 6e-8).all(), i
    assert np.allclose(got["dropped"].cpu().numpy()[list(rows)], want["dropped"][list(rows)], atol=2e-6)
    nv = got["node_value"].float().cpu().numpy()
    assert np.abs(nv - want["node_value"]).max() <= 2.5e-4      # fp16 in [0,1]


@pytest.mark.gpu
@pytest.mark.parametrize("fp32", [True, False])
def test_kernel_against_the_checker_on_random_playouts(fp32):
    from brokefish_amd.hip_impl import expand_edges
    n = 384
    b, c, r, m = positions.random_positions(n, plies=160, seed=5, stamp_queen=True)
    pol, pro, val = _logits(n, 7)
    tp, tq = torch.from_numpy(pol), torch.from_numpy(pro)
    if not fp32:
        tp, tq = tp.half(), tq.half()
    got = expand_edges(tp.cuda(), tq.cuda(), torch.from_numpy(val).cuda(), m.cuda(), b.cuda(), c.cuda(), 96)
    want = ox.expand(tp.float().numpy(), tq.float().numpy(), val, m.numpy(), b.numpy(), c.numpy(), 96)
    assert want["count"].max() > 40 and (want["count"] != want["n_edges"]).sum() == 0
    _check(got, want, n, 96)
    # nothing beyond n_edges
    ne = got["n_edges"].long()
    beyond = torch.arange(96, device="cuda")[None, :] >= ne[:, None]
    assert (got["edge_prior"][beyond] == 0).all() and (got["edge_move"][beyond] == 0).all()
    assert ((got["edge_prior"].float().sum(1) - 1).abs()[ne > 0] < 2e-3).all()


@pytest.mark.gpu
def test_kernel_truncation_ties_inactive_rows_and_dense_masks():
    from brokefish_amd.hip_impl import expand_edges
    n = 256
    b, c, r, m = positions.random_positions(n, plies=100, seed=9, stamp_queen=True)
    pol, pro, val = _logits(n, 11)
    dev = lambda *a: [torch.from_numpy(x).cuda() if isinstance(x, np.ndarray) else x.cuda() for x in a]
    for E in (1, 5, 16):
        got = expand_edges(*dev(pol, pro, val), m.cuda(), b.cuda(), c.cuda(), E)
        want = ox.expand(pol, pro, val, m.numpy(), b.numpy(), c.numpy(), E)
        assert (want["count"] > E).sum() > n // 2
        safe = [i for i in range(n) if want["margin"][i] > 1e-5]
        assert len(safe) > 0.95 * n
        _check(got, want, n, E, exact_rows=safe)
        assert (got["n_edges"].cpu().numpy() == np.minimum(want["count"], E)).all()
    # exact ties: all-equal logits keep the first E candidates in canonical order, uniformly
    zero = np.zeros_like(pol)
    zpro = np.zeros_like(pro)
    got = expand_edges(*dev(zero, zpro, val), m.cuda(), b.cuda(), c.cuda(), 6)
    want = ox.expand(zero, zpro, val, m.numpy(), b.numpy(), c.numpy(), 6)
    assert (got["edge_move"].cpu().numpy() == want["edge_move"]).all()
    assert (got["n_edges"].cpu().numpy() == want["n_edges"]).all()
    # inactive rows keep what the buffers held
    act = torch.arange(n) % 3 != 0
    out = expand_edges(*dev(pol, pro, val), m.cuda(), b.cuda(), c.cuda(), 16)
    for t in out.values():
        t.fill_(7)
    expand_edges(*dev(pol, pro, val), m.cuda(), b.cuda(), c.cuda(), 16, active=act.cuda(), out=out)
    assert (out["n_edges"][~act.cuda()] == 7).all() and (out["edge_move"][~act.cuda()] == 7).all()
    ref = expand_edges(*dev(pol, pro, val), m.cuda(), b.cuda(), c.cuda(), 16)
    assert torch.equal(out["edge_move"][act.cuda()], ref["edge_move"][act.cuda()])
    # masks denser than any chess position (every bit set: 2048 moves, pawns fan out on the last
    # rank) go through the same code: no candidate buffer to overflow
    full = torch.full((4, 32), -1, dtype=torch.int64)
    got = expand_edges(*dev(pol[:4], pro[:4], val[:4]), full.cuda(), b[:4].cuda(), c[:4].cuda(), 96)
    want = ox.expand(pol[:4], pro[:4], val[:4], full.numpy(), b[:4].numpy(), c[:4].numpy(), 96)
    assert (want["count"] >= 2048).all()
    safe = [i for i in range(4) if want["margin"][i] > 1e-5]
    _check(got, want, 4, 96, exact_rows=safe)
    # candidate counts around the kernel's lane-parallel layout: 65..256 candidates are two to four
    # per lane, 257 and more take the pass-per-walk path; with and without truncation, and with
    # all-equal logits (ties cut in canonical order across the lanes' second to fourth candidates)
    rng = np.random.default_rng(3)
    counts = [63, 64, 65, 100, 128, 129, 200, 255, 256, 257, 300, 500]
    dense = np.zeros((len(counts), 32), dtype=np.uint64)
    for i, k in enumerate(counts):
        for bit in rng.choice(2048, size=k, replace=False):
            dense[i, bit // 64] |= np.uint64(1) << np.uint64(bit % 64)
    dm = torch.from_numpy(dense.view(np.int64))
    k = len(counts)
    for E in (96, 255, 7):
        got = expand_edges(*dev(pol[:k], pro[:k], val[:k]), dm.cuda(), b[:k].cuda(), c[:k].cuda(), E)
        want = ox.expand(pol[:k], pro[:k], val[:k], dm.numpy(), b[:k].numpy(), c[:k].numpy(), E)
        assert (want["count"] >= np.array(counts)).all()          # promotions only add
        safe = [i for i in range(k) if want["margin"][i] > 1e-5]
        assert len(safe) >= k - 1
        _check(got, want, k, E, exact_rows=safe)
        tie = expand_edges(*dev(zero[:k], zpro[:k], val[:k]), dm.cuda(), b[:k].cuda(), c[:k].cuda(), E)
        wtie = ox.expand(zero[:k], zpro[:k], val[:k], dm.numpy(), b[:k].numpy(), c[:k].numpy(), E)
        assert (tie["edge_move"].cpu().numpy() == wtie["edge_move"]).all()
        assert (tie["n_edges"].cpu().numpy() == wtie["n_edges"]).all()
    # no legal move: zero edges, zero priors
    none = torch.zeros((4, 32), dtype=torch.int64)
    got = expand_edges(*dev(pol[:4], pro[:4], val[:4]), none.cuda(), b[:4].cuda(), c[:4].cuda(), 96)
    assert (got["n_edges"] == 0).all() and (got["edge_prior"] == 0).all()


@pytest.mark.gpu
def test_forward_expand_runs_the_evaluator_and_the_expansion_back_to_back():
    from brokefish_amd import encoder_impl
    from brokefish_amd.hip_impl import expand_edges
    from brokefish_amd.net import BrokefishNet
    torch.manual_seed(0)
    net = BrokefishNet().eval().randomise_layers_(seed=4)
    model = encoder_impl("hip")(net, int8=True)
    n = 300
    b, c, r, m = positions.random_positions(n, plies=120, seed=13)
    bd, cd, rd, md = b.cuda(), c.cuda(), r.cuda(), m.cuda()
    got = model.forward_expand(bd, cd, rd, md, 96)
    p, q, v = model.forward_full(bd, cd, rd)
    again = expand_edges(p, q, v, md, bd, cd, 96)
    for k in got:
        assert torch.equal(got[k], again[k]), k
    want = ox.expand(p.float().cpu().numpy(), q.float().cpu().numpy(), v.cpu().numpy(), m.numpy(), b.numpy(), c.numpy(), 96)
    _check(got, want, n, 96)
    # masked logits (illegal entries -inf) give the same edges: only legal entries are read
    pm = model.forward_full(bd, cd, rd, md)[0]
    masked = expand_edges(pm, model.promo_out, model.value_out, md, bd, cd, 96)
    assert torch.equal(masked["edge_move"], got["edge_move"]) and torch.equal(masked["edge_prior"], got["edge_prior"])
    with pytest.raises(ValueError):
        expand_edges(p, q.float(), v, md, bd, cd, 96)
    with pytest.raises(ValueError):
        expand_edges(p, q, v, md, bd, cd, 300)


@pytest.mark.gpu
@pytest.mark.parametrize("E", [96, 16])
def test_kernel_reproduces_the_references_expand(E):
    from brokefish_amd.hip_impl import expand_edges
    g, boards, control, pol, pro, val, ep = _reference_expand_case()
    dev = lambda x: torch.from_numpy(np.ascontiguousarray(x)).cuda()
    got = expand_edges(dev(pol), dev(pro), dev(val), dev(g["mask"]), dev(boards.view(np.int16)), dev(control), E)
    assert (got["count"].cpu().numpy() == g[f"count_E{E}"]).all() and (got["n_edges"].cpu().numpy() == g[f"n_edges_E{E}"]).all()
    assert (got["edge_move"].cpu().numpy() == g[f"edge_move_E{E}"]).all()
    ref = g[f"edge_prior_E{E}"].astype(np.float64)
    ep16 = got["edge_prior"].float().cpu().numpy().astype(np.float64)
    assert (np.abs(ep16 - ref) <= 1.2e-3 * ref + 1.2e-7).all()         # both sides are fp16 roundings: one ulp apart at most
    assert np.abs(got["dropped"].cpu().numpy() - g[f"dropped_E{E}"]).max() < 2e-6
    assert np.abs(got["node_value"].float().cpu().numpy() - g[f"node_value_E{E}"].astype(np.float32)).max() <= 5e-4
    # and the device's own move generation gives the reference's masks on these positions
    from brokefish_amd.hip_impl import movegen
    m, chk = movegen(dev(boards.view(np.int16)), dev(control))
    ok = _well_formed(boards)
    assert (m.cpu().numpy()[ok] == g["mask"][ok]).all() and (chk.cpu().numpy()[ok] == g["in_check"][ok]).all()
