"""The reference's edge-case positions (tests/edge_positions.py: reference
brokefish/nn/validate.py:81-87 and scripts/dump_cuda_testset.py:87-127) through the whole device
chain: FEN -> position words -> device move generation -> evaluator (every int8 kernel, and
e4m3) -> edge expansion, against the CPU generator, the C checker and the expansion's checker,
and against what the rules of chess fix for them (218 legal moves and a truncated edge list on
the max-mobility position, all-zero masks and zero edges on mate and stalemate, no castling out
of check, the pinned en-passant capture absent, four mask words of 2**62 on the position whose
words sum to 2**64).  The CPU twin of the rules part is in tests/test_positions.py.
"""
import numpy as np
import pytest
import torch

import edge_positions as ep
from brokefish_amd import encoder_impl, positions
from brokefish_amd.net import BrokefishNet
from oracle import c_oracle, emulated, expand as ox
from test_positions import check_edge_position_facts

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def edge():
    boards, control = ep.boards_of()
    n = boards.shape[0]
    rep = (np.arange(n) % 3).astype(np.uint8)
    bt = torch.from_numpy(boards.view(np.int16)).cuda()
    ct = torch.from_numpy(control).cuda()
    rt = torch.from_numpy(rep).cuda()
    torch.manual_seed(0)
    net = BrokefishNet().eval().randomise_layers_(seed=17)
    sd = {k: v.detach() for k, v in net.state_dict().items()}
    return dict(boards=boards, control=control, rep=rep, bt=bt, ct=ct, rt=rt, net=net, sd=sd,
                by={name: i for i, name in enumerate(ep.NAMES)})


def _device_masks(e):
    from brokefish_amd.hip_impl import movegen
    m, chk = movegen(e["bt"], e["ct"])
    return m, chk


def test_device_move_generation_equals_the_cpu_generator_and_the_rules(edge):
    m, chk = _device_masks(edge)
    want_m, want_c = positions.movegen(edge["boards"], edge["control"])
    got = m.cpu().numpy().view(np.uint64)
    assert (got == want_m).all() and (chk.cpu().numpy() == (want_c != 0)).all()
    check_edge_position_facts(ep, edge["boards"], edge["control"], got, chk.cpu().numpy(), edge["by"])


@pytest.mark.parametrize("kernel", ["twin", "duo", "octo", "board", "quad"])
def test_int8_evaluator_bit_exact_on_the_edge_positions(edge, kernel):
    m, _ = _device_masks(edge)
    model = encoder_impl("hip")(edge["net"], int8=True, out_dtype=torch.float32, kernel=kernel)
    p, q, v, best = [t.clone() for t in model.forward_masked(edge["bt"], edge["ct"], edge["rt"], m)]
    want = c_oracle.COracle(edge["sd"]).forward(edge["boards"], edge["control"], edge["rep"],
                                                mask=m.cpu().numpy().view(np.uint64))
    for got, key in ((p, "policy"), (q, "promo"), (v, "value")):
        assert (got.cpu().numpy().view(np.int32) == want[key].view(np.int32)).all(), key
    assert (best.cpu().numpy() == want["best"]).all()
    by = edge["by"]
    # no legal move: every entry -inf and no best move; otherwise the best move is a legal one
    for name in ("check-by-queen", "stalemate-queen"):
        assert torch.isinf(p[by[name]]).all() and best[by[name]] == -1
    legal = torch.isfinite(p)
    assert int(legal[by["max-mobility"]].sum()) == 218
    for i in range(p.shape[0]):
        if legal[i].any():
            assert legal[i].flatten()[int(best[i])]
    # raw logits (no mask) are finite everywhere, dead slots and nine queens included
    raw = model.forward_full(edge["bt"], edge["ct"], edge["rt"])
    assert all(torch.isfinite(t).all() for t in raw) and (raw[2].abs() <= 1).all()


def test_e4m3_kernels_agree_and_follow_the_emulation_on_the_edge_positions(edge):
    m, _ = _device_masks(edge)
    outs = {}
    for kernel in ("twin", "duo", "octo", "quad"):
        model = encoder_impl("hip")(edge["net"], fp8=True, out_dtype=torch.float32, kernel=kernel)
        outs[kernel] = [t.clone() for t in model.forward_masked(edge["bt"], edge["ct"], edge["rt"], m)]
    for kernel in ("duo", "octo", "quad"):
        for x, y in zip(outs[kernel], outs["twin"]):
            assert torch.equal(x, y), kernel
    raw = encoder_impl("hip")(edge["net"], fp8=True, out_dtype=torch.float32).forward_full(edge["bt"], edge["ct"], edge["rt"])
    with torch.no_grad():
        emu = emulated.forward(edge["sd"], torch.from_numpy(edge["boards"].view(np.int16)), torch.from_numpy(edge["control"]),
                               torch.from_numpy(edge["rep"]), mode="e4m3")
    d = (raw[0].cpu() - emu[0]).abs().flatten(1).max(1).values
    # free-running e4m3: a board either matches the emulation to 2e-2 or carries a flipped tie
    # (tests/test_parity_fp8_gpu.py proves the ties); most boards match
    assert (d < 2e-2).float().mean() > 0.5 and d.max() < 0.3, d


def test_movegen_evaluator_expansion_chain_on_the_edge_positions(edge):
    model = encoder_impl("hip")(edge["net"], int8=True)
    got = model.forward_expand(edge["bt"], edge["ct"], edge["rt"], max_edges=96)
    m = got["mask"].cpu().numpy()
    want = ox.expand(model.policy_out.float().cpu().numpy(), model.promo_out.float().cpu().numpy(),
                     model.value_out.cpu().numpy(), m, edge["boards"].view(np.int16), edge["control"], 96)
    by = edge["by"]
    ne, cnt = got["n_edges"].cpu().numpy(), got["count"].cpu().numpy()
    assert (cnt == want["count"]).all() and (ne == want["n_edges"]).all()
    # 218 candidates against 96 edge slots: the list is truncated and the dropped mass reported
    i = by["max-mobility"]
    assert cnt[i] == 218 and ne[i] == 96 and got["dropped"][i] > 0
    assert abs(float(got["edge_prior"][i].float().sum()) - 1.0) < 2e-3
    for name in ("check-by-queen", "stalemate-queen"):
        assert cnt[by[name]] == 0 and ne[by[name]] == 0 and (got["edge_prior"][by[name]] == 0).all()
    # every pawn move onto the last rank fans out into four edges: 2 king moves + ... on the race
    j = by["promotion-by-push"]
    assert cnt[j] == int(sum(bin(int(w) & 0xFFFFFFFFFFFFFFFF).count("1") for w in m[j])) + 3
    em, ep_ = got["edge_move"].cpu().numpy(), got["edge_prior"].float().cpu().numpy().astype(np.float64)
    for r in range(len(ep.ALL)):
        if want["margin"][r] > 1e-5:                    # the kept set is decided by more than rounding
            assert (em[r] == want["edge_move"][r]).all(), ep.NAMES[r]
            w = want["edge_prior"][r]
            assert (np.abs(ep_[r] - w) <= 6e-4 * w + 6e-8).all(), ep.NAMES[r]
