"""Parity of the one-position-per-workgroup kernels (one and two workgroups per compute unit),
through the C-ABI.

Same bar as tests/test_parity_gpu.py: operand bytes, int32 accumulators, residual stream, logits,
value and masked argmax bit-identical to the C checker.  For the 256-wide network the kernels
must also return exactly what the four-positions-per-workgroup kernel returns (the library picks
among them by batch size, and a position's result may not depend on the batch it is in); for the
512-wide, 16-head, 16-layer network (two 256-deep k-chunks per matmul of the width, eight for the
second feed-forward matmul, summed in float64) the one-workgroup-per-compute-unit form is the
only kernel.
"""
import numpy as np
import pytest
import torch

from brokefish_amd import encoder_impl, positions
from brokefish_amd.net import BrokefishNet
from oracle import c_oracle

pytestmark = pytest.mark.gpu

TAPS = ["embed", "qa_qkv", "acc_qkv", "qa_out", "acc_out", "qa_ff1", "acc_ff1", "qa_ff2", "acc_ff2", "resid", "normed"]


def _make(d, heads, layers, nv=1, seed=0):
    torch.manual_seed(seed)
    net = BrokefishNet(d_model=d, n_heads=heads, d_ff=4 * d, n_layers=layers, n_value=nv).eval()
    net.randomise_layers_(seed=seed + 3)
    sd = {k: v.detach() for k, v in net.state_dict().items()}
    return net, sd


@pytest.fixture(scope="module")
def base():
    net, sd = _make(256, 8, 8)
    return (net, sd, {k: encoder_impl("hip")(net, int8=True, out_dtype=torch.float32, kernel=k) for k in ("board", "twin", "octo", "duo")},
            encoder_impl("hip")(net, int8=True, out_dtype=torch.float32, kernel="quad"), c_oracle.COracle(sd))


@pytest.fixture(scope="module")
def stress():
    net, sd = _make(512, 16, 16)
    return net, sd, {k: encoder_impl("hip")(net, int8=True, out_dtype=torch.float32, kernel=k) for k in ("auto", "octo", "board")}, c_oracle.COracle(sd)


def _dev(*ts):
    return [t.cuda() for t in ts]


def _bits_equal(a: torch.Tensor, b: np.ndarray) -> bool:
    a = a.cpu().numpy()
    if a.dtype == np.uint8:
        b = b.view(np.uint8)
    return a.shape == b.shape and bool((a.view(np.int32 if a.dtype == np.float32 else a.dtype)
                                        == b.view(np.int32 if b.dtype == np.float32 else b.dtype)).all())


@pytest.mark.parametrize("kernel", ["board", "twin", "octo", "duo"])
def test_base_network_bit_exact_against_the_c_checker_with_every_tap(base, kernel):
    net, sd, boards, quad, co = base
    board = boards[kernel]
    b, c, r, m = positions.random_positions(48, plies=120, seed=11, stamp_queen=True)
    got = board.forward_taps(*_dev(b, c, r), mask=m.cuda())
    want = co.forward(b.numpy(), c.numpy(), r.numpy(), mask=m.numpy(), taps=True)
    for k in TAPS + ["policy", "promo", "value", "best"]:
        assert _bits_equal(got[k], want[k]), k


@pytest.mark.parametrize("kernel", ["board", "twin", "octo", "duo"])
def test_heads_alone_and_a_layer_range_from_a_given_residual_stream(base, kernel):
    # a run of no layers starts the weight stream at the head blocks (no layer block is fetched,
    # none exists to fetch past the last layer); a run of some layers continues into them
    net, sd, boards, quad, co = base
    model = boards[kernel]
    b, c, r, m = positions.random_positions(37, plies=90, seed=29)
    bd, cd, rd, md = _dev(b, c, r, m)
    want = co.forward(b.numpy(), c.numpy(), r.numpy(), mask=m.numpy(), taps=True)
    heads = model.forward_taps(bd, cd, rd, mask=md, x_in=torch.from_numpy(want["resid"][:, 7]).cuda(),
                               layer_begin=8, layer_end=8, want=["normed"])
    for k in ("normed", "policy", "promo", "value", "best"):
        assert _bits_equal(heads[k], want[k]), k
    tail = model.forward_taps(bd, cd, rd, mask=md, x_in=torch.from_numpy(want["resid"][:, 4]).cuda(),
                              layer_begin=5, layer_end=8, want=["resid"])
    assert _bits_equal(tail["resid"][:, -1], want["resid"][:, 7])
    for k in ("policy", "promo", "value", "best"):
        assert _bits_equal(tail[k], want[k]), k


@pytest.mark.parametrize("kernel", ["board", "twin", "octo", "duo"])
@pytest.mark.parametrize("nv", [1, 3])
def test_the_kernels_return_the_same_bits(base, nv, kernel):
    if nv == 1:
        net, sd, boards, quad, co = base
        board = boards[kernel]
    else:
        net, sd = _make(256, 8, 8, nv=3, seed=5)
        board = encoder_impl("hip")(net, int8=True, out_dtype=torch.float32, kernel=kernel)
        quad = encoder_impl("hip")(net, int8=True, out_dtype=torch.float32, kernel="quad")
    b, c, r, m = positions.random_positions(301, plies=120, seed=21)           # odd on purpose
    bd, cd, rd, md = _dev(b, c, r, m)
    pq, qq, vq = [t.clone() for t in quad.forward_full(bd, cd, rd, md)]
    bestq = quad.best_move.clone()
    pb, qb, vb = board.forward_full(bd, cd, rd, md)
    assert torch.equal(pb, pq) and torch.equal(qb, qq) and torch.equal(vb, vq) and torch.equal(board.best_move, bestq)
    raw_q = quad.forward_full(bd, cd, rd)[0].clone()
    assert torch.equal(board.forward_full(bd, cd, rd)[0], raw_q) and torch.isfinite(raw_q).all()
    one = board.forward_full(bd[7:8], cd[7:8], rd[7:8])[0]
    assert torch.equal(one, raw_q[7:8])
    half_b = encoder_impl("hip")(net, int8=True, kernel=kernel).forward_full(bd, cd, rd)[0]
    assert half_b.dtype is torch.float16 and torch.equal(half_b, raw_q.half())
    # teacher-forced single layers and the heads alone agree as well
    x = torch.randn(301, 32, 256, generator=torch.Generator().manual_seed(3)).cuda()
    for l0, l1 in ((2, 3), (5, 8), (8, 8)):
        tb = board.forward_taps(bd, cd, rd, x_in=x, layer_begin=l0, layer_end=l1, want=["resid", "acc_ff2", "normed"])
        tq = quad.forward_taps(bd, cd, rd, x_in=x, layer_begin=l0, layer_end=l1, want=["resid", "acc_ff2", "normed"])
        for k in ("resid", "acc_ff2", "normed", "policy", "value"):
            assert torch.equal(tb[k], tq[k]), (l0, l1, k)


def test_automatic_choice_switches_kernel_by_batch_size_without_changing_results(base):
    net, sd, boards, quad, co = base
    auto = encoder_impl("hip")(net, int8=True, out_dtype=torch.float32)
    cut = int(auto._lib.bf_board_max_n())
    assert auto.kernel_choice(1) == "octo" and auto.kernel_choice(cut) == "octo"
    assert auto.kernel_choice(cut + 1) == "duo" and auto.kernel_choice(4096) == "duo"
    assert "by batch size" in auto.label
    b, c, r, m = positions.random_positions(cut + 4, plies=120, seed=22)
    bd, cd, rd, md = _dev(b, c, r, m)
    big = [t.clone() for t in auto.forward_masked(bd, cd, rd, md)]                        # two positions per workgroup
    small = auto.forward_masked(bd[:cut], cd[:cut], rd[:cut], md[:cut])                  # one
    for x, y in zip(big, small):
        assert torch.equal(x[:cut], y)
    ref = quad.forward_masked(bd, cd, rd, md)
    for x, y in zip(big, ref):
        assert torch.equal(x, y)
    fp8 = encoder_impl("hip")(net, fp8=True)                                             # the same rule in e4m3
    assert fp8.kernel_choice(1) == "octo" and fp8.kernel_choice(cut) == "octo" and fp8.kernel_choice(4096) == "twin"


@pytest.mark.parametrize("fp16_out", [False, True])
def test_a_small_last_round_goes_to_the_one_position_form_without_changing_results(base, fp16_out):
    # above 512 positions the automatic choice launches the two-position kernel on the whole rounds
    # of 512 and, when at most 256 positions remain, the one-position form on those: every output
    # row, the skipped rows of an `active` launch and the masked argmax must be what one launch of
    # the two-position kernel writes
    net, sd, boards, quad, co = base
    kw = dict(int8=True) if fp16_out else dict(int8=True, out_dtype=torch.float32)
    auto, duo = encoder_impl("hip")(net, **kw), encoder_impl("hip")(net, kernel="duo", **kw)
    for n in (513, 640, 768, 769, 1100, 1281):           # tails of 1, 128, 256 (split); 257, 76 + 2 rounds, 257 (not / split / not)
        b, c, r, m = positions.random_positions(n, plies=120, seed=200 + n)
        bd, cd, rd, md = _dev(b, c, r, m)
        act = (torch.arange(n, device="cuda") % 5 != 0)
        want = [t.clone() for t in duo.forward_masked(bd, cd, rd, md)]
        got = [t.clone() for t in auto.forward_masked(bd, cd, rd, md)]
        for x, y in zip(got, want):
            assert torch.equal(x, y), n
        for mod in (auto, duo):
            for t in (mod.policy_out, mod.promo_out, mod.value_out):
                t.fill_(3.0)
        pa = [t.clone() for t in auto.forward_full(bd, cd, rd, active=act)]
        pd = [t.clone() for t in duo.forward_full(bd, cd, rd, active=act)]
        for x, y in zip(pa, pd):
            assert torch.equal(x, y) and (x[~act] == 3.0).all(), n
    if not fp16_out:
        idx = np.arange(500, 640, 7)                     # rows either side of the split, against the C checker
        b, c, r, m = positions.random_positions(640, plies=120, seed=840)
        got = auto.forward_masked(*_dev(b, c, r, m))
        ref = co.forward(b.numpy()[idx], c.numpy()[idx], r.numpy()[idx], mask=m.numpy()[idx])
        assert _bits_equal(got[0][idx], ref["policy"]) and _bits_equal(got[2][idx], ref["value"])
        assert (got[3].cpu().numpy()[idx] == ref["best"]).all()


def test_e4m3_on_the_throughput_kernel_equals_the_four_per_workgroup_kernel(base):
    # same quantiser, same MFMA sequence per accumulator, same reduction orders: the same bits
    # (the e4m3 parity statement against the emulation is in tests/test_parity_fp8_gpu.py)
    net, sd, boards, quad, co = base
    twin = encoder_impl("hip")(net, fp8=True, out_dtype=torch.float32, kernel="twin")
    ref = encoder_impl("hip")(net, fp8=True, out_dtype=torch.float32, kernel="quad")
    b, c, r, m = positions.random_positions(333, plies=120, seed=23)
    bd, cd, rd, md = _dev(b, c, r, m)
    got = [t.clone() for t in twin.forward_masked(bd, cd, rd, md)]
    want = ref.forward_masked(bd, cd, rd, md)
    for x, y in zip(got, want):
        assert torch.equal(x, y)
    assert torch.isfinite(twin.forward_full(bd, cd, rd)[0]).all()
    tt = twin.forward_taps(bd[:40], cd[:40], rd[:40])
    tq = ref.forward_taps(bd[:40], cd[:40], rd[:40])
    for k in TAPS:
        assert tt[k].dtype == tq[k].dtype and torch.equal(tt[k].view(torch.uint8), tq[k].view(torch.uint8)), k
    int8 = boards["twin"].forward_full(bd, cd, rd)[0]
    assert not torch.equal(int8, twin.forward_full(bd, cd, rd)[0])
    # the other one-position kernels and the two-position kernel carry the format too, and AUTO
    # switches by size
    for kernel in ("board", "octo", "duo"):
        other = encoder_impl("hip")(net, fp8=True, out_dtype=torch.float32, kernel=kernel)
        for x, y in zip(other.forward_masked(bd, cd, rd, md), got):
            assert torch.equal(x, y), kernel
        tb = other.forward_taps(bd[:40], cd[:40], rd[:40])
        for k in TAPS:
            assert torch.equal(tb[k].view(torch.uint8), tq[k].view(torch.uint8)), (kernel, k)
    auto = encoder_impl("hip")(net, fp8=True, out_dtype=torch.float32)
    assert auto.kernel_choice(256) == "octo" and auto.kernel_choice(257) == "twin"
    small = [t.clone() for t in auto.forward_masked(bd[:200], cd[:200], rd[:200], md[:200])]
    for x, y in zip(small, got):
        assert torch.equal(x, y[:200])


@pytest.mark.parametrize("kernel", ["board", "twin", "octo", "duo", "quad"])
def test_skipped_positions_keep_their_output_rows(base, kernel):
    # the search's flat leaf staging: only flagged leaves are evaluated (reference
    # brokefish/search/cuda_impl.py:137-145), the others cost nothing and change nothing
    net, sd, boards, quad, co = base
    model = quad if kernel == "quad" else boards[kernel]
    b, c, r, m = positions.random_positions(203, plies=120, seed=24)
    bd, cd, rd, md = _dev(b, c, r, m)
    full = [t.clone() for t in model.forward_masked(bd, cd, rd, md)]
    act = (torch.arange(203) % 3 != 1).cuda()
    for t in (model.policy_out, model.promo_out, model.value_out, model.best_out):
        t.fill_(5)
    p, q, v = model.forward_full(bd, cd, rd, md, active=act)
    for got, want in zip((p, q, v, model.best_out), full):
        assert torch.equal(got[act], want[act])
        assert (got[~act] == 5).all()
    p2 = model.forward_full(bd, cd, rd, md, active=act.to(torch.uint8))[0]
    assert torch.equal(p2[act], full[0][act])
    with pytest.raises(ValueError):
        model.forward_full(bd, cd, rd, md, active=act[:10])


@pytest.mark.parametrize("kernel", ["twin", "octo", "duo", "board", "quad"])
def test_compacted_leaf_list_with_a_device_side_count_equals_the_flag_route(base, kernel):
    # the "compacted list plus a count" of the reference's design retrospective
    # (docs/journal/2026-08-09-kernel-design-retrospective.md:140-154) over its flat leaf staging
    # (brokefish/search/cuda_impl.py:137-145): same rows written, same bits, other rows untouched
    from brokefish_amd import hip_impl
    net, sd, boards, quad, co = base
    model = quad if kernel == "quad" else boards[kernel]
    b, c, r, m = positions.random_positions(301, plies=120, seed=31)
    bd, cd, rd, md = _dev(b, c, r, m)
    g = torch.Generator().manual_seed(4)
    for flags in (torch.rand(301, generator=g) < 0.4, torch.zeros(301, dtype=torch.bool), torch.ones(301, dtype=torch.bool),
                  torch.arange(301) == 300):
        fd = flags.cuda()
        index, count = hip_impl.compact_leaves(fd)
        k = int(flags.sum())
        assert int(count.item()) == k and torch.equal(index[:k].cpu().long(), flags.nonzero()[:, 0])
        outs = []
        for route in ("flags", "list"):
            model.forward_full(bd, cd, rd, md)                      # size the buffers, then mark them
            for t in (model.policy_out, model.promo_out, model.value_out):
                t.fill_(7.0)
            model.best_out.fill_(-7)
            kw = {"active": fd} if route == "flags" else {"leaves": (index, count)}
            p, q, v = model.forward_full(bd, cd, rd, md, **kw)
            outs.append([t.clone() for t in (p, q, v, model.best_out)])
            assert (v[~fd] == 7.0).all() and (model.best_out[~fd] == -7).all()
        for x, y in zip(*outs):
            assert torch.equal(x, y)
        if k:
            full = model.forward_full(bd, cd, rd, md)
            assert torch.equal(outs[1][0][fd], full[0][fd]) and torch.equal(outs[1][2][fd], full[2][fd])
        # the expansion takes the same list
        pol, pro, val = [t.clone() for t in model.forward_full(bd, cd, rd)]
        e1 = {k_: t.clone() for k_, t in hip_impl.expand_edges(pol, pro, val, md, bd, cd, active=fd).items()}
        e2 = hip_impl.expand_edges(pol, pro, val, md, bd, cd, leaves=(index, count))
        for k_ in e1:
            assert torch.equal(e1[k_], e2[k_]), k_
    with pytest.raises(ValueError):
        model.forward_full(bd, cd, rd, active=fd, leaves=(index, count))
    # the chain movegen -> compaction -> evaluator -> expansion stays on the device
    edges = model.forward_expand(bd, cd, rd, leaves=hip_impl.compact_leaves(torch.arange(301, device="cuda") % 2 == 0))
    assert (edges["n_edges"][1::2] == 0).all() and (edges["n_edges"][0::2] > 0).any()


@pytest.mark.parametrize("n", [5000, 65536])
def test_compaction_of_more_flags_than_one_pass_holds(n):
    # the compaction kernel walks the flags 1024 at a time, carrying the count from pass to pass
    from brokefish_amd import hip_impl
    g = torch.Generator().manual_seed(n)
    for flags in (torch.rand(n, generator=g) < 0.37, torch.ones(n, dtype=torch.bool), torch.arange(n) == n - 1,
                  torch.arange(n) % 1024 == 1023, torch.zeros(n, dtype=torch.bool)):
        index, count = hip_impl.compact_leaves(flags.cuda())
        k = int(flags.sum())
        assert int(count.item()) == k
        assert torch.equal(index[:k].cpu().long(), flags.nonzero()[:, 0])
    # uint8 flags with values other than 1 count as set; a reused output pair keeps its tail
    f8 = (torch.arange(n) % 5 == 0).to(torch.uint8) * 200
    out = hip_impl.compact_leaves(torch.ones(n, dtype=torch.bool).cuda())
    index, count = hip_impl.compact_leaves(f8.cuda(), out=out)
    k = int((f8 != 0).sum())
    assert int(count.item()) == k and torch.equal(index[:k].cpu().long(), f8.nonzero()[:, 0])
    assert torch.equal(index[k:].cpu().long(), torch.arange(k, n))


@pytest.mark.parametrize("kernel", ["twin", "octo", "duo", "board", "quad"])
def test_a_leaf_list_entry_that_is_no_position_of_the_launch_is_skipped(base, kernel):
    # every kernel treats a malformed entry (negative, or past n) like a slot past the count:
    # nothing is evaluated for it and no row is written
    net, sd, boards, quad, co = base
    model = quad if kernel == "quad" else boards[kernel]
    b, c, r, m = positions.random_positions(37, plies=120, seed=33)
    bd, cd, rd, md = _dev(b, c, r, m)
    full = [t.clone() for t in model.forward_full(bd, cd, rd, md)]
    best = model.best_out.clone()
    index = torch.tensor([5, -1, 36, 37, 1 << 20, 0, 11] + [0] * 30, dtype=torch.int32).cuda()
    count = torch.tensor([7], dtype=torch.int32).cuda()
    for t in (model.policy_out, model.promo_out, model.value_out):
        t.fill_(7.0)
    model.best_out.fill_(-7)
    p, q, v = model.forward_full(bd, cd, rd, md, leaves=(index, count))
    hit = torch.zeros(37, dtype=torch.bool)
    hit[[5, 36, 0, 11]] = True
    hd = hit.cuda()
    assert torch.equal(p[hd], full[0][hd]) and torch.equal(v[hd], full[2][hd]) and torch.equal(model.best_out[hd], best[hd])
    assert (v[~hd] == 7.0).all() and (p[~hd] == 7.0).all() and (model.best_out[~hd] == -7).all()


def test_full_batch_at_4096_on_the_throughput_kernel(base):
    net, sd, boards, quad, co = base
    auto = encoder_impl("hip")(net, int8=True, out_dtype=torch.float32)
    assert auto.kernel_choice(4096) == "duo"
    b, c, r, m = positions.random_positions(4096, plies=120, seed=0)
    bd, cd, rd, md = _dev(b, c, r, m)
    p, q, v, best = [t.clone() for t in auto.forward_masked(bd, cd, rd, md)]
    idx = np.arange(3, 4096, 41)
    want = co.forward(b.numpy()[idx], c.numpy()[idx], r.numpy()[idx], mask=m.numpy()[idx])
    assert _bits_equal(p[idx], want["policy"]) and _bits_equal(q[idx], want["promo"])
    assert _bits_equal(v[idx], want["value"]) and (best.cpu().numpy()[idx] == want["best"]).all()
    ref = quad.forward_masked(bd, cd, rd, md)
    assert torch.equal(p, ref[0]) and torch.equal(q, ref[1]) and torch.equal(v, ref[2]) and torch.equal(best, ref[3])
    again = auto.forward_masked(bd, cd, rd, md)
    assert torch.equal(again[0], p) and torch.equal(again[3], best)                       # deterministic
    legal = ((md[..., None] >> torch.arange(64, device="cuda")) & 1).bool()
    assert torch.isneginf(p[~legal]).all() and torch.isfinite(p[legal]).all() and (v.abs() <= 1).all()


def test_largest_batch_of_the_sweep_is_independent_of_batch_composition(base):
    # 65536 positions (the top of the batch sweep): 2048 distinct positions repeated 32 times in a
    # shuffled order must each come back with the bits the 2048-position launch gave them
    net, sd, boards, quad, co = base
    model = encoder_impl("hip")(net, int8=True)              # fp16 logits, the search's contract
    b, c, r, m = positions.random_positions(2048, plies=120, seed=31)
    small = [t.clone() for t in model.forward_masked(*_dev(b, c, r, m))]
    g = torch.Generator().manual_seed(7)
    order = torch.cat([torch.randperm(2048, generator=g) for _ in range(32)])
    assert model.kernel_choice(65536) == "duo"
    big = model.forward_masked(*_dev(b[order], c[order], r[order], m[order]))
    od = order.cuda()
    for got, want in zip(big, small):
        assert got.shape[0] == 65536 and torch.equal(got, want[od])


@pytest.mark.parametrize("kernel", ["auto", "board"])
def test_stress_network_bit_exact_against_the_c_checker_with_every_tap(stress, kernel):
    net, sd, models, co = stress
    model = models[kernel]
    assert model.kernel_choice(16384) == ("octo" if kernel == "auto" else "board") and model.wstream is None
    assert models["octo"].kernel_choice(1) == "octo"
    b, c, r, m = positions.random_positions(12, plies=120, seed=31, stamp_queen=True)
    got = model.forward_taps(*_dev(b, c, r), mask=m.cuda())
    want = co.forward(b.numpy(), c.numpy(), r.numpy(), mask=m.numpy(), taps=True)
    for k in TAPS + ["policy", "promo", "value", "best"]:
        assert _bits_equal(got[k], want[k]), k
    assert got["acc_qkv"].shape == (12, 16, 2, 32, 1536) and got["acc_ff2"].shape == (12, 16, 8, 32, 512)
    # the accumulators are the exact integer products of the kernel's own operand bytes, per k-chunk
    q, _ = co.qweight("ff2", 9)
    a = got["qa_ff2"][:, 9].cpu().numpy().astype(np.int64)                     # [n,32,2048] unsigned
    acc = np.stack([a[..., 256 * k:256 * k + 256] @ q[:, 256 * k:256 * k + 256].astype(np.int64).T for k in range(8)], 1)
    assert (acc == got["acc_ff2"][:, 9].cpu().numpy()).all()
    q, _ = co.qweight("qkv", 15)
    a = got["qa_qkv"][:, 15].cpu().numpy().astype(np.int64)
    acc = np.stack([a[..., 256 * k:256 * k + 256] @ q[:, 256 * k:256 * k + 256].astype(np.int64).T for k in range(2)], 1)
    assert (acc == got["acc_qkv"][:, 15].cpu().numpy()).all()
    # production launch, fp16 contract, teacher forcing of a layer range and of the heads alone
    bd, cd, rd, md = _dev(b, c, r, m)
    p, q2, v = model.forward_full(bd, cd, rd, md)
    assert torch.equal(p, got["policy"]) and torch.equal(q2, got["promo"]) and torch.equal(v, got["value"])
    assert torch.equal(model.best_move, got["best"])
    half = encoder_impl("hip")(net, int8=True, kernel=kernel).forward_full(bd, cd, rd, md)[0]
    assert half.dtype is torch.float16 and torch.equal(half, p.half())
    x_in = torch.from_numpy(want["resid"][:, 10]).cuda()
    tail = model.forward_taps(bd, cd, rd, mask=md, x_in=x_in, layer_begin=11, layer_end=16, want=["resid"])
    assert _bits_equal(tail["resid"][:, -1], want["resid"][:, 15]) and torch.equal(tail["policy"], got["policy"])
    mid = model.forward_taps(bd, cd, rd, x_in=x_in, layer_begin=11, layer_end=12, want=["resid"])
    assert _bits_equal(mid["resid"][:, 0], want["resid"][:, 11])
    heads = model.forward_taps(bd, cd, rd, mask=md, x_in=torch.from_numpy(want["resid"][:, 15]).cuda(),
                               layer_begin=16, layer_end=16, want=["normed"])
    assert torch.equal(heads["policy"], got["policy"]) and torch.equal(heads["value"], got["value"])
    with pytest.raises(NotImplementedError):
        encoder_impl("hip")(net, fp8=True)
    for k in ("quad", "twin"):
        with pytest.raises(NotImplementedError):
            encoder_impl("hip")(net, int8=True, kernel=k)


def test_stress_network_win_draw_loss_head_and_full_batch_properties():
    # the configuration's batch size, 16384 positions: spot-check against the C checker,
    # size-independent properties on everything
    net, sd = _make(512, 16, 16, nv=3, seed=2)
    model = encoder_impl("hip")(net, int8=True, out_dtype=torch.float32)
    assert model.kernel_choice(16384) == "octo"
    co = c_oracle.COracle(sd)
    n = 16384
    b, c, r, m = positions.random_positions(n, plies=120, seed=0)
    bd, cd, rd, md = _dev(b, c, r, m)
    p, q, v, best = [t.clone() for t in model.forward_masked(bd, cd, rd, md)]
    idx = np.arange(5, n, 2731)
    want = co.forward(b.numpy()[idx], c.numpy()[idx], r.numpy()[idx], mask=m.numpy()[idx])
    assert _bits_equal(p[idx], want["policy"]) and _bits_equal(q[idx], want["promo"])
    assert _bits_equal(v[idx], want["value"]) and (best.cpu().numpy()[idx] == want["best"]).all()
    part = model.forward_masked(bd[9000:9700], cd[9000:9700], rd[9000:9700], md[9000:9700])
    assert torch.equal(part[0], p[9000:9700]) and torch.equal(part[3], best[9000:9700])
    # the four-wavefront form returns the same bits
    other = encoder_impl("hip")(net, int8=True, out_dtype=torch.float32, kernel="board")
    part = other.forward_masked(bd[3000:4100], cd[3000:4100], rd[3000:4100], md[3000:4100])
    for x, y in zip(part, (p, q, v, best)):
        assert torch.equal(x, y[3000:4100])
    legal = ((md[..., None] >> torch.arange(64, device="cuda")) & 1).bool()
    assert torch.isneginf(p[~legal]).all() and torch.isfinite(p[legal]).all() and (v.abs() <= 1).all()
    has = legal.reshape(n, -1).any(1)
    assert torch.gather(legal.reshape(n, -1)[has], 1, best[has].long()[:, None]).all()


@pytest.mark.parametrize("head", ["pooled", "prenorm"])
@pytest.mark.parametrize("nv", [1, 3])
def test_pooled_value_heads_bit_exact_on_every_kernel(head, nv):
    # reference brokefish/nn/model.py:576-617 (its tests: tests/test_b2.py:520-650): the value row is
    # the mean of the live tokens (after or before norm_f) and the result is negated for Black
    torch.manual_seed(1)
    net = BrokefishNet(n_value=nv, value_head=head).eval().randomise_layers_(seed=4)
    sd = {k: v.detach() for k, v in net.state_dict().items()}
    b, c, r, m = positions.random_positions(96, plies=120, seed=13, stamp_queen=True)
    assert (c < 0).any() and (c > 0).any()
    want = c_oracle.COracle(sd).forward(b.numpy(), c.numpy(), r.numpy(), mask=m.numpy())
    bd, cd, rd, md = _dev(b, c, r, m)
    for kernel in ("twin", "octo", "duo", "board", "auto"):
        model = encoder_impl("hip")(net, int8=True, out_dtype=torch.float32, kernel=kernel)
        assert model.vmode == {"pooled": 1, "prenorm": 2}[head]
        p, q, v, best = model.forward_masked(bd, cd, rd, md)
        assert _bits_equal(v, want["value"]), (kernel, np.abs(v.cpu().numpy() - want["value"]).max())
        assert _bits_equal(p, want["policy"]) and _bits_equal(q, want["promo"]) and (best.cpu().numpy() == want["best"]).all()
    # the king head of the same weights gives other values; the sign flip shows on a colour swap of the control word
    king = BrokefishNet(n_value=nv).eval()
    king.load_state_dict({k: v for k, v in sd.items() if k != "value_mode"})
    vk = encoder_impl("hip")(king, int8=True, out_dtype=torch.float32).forward_full(bd, cd, rd)[2]
    assert not torch.allclose(vk, v, atol=1e-3)
    with pytest.raises(NotImplementedError):
        encoder_impl("hip")(net, int8=True, kernel="quad")
    wide = BrokefishNet(d_model=512, n_heads=16, d_ff=2048, n_layers=2, n_value=nv, value_head=head).eval().randomise_layers_(seed=6)
    sdw = {k: v.detach() for k, v in wide.state_dict().items()}
    ww = c_oracle.COracle(sdw).forward(b.numpy()[:24], c.numpy()[:24], r.numpy()[:24])
    for kernel in ("octo", "board"):
        vw = encoder_impl("hip")(wide, int8=True, out_dtype=torch.float32, kernel=kernel).forward_full(bd[:24], cd[:24], rd[:24])[2]
        assert _bits_equal(vw, ww["value"]), kernel


@pytest.mark.parametrize("head", ["pooled", "prenorm"])
@pytest.mark.parametrize("nv", [1, 3])
def test_pooled_value_heads_in_the_e4m3_format(head, nv):
    # the value heads are fp32 arithmetic behind either operand format: in e4m3 the kernels must
    # agree with each other bit for bit, give the emulation's value when started from the emulation's
    # own final residual stream, and follow it free-running wherever no byte flipped at a tie
    from oracle import emulated
    torch.manual_seed(2)
    net = BrokefishNet(n_value=nv, value_head=head).eval().randomise_layers_(seed=7)
    sd = {k: v.detach() for k, v in net.state_dict().items()}
    b, c, r, m = positions.random_positions(64, plies=120, seed=19, stamp_queen=True)
    assert (c < 0).any() and (c > 0).any()
    bd, cd, rd, md = _dev(b, c, r, m)
    etaps = {}
    with torch.no_grad():
        emu = emulated.forward(sd, b, c, r, mode="e4m3", taps=etaps)
    outs = {}
    for kernel in ("twin", "octo", "duo", "board"):
        model = encoder_impl("hip")(net, fp8=True, out_dtype=torch.float32, kernel=kernel)
        assert model.vmode == {"pooled": 1, "prenorm": 2}[head]
        outs[kernel] = [t.clone() for t in model.forward_masked(bd, cd, rd, md)]
        for x, y in zip(outs[kernel], outs["twin"]):
            assert torch.equal(x, y), kernel
    forced = model.forward_taps(bd, cd, rd, x_in=etaps["resid"][7].cuda(), layer_begin=8, layer_end=8, want=["normed"])
    assert (forced["value"].cpu() - emu[2]).abs().max() < 1e-5
    assert (forced["policy"].cpu() - emu[0]).abs().max() < 1e-4
    dv = (outs["twin"][2].cpu() - emu[2]).abs()
    assert (dv < 2e-2).float().mean() > 0.5 and dv.max() < 0.5 and (outs["twin"][2].abs() <= 1).all()
    # Black to move flips the sign of the White-frame prediction: the same board under the other
    # mover gives a value of the other sign from these heads only through the control word
    king = BrokefishNet(n_value=nv).eval()
    king.load_state_dict({k: v for k, v in sd.items() if k != "value_mode"})
    vk = encoder_impl("hip")(king, fp8=True, out_dtype=torch.float32).forward_full(bd, cd, rd)[2]
    assert not torch.allclose(vk, outs["twin"][2], atol=1e-3)


def test_matrix_pipe_probe_reports_a_plausible_rate():
    # a register-resident MFMA loop cannot beat the datasheet peak (5.0 POP/s dense int8 / fp8)
    # and, on a healthy part, reaches most of it; the evaluator's own rate must lie below it
    from brokefish_amd.hip_impl import mfma_rate
    for fmt in ("int8", "e4m3"):
        rate = mfma_rate(fmt, iters=5000, reps=3)
        assert 1000.0 < rate < 5500.0, (fmt, rate)


def test_weight_stream_probe_reports_a_plausible_rate():
    # a buffer that fits every L2 streams faster than one the size of the 512-wide network (50 MB,
    # more than the L2s hold); both lie between HBM speed and the L1 fill paths' nominal 39 TB/s
    from brokefish_amd.hip_impl import stream_rate
    small, large = stream_rate(1 << 20, workgroups=2048), stream_rate(50_626_560, workgroups=1024, reps=1)
    assert 8.0 < small < 45.0 and 2.0 < large < small, (small, large)


@pytest.mark.parametrize("kernel,n,fmt", [("auto", 64, "int8"), ("auto", 1000, "int8"), ("quad", 64, "int8"), ("board", 40, "int8"),
                                          ("twin", 300, "e4m3"), ("duo", 301, "e4m3"), ("octo", 33, "e4m3"), ("board", 20, "e4m3"),
                                          ("quad", 30, "e4m3")])
def test_phase_profile_runs_on_the_kernel_the_call_selects_and_leaves_the_outputs_right(kernel, n, fmt):
    torch.manual_seed(0)
    net = BrokefishNet().eval()
    model = encoder_impl("hip")(net, int8=fmt == "int8", fp8=fmt == "e4m3", kernel=kernel)
    b, c, r, m = positions.random_positions(n, plies=120, seed=5)
    bd, cd, rd, md = (t.cuda() for t in (b, c, r, m))
    want = [t.clone() for t in model.forward_full(bd, cd, rd, md)]
    for t in (model.policy_out, model.promo_out, model.value_out):
        t.zero_()
    ph = model.profile_phases(bd, cd, rd, md)
    assert set(ph) >= {"embed", "attention", "ffn1", "ffn2", "heads", "sync_wait", "total"}
    assert all(v >= 0 for v in ph.values()) and ph["total"] > 0
    parts = sum(v for k, v in ph.items() if k not in ("sync_wait", "total"))
    assert 0.9 * ph["total"] <= parts <= 1.0001 * ph["total"], ph   # the phases tile the wavefront's life
    for got, w in zip((model.policy_out, model.promo_out, model.value_out), want):
        assert torch.equal(got, w)


def test_phase_profile_of_the_512_wide_network_on_both_of_its_kernels():
    torch.manual_seed(0)
    net = BrokefishNet(d_model=512, n_heads=16, d_ff=2048, n_layers=2).eval()
    b, c, r, m = positions.random_positions(24, plies=120, seed=6)
    bd, cd, rd, md = (t.cuda() for t in (b, c, r, m))
    for kernel in ("board", "octo"):
        model = encoder_impl("hip")(net, int8=True, kernel=kernel)
        want = [t.clone() for t in model.forward_full(bd, cd, rd, md)]
        ph = model.profile_phases(bd, cd, rd, md)
        parts = sum(v for k, v in ph.items() if k not in ("sync_wait", "total"))
        assert ph["total"] > 0 and 0.9 * ph["total"] <= parts <= 1.0001 * ph["total"], (kernel, ph)
        for got, w in zip((model.policy_out, model.promo_out, model.value_out), want):
            assert torch.equal(got, w)


def test_set_profile_accumulates_over_calls_until_reset_like_the_references_switch():
    """reference csrc/encoder.cu:1886-1903 and bench/bench_phases.py:99-105: set_profile(True),
    reset_profile(), run, read_profile(), set_profile(False)."""
    torch.manual_seed(0)
    net = BrokefishNet().eval()
    model = encoder_impl("hip")(net, int8=True)
    b, c, r, m = positions.random_positions(600, plies=120, seed=7)
    bd, cd, rd, md = (t.cuda() for t in (b, c, r, m))
    want = [t.clone() for t in model.forward_full(bd, cd, rd, md)]
    names = model.profile_phase_names()
    assert names[-1] == "total" and "sync_wait" in names
    cyc, waves = model.read_profile()
    assert waves == 0 and int(cyc.sum()) == 0               # nothing recorded before it is switched on
    model.set_profile(True)
    model.reset_profile()
    model.forward_full(bd, cd, rd, md)
    one, w1 = model.read_profile()
    assert w1 == 8 * 300 and int(one[-1]) > 0               # 600 positions on the two-position kernel
    model.forward_full(bd, cd, rd, md)
    model.forward_full(bd[:100], cd[:100], rd[:100], md[:100])       # a small call: eight wavefronts per position
    two, w2 = model.read_profile()
    assert w2 == 2 * w1 + 800 and (two >= one).all() and int(two[-1]) > 1.5 * int(one[-1])
    model.set_profile(False)
    kept, wk = model.read_profile()
    assert wk == w2 and torch.equal(kept, two)              # switched off: the counters stay readable
    got = model.forward_full(bd, cd, rd, md)                # and calls are no longer counted
    assert all(torch.equal(g, w) for g, w in zip(got, want))
    assert model.read_profile()[1] == w2
    model.reset_profile()
    assert model.read_profile()[1] == 0


def test_two_hundred_thousand_positions_agree_bit_for_bit_across_the_kernels(base):
    # size-independent property at the sweep's largest launches: the kernels are the same function
    # (two positions per workgroup, one per workgroup with two workgroups per unit, four per
    # workgroup, and the automatic choice with its split last round), in int8 and in e4m3, on
    # launches whose sizes are multiples of nothing; a sample goes against the C checker
    net, sd, boards, quad, co = base
    hip = encoder_impl("hip")
    mods = {k: hip(net, int8=True, out_dtype=torch.float32, kernel=k) for k in ("duo", "twin", "auto")}
    f8 = {k: hip(net, fp8=True, out_dtype=torch.float32, kernel=k) for k in ("duo", "twin")}
    for seed, n in ((0, 65536), (1, 65536 - 771), (2, 65536 + 130)):
        b, c, r, m = positions.random_positions(n, plies=200, seed=3000 + seed)
        dev = _dev(b, c, r, m)
        ref = [t.clone() for t in mods["duo"].forward_masked(*dev)]
        for other in (mods["twin"], mods["auto"], quad):
            for g, w in zip(other.forward_masked(*dev), ref):
                assert torch.equal(g, w), seed
        e = [t.clone() for t in f8["duo"].forward_masked(*dev)]
        for g, w in zip(f8["twin"].forward_masked(*dev), e):
            assert torch.equal(g, w), seed
        idx = np.arange(seed, n, 1999)
        want = co.forward(b.numpy()[idx], c.numpy()[idx], r.numpy()[idx], mask=m.numpy()[idx])
        assert _bits_equal(ref[0][idx], want["policy"]) and _bits_equal(ref[1][idx], want["promo"])
        assert _bits_equal(ref[2][idx], want["value"]) and (ref[3].cpu().numpy()[idx] == want["best"]).all()
