"""Parity of the HIP evaluator, through the C-ABI, against the CPU checkers.

The bar: everything integer (operand bytes, int32 accumulators, the masked argmax) is
bit-exact; the fp32 outputs are bit-exact as well against the C checker, because the
kernel's fp32 operation order is the one that file spells out.  fp16 outputs are the
fp32 outputs rounded once.  Against the torch restatement (library summation order) the
comparison is teacher-forced layer by layer, tolerance 2e-5 of the stream's scale on rows
whose operand bytes agree (the tolerance of an fp32 re-ordering, far inside the 1e-3 the
target states); free-running, the forward's own sensitivity bounds what any two
orderings can agree to, and that spread is recorded in tests/test_oracle.py.
"""
import numpy as np
import pytest
import torch

from brokefish_amd import encoder_impl, positions
from brokefish_amd.net import BrokefishNet
from oracle import c_oracle, emulated
import reflayers

pytestmark = pytest.mark.gpu

TAPS_INT = ["qa_qkv", "acc_qkv", "qa_out", "acc_out", "qa_ff1", "acc_ff1", "qa_ff2", "acc_ff2"]
TAPS_F32 = ["embed", "resid", "normed"]


def _make(nv=1, distinct=True, seed=0, n_layers=8):
    torch.manual_seed(seed)
    net = BrokefishNet(n_value=nv, n_layers=n_layers).eval()
    if distinct:
        net.randomise_layers_(seed=seed + 3)
    sd = {k: v.detach() for k, v in net.state_dict().items()}
    return net, sd


@pytest.fixture(scope="module")
def nets():
    out = {}
    for key, (nv, distinct) in {"distinct": (1, True), "seed0": (1, False), "wdl": (3, True)}.items():
        net, sd = _make(nv, distinct)
        out[key] = (net, sd, encoder_impl("hip")(net, int8=True, out_dtype=torch.float32), c_oracle.COracle(sd))
    return out


def _dev(*ts):
    return [t.cuda() for t in ts]


def _bits_equal(a: torch.Tensor, b: np.ndarray) -> bool:
    a = a.cpu().numpy()
    if a.dtype == np.uint8:
        b = b.view(np.uint8)
    return a.shape == b.shape and bool((a.view(np.int32 if a.dtype == np.float32 else a.dtype)
                                        == b.view(np.int32 if b.dtype == np.float32 else b.dtype)).all())


@pytest.mark.parametrize("key", ["distinct", "seed0", "wdl"])
def test_bit_exact_against_the_c_checker_with_every_tap(nets, key):
    net, sd, model, co = nets[key]
    b, c, r, m = positions.random_positions(64, plies=120, seed=11, stamp_queen=True)
    got = model.forward_taps(*_dev(b, c, r), mask=m.cuda())
    want = co.forward(b.numpy(), c.numpy(), r.numpy(), mask=m.numpy(), taps=True)
    for k in TAPS_INT + TAPS_F32 + ["policy", "promo", "value", "best"]:
        assert _bits_equal(got[k], want[k]), k
    # the reference's stage numbers that exist outside its kernel: 9 = embeddings, 8 = norm_f output
    assert _bits_equal(model.forward_stage(*_dev(b, c, r), 9), want["embed"])
    assert _bits_equal(model.forward_stage(*_dev(b, c, r), 8), want["normed"])
    with pytest.raises(NotImplementedError):
        model.forward_stage(*_dev(b, c, r), 3)
    # the accumulators really are the exact integer product of the kernel's own operand bytes
    q, _ = co.qweight("ff2", 3)
    a = got["qa_ff2"][:, 3].cpu().numpy().astype(np.int64)                 # [n,32,1024] unsigned
    acc = np.stack([a[..., 256 * k:256 * k + 256] @ q[:, 256 * k:256 * k + 256].astype(np.int64).T for k in range(4)], 1)
    assert (acc == got["acc_ff2"][:, 3].cpu().numpy()).all()
    q, _ = co.qweight("qkv", 0)
    a = got["qa_qkv"][:, 0].cpu().numpy().astype(np.int64)
    assert ((a @ q.astype(np.int64).T) == got["acc_qkv"][:, 0, 0].cpu().numpy()).all()


def test_production_launch_equals_the_tapped_launch_and_fp16_is_one_rounding(nets):
    net, sd, model, co = nets["distinct"]
    b, c, r, m = positions.random_positions(96, plies=120, seed=12)
    bd, cd, rd, md = _dev(b, c, r, m)
    tapped = model.forward_taps(bd, cd, rd, mask=md, want=["normed"])
    p, q, v = model.forward_full(bd, cd, rd, md)
    assert torch.equal(p, tapped["policy"]) and torch.equal(q, tapped["promo"]) and torch.equal(v, tapped["value"])
    assert torch.equal(model.best_move, tapped["best"])
    praw, qraw, vraw = [t.clone() for t in model.forward_full(bd, cd, rd)]
    assert model.best_move is None and torch.isfinite(praw).all()
    half = encoder_impl("hip")(net, int8=True)                              # default: the fp16 contract
    ph, qh, vh = half.forward_full(bd, cd, rd)
    assert ph.dtype is torch.float16 and qh.dtype is torch.float16 and vh.dtype is torch.float32
    assert ph.shape == (96, 32, 64) and qh.shape == (96, 32, 4) and vh.shape == (96,)
    assert torch.equal(ph, praw.half()) and torch.equal(qh, qraw.half()) and torch.equal(vh, vraw)
    assert (vh.abs() <= 1).all()


def test_raw_logits_are_not_masked_and_the_mask_is_an_exact_and(nets):
    # reference tests/test_b2.py:226-247: the evaluator returns raw logits unless asked
    net, sd, model, co = nets["distinct"]
    b, c, r, m = positions.random_positions(64, plies=120, seed=13)
    bd, cd, rd, md = _dev(b, c, r, m)
    raw = model.forward_full(bd, cd, rd)[0].clone()
    masked, _, _, best = model.forward_masked(bd, cd, rd, md)
    legal = ((md[..., None] >> torch.arange(64, device="cuda")) & 1).bool()
    assert torch.isfinite(raw).all()
    assert torch.equal(masked[legal], raw[legal]) and torch.isneginf(masked[~legal]).all()
    flat = torch.where(legal, raw, torch.full_like(raw, float("-inf"))).reshape(64, -1)
    has = legal.reshape(64, -1).any(1)
    assert torch.equal(best[has].long(), flat.argmax(1)[has])
    want = co.forward(b.numpy(), c.numpy(), r.numpy(), mask=m.numpy())
    assert (best.cpu().numpy() == want["best"]).all()
    # a position with no legal move reports -1; equal logits resolve to the lowest legal index
    none = torch.zeros_like(md)
    assert (model.forward_masked(bd, cd, rd, none)[3] == -1).all()
    net0, _ = _make()
    with torch.no_grad():
        net0.policy.weight.zero_()
    tie = encoder_impl("hip")(net0, int8=True, out_dtype=torch.float32)
    first = legal.reshape(64, -1).float().argmax(1)
    assert torch.equal(tie.forward_masked(bd, cd, rd, md)[3][has].long(), first[has])


def test_batch_sizes_composition_independence_and_determinism(nets):
    # reference tests/test_quant.py:309-339, :395-418 and tests/test_b2.py:314-322
    net, sd, model, co = nets["distinct"]
    b, c, r, m = positions.random_positions(1027, plies=120, seed=14)
    bd, cd, rd, md = _dev(b, c, r, m)
    full = [t.clone() for t in model.forward_masked(bd, cd, rd, md)]
    again = model.forward_masked(bd, cd, rd, md)
    for x, y in zip(full, again):
        assert torch.equal(x, y)                                            # bit-deterministic
    for n in (1, 3, 31, 33, 127, 257, 1024):
        part = model.forward_masked(bd[:n], cd[:n], rd[:n], md[:n])
        for x, y in zip(full, part):
            assert y.shape[0] == n and torch.equal(x[:n], y)
    perm = torch.randperm(1027, generator=torch.Generator().manual_seed(0)).cuda()
    shuffled = model.forward_masked(bd[perm], cd[perm], rd[perm], md[perm])
    for x, y in zip(full, shuffled):
        assert torch.equal(x[perm], y)


def test_outputs_are_views_of_buffers_the_object_owns(nets):
    # reference brokefish/nn/cuda_impl.py:467-472, pinned by tests/test_validate.py:82-98
    net, sd, model, co = nets["distinct"]
    b, c, r, _ = positions.random_positions(8, plies=60, seed=15)
    bd, cd, rd = _dev(b, c, r)
    p1, q1, v1 = model.forward_full(bd, cd, rd)
    keep = p1.clone()
    p2, _, _ = model.forward_full(bd.flip(0), cd.flip(0), rd.flip(0))
    assert p1.data_ptr() == p2.data_ptr() and torch.equal(p2, keep.flip(0))
    p3, _, _ = model.forward_full(bd[:4], cd[:4], rd[:4])
    assert p3.shape[0] == 4 and torch.equal(p3, keep[:4])


def test_bad_inputs_are_rejected(nets):
    # reference tests/test_b2.py:325-343
    net, sd, model, co = nets["distinct"]
    b, c, r, m = _dev(*positions.random_positions(4, plies=10, seed=1))
    for bad in [(b.int(), c, r), (b[:, :31], c, r), (b, c.int(), r), (b, c[:3], r), (b, c, r.int()),
                (b.cpu(), c, r), (b, c, r, m.int()), (b, c, r, m[:2])]:
        with pytest.raises(ValueError):
            model.forward_full(*bad)
    with pytest.raises(ValueError):
        model.forward_taps(b, c, r, x_in=torch.zeros(4, 32, 128, device="cuda"))


def test_every_clock_and_rep_and_dead_slot_inertness_on_device(nets):
    # reference tests/test_b2.py:110-153 (all clocks x signs x reps) and :270-293 (dead slots)
    net, sd, model, co = nets["distinct"]
    base = positions.random_positions_np(1, plies=0)[0]
    ctrl = np.array([s * mag for mag in range(1, 103) for s in (1, -1) for _ in range(3)], np.int16)
    reps = np.array([rp for _ in range(1, 103) for _ in (1, -1) for rp in (0, 1, 2)], np.uint8)
    bb = np.repeat(base, len(ctrl), axis=0).view(np.int16)
    got = model.forward_taps(torch.from_numpy(bb).cuda(), torch.from_numpy(ctrl).cuda(),
                             torch.from_numpy(reps).cuda(), want=["embed"])
    want = co.forward(bb, ctrl, reps, taps=True)
    assert _bits_equal(got["embed"], want["embed"]) and _bits_equal(got["policy"], want["policy"])
    assert len({got["embed"][i, 0].cpu().numpy().tobytes() for i in range(len(ctrl))}) == 101 * 2 * 3

    b, c, r, _ = positions.random_positions_np(128, plies=120, seed=8)
    dead = (b & 0x800) != 0
    rng = np.random.default_rng(1)
    junk = (rng.integers(0, 6, size=b.shape).astype(np.uint16) << 6) | rng.integers(0, 64, size=b.shape).astype(np.uint16) \
        | (rng.integers(0, 4, size=b.shape).astype(np.uint16) << 9)
    b2 = b.copy()
    b2[dead] = 0x800 | junk[dead]
    args = lambda x: _dev(torch.from_numpy(x.view(np.int16)), torch.from_numpy(c), torch.from_numpy(r))
    p1, q1, v1 = [t.clone() for t in model.forward_full(*args(b))]
    p2, q2, v2 = model.forward_full(*args(b2))
    live = torch.from_numpy(~dead).cuda()
    assert torch.equal(p1[live], p2[live]) and torch.equal(q1[live], q2[live]) and torch.equal(v1, v2)
    assert torch.isfinite(p2).all()


def test_teacher_forced_layers_against_the_torch_restatement(nets, capsys):
    net, sd, model, co = nets["distinct"]
    n = 32
    b, c, r, _ = positions.random_positions(n, plies=100, seed=16, stamp_queen=True)
    taps = {}
    with torch.no_grad():
        ref = emulated.forward(sd, b, c, r, mode="int8", taps=taps)
    bd, cd, rd = _dev(b, c, r)
    x_in = taps["embed"]
    n_flips, n_bytes, worst = 0, 0, 0.0
    for l in range(8):
        got = model.forward_taps(bd, cd, rd, x_in=x_in.cuda(), layer_begin=l, layer_end=l + 1,
                                 want=TAPS_INT + ["resid"])
        dirty = np.zeros((n, 32), bool)
        for name in ("qkv", "out", "ff1", "ff2"):
            qt = taps["qa_" + name][l].numpy().reshape(n, 32, -1).astype(np.int32)
            qg = got["qa_" + name][:, 0].cpu().numpy().astype(np.int32)
            mism = qt != qg
            assert np.abs(qt - qg)[~dirty].max() <= 1
            # every flipped byte on a clean row is a provable tie: the quotient x / s (float64, from
            # the restatement's own fp32 x and s) sits within 2^-18 of full scale of a rounding boundary
            flips = mism & ~dirty[..., None]
            dist = reflayers.tie_distance(taps["quot_" + name][l].numpy().reshape(n, 32, -1))
            tol = reflayers.TIE_TOL_U8 if name == "ff2" else reflayers.TIE_TOL
            assert (dist[flips] <= tol).all(), (l, name, int(flips.sum()), float(dist[flips].max()))
            n_flips += int(flips.sum())
            n_bytes += int((~dirty).sum()) * qt.shape[-1]
            worst = max(worst, float(dist[flips].max()) if flips.any() else 0.0)
            at = taps["acc_" + name][l].numpy()
            at = at.reshape(at.shape[0], n, 32, -1).transpose(1, 2, 0, 3)           # [n,32,kc,N]
            ag = got["acc_" + name][:, 0].cpu().numpy().transpose(0, 2, 1, 3)
            ok = ~mism.any(-1)
            assert (at[ok] == ag[ok]).all()           # int32 accumulators bit-exact given equal operands
            dirty |= mism.any(-1)
            if name == "qkv":
                dirty |= mism.any(-1).any(-1)[:, None]
        x_next = taps["resid"][l]
        d = (got["resid"][:, 0].cpu() - x_next).abs().amax(-1).numpy()
        assert d[~dirty].max() < 2e-5 * max(float(x_next.abs().max()), 1.0)
        assert (~dirty).mean() > 0.5
        x_in = x_next
    with capsys.disabled():
        print(f"\n  HIP vs torch restatement, teacher-forced: {n_flips} flipped bytes of {n_bytes} on clean rows, "
              f"every one within {worst:.2e} steps of a tie (allowed {reflayers.TIE_TOL:.2e})")
    # heads, teacher-forced on the torch restatement's final residual stream
    got = model.forward_taps(bd, cd, rd, x_in=taps["resid"][7].cuda(), layer_begin=8, layer_end=8, want=["normed"])
    assert (got["policy"].cpu() - ref[0]).abs().max() < 1e-4            # tolerance: fp32 re-ordering, << 1e-3
    assert (got["promo"].cpu() - ref[1]).abs().max() < 1e-4
    assert (got["value"].cpu() - ref[2]).abs().max() < 1e-5


def _first_divergence_walk(sd, model, b, c, r, library_stack=False):
    """Free-running comparison of the kernel with the torch restatement (reference
    brokefish/nn/quant.py:281-305, :443-506 over brokefish/nn/model.py:621-645), board by board:
    both run with taps; each board's quantisers are walked in order (layer, then qkv / out / ff1 /
    ff2) to its FIRST differing operand byte, which must be a provable tie (up to there both sides
    computed the same numbers to fp32 summation order).  Returns (emulation outputs, kernel outputs,
    flipped [n] bool, worst tie distance)."""
    n = b.shape[0]
    etaps = {}
    with torch.no_grad():
        emu = (emulated.forward_library_stack if library_stack else emulated.forward)(sd, b, c, r, mode="int8", taps=etaps)
    gtaps = model.forward_taps(*_dev(b, c, r), want=["qa_qkv", "qa_out", "qa_ff1", "qa_ff2"])
    flipped = np.zeros(n, bool)
    worst = 0.0
    for l in range(8):
        for name in ("qkv", "out", "ff1", "ff2"):
            qt = etaps["qa_" + name][l].numpy().reshape(n, 32, -1).astype(np.int32)
            qg = gtaps["qa_" + name][:, l].cpu().numpy().astype(np.int32)
            mism = qt != qg
            first = mism & ~flipped[:, None, None]
            if first.any():
                dist = reflayers.tie_distance(etaps["quot_" + name][l].numpy().reshape(n, 32, -1))[first]
                tol = reflayers.TIE_TOL_U8 if name == "ff2" else reflayers.TIE_TOL
                assert (dist <= tol).all(), (l, name, float(dist.max()))
                assert np.abs(qt - qg)[first].max() == 1
                worst = max(worst, float(dist.max()))
            flipped |= mism.any((1, 2))
    got = [gtaps[k].cpu() for k in ("policy", "promo", "value")]
    return emu, got, flipped, worst


@pytest.mark.parametrize("key", ["distinct", "seed0"])
def test_free_running_every_board_without_a_flipped_byte_meets_the_stated_tolerance(nets, key, capsys):
    # The target "logits and value within 1e-3 of the int8-simulated forward", free-running, board
    # by board: a board whose operand bytes all equal the emulation's must meet it -- every such
    # board -- and a board that differs must do so first at a provable rounding tie.
    net, sd, model, co = nets[key]
    n = 256
    b, c, r, _ = positions.random_positions(n, plies=120, seed=41, stamp_queen=True)
    emu, got, flipped, worst = _first_divergence_walk(sd, model, b, c, r)
    dp = (got[0] - emu[0]).abs().reshape(n, -1).amax(1).numpy()
    dq = (got[1] - emu[1]).abs().reshape(n, -1).amax(1).numpy()
    dv = (got[2] - emu[2]).abs().numpy()
    clean = ~flipped
    with capsys.disabled():
        print(f"\n  int8 free-running ({key} network), {n} boards: {int(clean.sum())} without a flipped byte, worst of them "
              f"{dp[clean].max():.2e} (policy) / {dv[clean].max():.2e} (value) from the emulation (target 1e-3); "
              f"{int(flipped.sum())} with a first flip (a tie to {worst:.2e} steps), of them "
              f"{int((dp[flipped] <= 1e-3).sum())} still within 1e-3, worst {dp.max():.2e}")
    assert clean.sum() >= n // 2
    assert (dp[clean] <= 1e-3).all() and (dq[clean] <= 1e-3).all() and (dv[clean] <= 1e-3).all()
    assert dp[clean].max() < 1e-4 and dv[clean].max() < 1e-4        # in fact they agree to fp32 re-ordering
    assert dp.max() < 0.1                                          # a flipped byte moves the logits by a bounded amount


def test_free_running_against_the_references_golden_logits_board_by_board(capsys):
    # the same statement against what the reference's own emulated_forward wrote for its eight
    # golden positions (tests/golden/reference_vectors.npz): the walk is against the taps of the
    # restatement's route through torch's own encoder modules, which reproduces the golden logits
    # bit for bit (tests/test_oracle.py, on the CPU that wrote them); the tolerance is against the
    # golden numbers themselves
    import os
    import make_golden as mg
    g = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "reference_vectors.npz"))
    torch.manual_seed(0)
    gnet = BrokefishNet().eval()
    gnet.load_state_dict(mg.fill_state_dict(gnet.state_dict()))
    sd = {k: v.detach() for k, v in gnet.state_dict().items()}
    model = encoder_impl("hip")(gnet, int8=True, out_dtype=torch.float32)
    b, c, r = mg.positions()
    emu, got, flipped, worst = _first_divergence_walk(sd, model, b, c, r, library_stack=True)
    dp = np.abs(got[0].numpy() - g["int8_policy_nv1"]).reshape(len(flipped), -1).max(1)
    dv = np.abs(got[2].numpy() - g["int8_value_nv1"])
    with capsys.disabled():
        print(f"\n  int8 free-running, the reference's 8 golden positions: {int((~flipped).sum())} without a flipped byte "
              f"(worst {dp[~flipped].max() if (~flipped).any() else 0:.2e} from the golden logits), {int(flipped.sum())} "
              f"with a first flip at a tie ({worst:.2e} steps), worst of all {dp.max():.2e}")
    assert (dp[~flipped] <= 1e-3).all() and (dv[~flipped] <= 1e-3).all()
    assert dp.max() < 2e-2 and dv.max() < 2e-2


def test_backbone_call_from_a_bare_encoder_stack(nets):
    # reference brokefish/nn/cuda_impl.py:447-463 and tests/test_model.py: the stack alone, x in, x out
    net, sd, model, co = nets["distinct"]
    bare = encoder_impl("hip")(net.encoder, int8=True)
    with pytest.raises(ValueError):
        bare.forward_full(*_dev(*positions.random_positions(2, plies=4, seed=1, with_mask=False)))
    b, c, r, _ = positions.random_positions(24, plies=100, seed=17)
    with torch.no_grad():
        x, alive = emulated.embed(sd, b, c, r)
    want = co.forward(b.numpy(), c.numpy(), r.numpy(), taps=True)["resid"][:, -1]
    got = bare(x.cuda(), alive.cuda())
    assert got.shape == (24, 32, 256) and _bits_equal(got, want)
    same = model.forward(x.cuda(), alive.to(torch.int8).cuda())
    assert torch.equal(same, got)
    half = bare(x.half().cuda(), alive.cuda())
    assert half.dtype is torch.float16
    # dead tokens are inert as keys: garbage in their rows changes no live row
    x2 = x.clone()
    x2[~alive] = 7.5
    got2 = bare(x2.cuda(), alive.cuda())
    assert torch.equal(got2[alive.cuda()], got[alive.cuda()])


def test_backbone_call_with_an_output_buffer_allocates_nothing_once_warm(nets):
    # reference brokefish/nn/cuda_impl.py:447-463 takes out= so that a serving loop can reuse one
    # buffer; here the whole call then runs out of buffers kept between calls
    net, sd, model, co = nets["distinct"]
    b, c, r, _ = positions.random_positions(700, plies=100, seed=18)
    with torch.no_grad():
        x, alive = emulated.embed(sd, b, c, r)
    xd, ad = x.cuda(), alive.cuda()
    out = torch.empty_like(xd)
    want = model.forward(xd, ad).clone()                       # two positions per workgroup at this size
    idx = np.arange(0, 700, 29)
    ref = co.forward(b.numpy()[idx], c.numpy()[idx], r.numpy()[idx], taps=True)["resid"][:, -1]
    assert _bits_equal(want[idx], ref)
    model.forward(xd, ad, out=out)                             # warm: buffers exist from here on
    torch.cuda.synchronize()
    count = lambda: torch.cuda.memory_stats()["allocation.all.allocated"]
    before = count()
    out.zero_()
    assert model.forward(xd, ad, out=out) is out
    model.forward(xd[:40], ad[:40], out=out[:40])              # a smaller call reuses the same buffers
    model.forward(xd[:40], None, out=out[:40])
    assert count() == before
    assert torch.equal(out[40:], want[40:])
    everyone = model.forward(xd[:40], torch.ones_like(ad[:40]))
    assert torch.equal(out[:40], everyone)
    # a half-precision caller: converted through kept buffers, the result comes back in its dtype
    oh = torch.empty(700, 32, 256, dtype=torch.float16, device="cuda")
    model.forward(xd.half(), ad, out=oh)
    assert torch.equal(oh, model.forward(xd.half().float(), ad).half())


def test_full_batch_properties_at_4096(nets):
    # the metric's batch size: spot-check against the C checker, and size-independent properties
    net, sd, model, co = nets["seed0"]
    b, c, r, m = positions.random_positions(4096, plies=120, seed=0)
    bd, cd, rd, md = _dev(b, c, r, m)
    p, q, v, best = [t.clone() for t in model.forward_masked(bd, cd, rd, md)]
    idx = np.arange(0, 4096, 37)
    want = co.forward(b.numpy()[idx], c.numpy()[idx], r.numpy()[idx], mask=m.numpy()[idx])
    assert _bits_equal(p[idx], want["policy"]) and _bits_equal(q[idx], want["promo"])
    assert _bits_equal(v[idx], want["value"]) and (best.cpu().numpy()[idx] == want["best"]).all()
    half = model.forward_masked(bd[2048:], cd[2048:], rd[2048:], md[2048:])
    assert torch.equal(half[0], p[2048:]) and torch.equal(half[3], best[2048:])
    legal = ((md[..., None] >> torch.arange(64, device="cuda")) & 1).bool()
    assert torch.isneginf(p[~legal]).all() and torch.isfinite(p[legal]).all() and (v.abs() <= 1).all()
    has = legal.reshape(4096, -1).any(1)
    chosen = torch.gather(legal.reshape(4096, -1)[has], 1, best[has].long()[:, None])
    assert chosen.all()                                                  # the argmax is always a legal move
