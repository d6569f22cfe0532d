"""Parity of the e4m3 variant of the HIP evaluator, through the C-ABI, against the torch
restatement of the reference's fp8 emulation (``oracle/emulated.py``, mode "e4m3").

What can and cannot agree, and the tolerance of each comparison:

* operand bytes are produced by exact arithmetic (correctly rounded quotient, round to nearest
  even e4m3): given identical inputs they are IDENTICAL -- asserted on the first matmul of every
  teacher-forced layer, whose input is the checker's own residual stream;
* the accumulators come from the fp16 matrix instruction fed with the e4m3 operands widened
  exactly: products are exact and the sum carries fp32 precision, so they agree with the exact
  product of the kernel's own operand bytes to 2e-7 of sum|a*w| (measured 3.3e-8) -- the
  distance between two fp32 summation orders, which is also all that separates them from the
  emulation's library matmul.  (The fp8 instruction itself keeps only about 16 bits below its
  largest addend -- 3e-5 of sum|a*w| -- and is not used.);
* that difference still flips about 1e-6 of the next quantiser's bytes (a quotient within
  rounding of an e4m3 tie; the flipped byte is the neighbouring value, 6 % of the element).
  Rows with no flipped byte leave a layer within 1e-5 of the emulation (measured 2e-6); a row
  with a flip differs by up to 0.1;
* free-running, a flip anywhere in the eight layers moves that board's logits by about 0.1 --
  the format's own sensitivity, the same spread two orderings of the emulation itself show
  (tests/test_oracle_e4m3.py).  Boards without a flip (the majority: measured 67-72 %) match
  the emulation to 2e-2, most of them bit for bit; over all boards the kernel is as close to the
  fp32 network as the emulation is.
"""
import os

import numpy as np
import pytest
import torch

import make_golden as mg
import reflayers
from brokefish_amd import encoder_impl, positions
from brokefish_amd.net import BrokefishNet
from oracle import emulated

pytestmark = pytest.mark.gpu

WEIGHT = {"qkv": "self_attn.in_proj_weight", "out": "self_attn.out_proj.weight",
          "ff1": "linear1.weight", "ff2": "linear2.weight"}


@pytest.fixture(scope="module")
def setup():
    torch.manual_seed(0)
    net = BrokefishNet().eval()
    net.randomise_layers_(seed=3)
    sd = {k: v.detach() for k, v in net.state_dict().items()}
    return net, sd, encoder_impl("hip")(net, fp8=True, out_dtype=torch.float32)


def _dev(*ts):
    return [t.cuda() for t in ts]


def test_teacher_forced_layers_against_the_emulation(setup, capsys):
    net, sd, model = setup
    n = 32
    b, c, r, _ = positions.random_positions(n, plies=100, seed=16, stamp_queen=True)
    taps = {}
    with torch.no_grad():
        ref = emulated.forward(sd, b, c, r, mode="e4m3", taps=taps)
    bd, cd, rd = _dev(b, c, r)
    x_in = taps["embed"]
    n_flips, n_bytes, worst = 0, 0, [0.0, 0.0]
    for l in range(8):
        got = model.forward_taps(bd, cd, rd, x_in=x_in.cuda(), layer_begin=l, layer_end=l + 1)
        dirty = np.zeros((n, 32), bool)
        for name in ("qkv", "out", "ff1", "ff2"):
            qt = taps["qa_" + name][l].reshape(n, 32, -1).numpy()
            qg = got["qa_" + name][:, 0].cpu().float().numpy()
            mism = qt != qg
            # Every flipped byte on a row whose inputs were still clean is the neighbouring e4m3 value
            # (one step is at most 1/8 of the magnitude) and a provable tie: the emulation's own
            # quotient x / s (float64) sits on the midpoint of two neighbouring e4m3 values to within
            # the distance two fp32 summation orders of the same input can differ by.
            first = mism & ~dirty[..., None]
            assert (np.abs(qt - qg)[first] <= 0.1251 * np.maximum(np.abs(qt), np.abs(qg))[first] + 2.0 ** -9).all()
            dist = reflayers.e4m3_tie_distance(taps["quot_" + name][l].numpy().reshape(n, 32, -1))
            tol = reflayers.E4M3_TIE_TOL if name == "qkv" else reflayers.E4M3_TIE_TOL_AFTER_MATMUL
            assert (dist[first] <= tol).all(), (l, name, int(first.sum()), float(dist[first].max()))
            n_flips += int(first.sum())
            n_bytes += int((~dirty).sum()) * qt.shape[-1]
            worst[name != "qkv"] = max(worst[name != "qkv"], float(dist[first].max()) if first.any() else 0.0)
            # the accumulators against the exact product of the kernel's OWN operand bytes
            wq = emulated.quantise_weights_e4m3(sd[f"encoder.layers.{l}.{WEIGHT[name]}"])[0].numpy().astype(np.float64)
            ag = got["acc_" + name][:, 0].cpu().numpy()                       # [n, kc, 32, N]
            for k in range(ag.shape[1]):
                a = qg[..., 256 * k:256 * k + 256].astype(np.float64)
                w = wq[:, 256 * k:256 * k + 256]
                exact, mag = a @ w.T, np.abs(a) @ np.abs(w).T
                assert (np.abs(ag[:, k] - exact) <= 2e-7 * mag + 1e-9).all(), (l, name, k)
            dirty |= mism.any(-1)
            if name == "qkv":
                dirty |= mism.any(-1).any(-1)[:, None]
        x_next = taps["resid"][l]
        d = (got["resid"][:, 0].cpu() - x_next).abs().amax(-1).numpy()
        assert d[~dirty].max() < 1e-5 and (~dirty).mean() > 0.9
        assert d.max() < 0.5                        # a flipped byte moves a row by a bounded amount
        x_in = x_next
    with capsys.disabled():
        print(f"\n  e4m3 HIP vs emulation, teacher-forced: {n_flips} flipped bytes of {n_bytes} on clean rows; distance from an "
              f"e4m3 tie at most {worst[0]:.2e} (first quantiser, allowed {reflayers.E4M3_TIE_TOL:.2e}) / {worst[1]:.2e} "
              f"(behind a matmul, allowed {reflayers.E4M3_TIE_TOL_AFTER_MATMUL:.2e})")
    got = model.forward_taps(bd, cd, rd, x_in=taps["resid"][7].cuda(), layer_begin=8, layer_end=8, want=["normed"])
    assert (got["policy"].cpu() - ref[0]).abs().max() < 1e-4
    assert (got["promo"].cpu() - ref[1]).abs().max() < 1e-4
    assert (got["value"].cpu() - ref[2]).abs().max() < 1e-5


def test_free_running_accuracy_equals_the_emulations(setup, capsys):
    net, sd, model = setup
    b, c, r, _ = positions.random_positions(64, plies=120, seed=11, stamp_queen=True)
    with torch.no_grad():
        emu = emulated.forward(sd, b, c, r, mode="e4m3")
        f32 = emulated.forward(sd, b, c, r, mode="fp32")
    got = [t.cpu() for t in model.forward_full(*_dev(b, c, r))]
    assert all(torch.isfinite(t).all() for t in got)
    # The stated target (logits within 2e-2 of the emulation) board by board: run both with taps,
    # walk each board's quantisers in order (layer, then qkv / out / ff1 / ff2) to its FIRST
    # diverging operand byte.  A board with none must meet the target -- every such board, not a
    # share of them; and every first divergence must be a provable e4m3 tie (up to there the two
    # sides computed the same numbers to fp32 summation order).
    etaps = {}
    with torch.no_grad():
        emulated.forward(sd, b, c, r, mode="e4m3", taps=etaps)
    gtaps = model.forward_taps(*_dev(b, c, r), want=["qa_qkv", "qa_out", "qa_ff1", "qa_ff2"])
    assert torch.equal(gtaps["policy"].cpu(), got[0])
    per_board = (got[0] - emu[0]).abs().reshape(64, -1).amax(1).numpy()
    per_board_v = (got[2] - emu[2]).abs().numpy()
    flipped = np.zeros(64, bool)
    worst = 0.0
    for l in range(8):
        for name in ("qkv", "out", "ff1", "ff2"):
            qt = etaps["qa_" + name][l].reshape(64, 32, -1).numpy()
            qg = gtaps["qa_" + name][:, l].cpu().float().numpy()
            mism = qt != qg
            first = mism & ~flipped[:, None, None]
            if first.any():
                dist = reflayers.e4m3_tie_distance(etaps["quot_" + name][l].numpy().reshape(64, 32, -1))[first]
                worst = max(worst, float(dist.max()))
                tol = reflayers.E4M3_TIE_TOL if (l == 0 and name == "qkv") else reflayers.E4M3_TIE_TOL_AFTER_MATMUL
                assert (dist <= tol).all(), (l, name, float(dist.max()))
            flipped |= mism.any((1, 2))
    with capsys.disabled():
        print(f"\n  e4m3 free-running, 64 boards: {int((~flipped).sum())} without a flipped byte, worst of them "
              f"{per_board[~flipped].max():.2e} from the emulation (target 2e-2); {int(flipped.sum())} with a first flip "
              f"(a tie to {worst:.2e}), of them {(per_board[flipped] <= 2e-2).sum()} still within 2e-2, worst {per_board.max():.3f}")
    assert (~flipped).sum() >= 16
    assert (per_board[~flipped] <= 2e-2).all() and (per_board_v[~flipped] <= 2e-2).all()
    assert per_board[~flipped].max() < 1e-4          # in fact they agree to fp32 rounding
    assert per_board.max() < 0.3
    for i in (0, 1, 2):
        err_kernel, err_emu = (got[i] - f32[i]).abs(), (emu[i] - f32[i]).abs()
        # the mean over the batch is a stable statistic; the maximum over 64 boards moves with
        # which single board happened to flip a byte
        assert err_kernel.mean() < 1.15 * err_emu.mean() and err_kernel.max() < 1.5 * err_emu.max()
        assert (got[i] - emu[i]).abs().max() < err_emu.max()
    # same statement against what the reference itself wrote for its formula-weight network
    g8 = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "reference_vectors_e4m3.npz"))
    g32 = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "reference_vectors.npz"))
    torch.manual_seed(0)
    gnet = BrokefishNet().eval()
    gnet.load_state_dict(mg.fill_state_dict(gnet.state_dict()))
    p, q, v = [t.cpu().numpy() for t in encoder_impl("hip")(gnet, fp8=True, out_dtype=torch.float32)
               .forward_full(*_dev(*mg.positions()))]
    noise = np.abs(g8["e4m3_policy_nv1"] - g32["fp32_policy_nv1"]).max()
    assert np.abs(p - g8["e4m3_policy_nv1"]).max() < noise
    assert np.abs(p - g32["fp32_policy_nv1"]).max() < 1.15 * noise
    assert np.abs(v - g8["e4m3_value_nv1"]).max() < 5e-2


def test_launch_variants_agree_and_the_call_contract_holds(setup):
    net, sd, model = setup
    b, c, r, m = positions.random_positions(96, plies=120, seed=12)
    bd, cd, rd, md = _dev(b, c, r, m)
    tapped = model.forward_taps(bd, cd, rd, mask=md, want=["normed"])
    p, q, v = [t.clone() for t in model.forward_full(bd, cd, rd, md)]
    best = model.best_move.clone()
    assert torch.equal(p, tapped["policy"]) and torch.equal(q, tapped["promo"]) and torch.equal(v, tapped["value"])
    assert torch.equal(best, tapped["best"])
    legal = ((md[..., None] >> torch.arange(64, device="cuda")) & 1).bool()
    raw = model.forward_full(bd, cd, rd)[0].clone()
    assert torch.equal(p[legal], raw[legal]) and torch.isneginf(p[~legal]).all()
    flat = torch.where(legal, raw, torch.full_like(raw, float("-inf"))).reshape(96, -1)
    has = legal.reshape(96, -1).any(1)
    assert torch.equal(best[has].long(), flat.argmax(1)[has])
    half = encoder_impl("hip")(net, fp8=True)                                # default: the fp16 contract
    assert half.fp8 and not half.int8 and half.quant == 1 and "e4m3" in half.label
    ph, qh, vh = half.forward_full(bd, cd, rd)
    assert ph.dtype is torch.float16 and torch.equal(ph, raw.half()) and vh.dtype is torch.float32
    # deterministic, and independent of what else is in the batch
    again = model.forward_full(bd, cd, rd)[0]
    assert torch.equal(again, raw)
    perm = torch.randperm(96, generator=torch.Generator().manual_seed(1)).cuda()
    assert torch.equal(model.forward_full(bd[perm], cd[perm], rd[perm])[0], raw[perm])
    assert torch.equal(model.forward_full(bd[:5], cd[:5], rd[:5])[0], raw[:5])
    # the int8 object built from the same network is a different function of the same inputs
    i8 = encoder_impl("hip")(net, int8=True, out_dtype=torch.float32).forward_full(bd, cd, rd)[0]
    assert not torch.equal(i8, raw) and (i8 - raw).abs().max() < 1.0


def test_full_batch_properties_at_4096(setup):
    net, sd, model = setup
    b, c, r, m = positions.random_positions(4096, plies=120, seed=0)
    bd, cd, rd, md = _dev(b, c, r, m)
    p, q, v, best = [t.clone() for t in model.forward_masked(bd, cd, rd, md)]
    half = model.forward_masked(bd[2048:], cd[2048:], rd[2048:], md[2048:])
    assert torch.equal(half[0], p[2048:]) and torch.equal(half[3], best[2048:])
    legal = ((md[..., None] >> torch.arange(64, device="cuda")) & 1).bool()
    assert torch.isneginf(p[~legal]).all() and torch.isfinite(p[legal]).all() and (v.abs() <= 1).all()
    has = legal.reshape(4096, -1).any(1)
    assert torch.gather(legal.reshape(4096, -1)[has], 1, best[has].long()[:, None]).all()
    idx = torch.arange(0, 4096, 64)
    with torch.no_grad():
        emu = emulated.forward(sd, b[idx], c[idx], r[idx], mode="e4m3")
        f32 = emulated.forward(sd, b[idx], c[idx], r[idx], mode="fp32")
    raw = model.forward_full(bd, cd, rd)[0][idx.cuda()].cpu()
    # boards whose free-running logits stay within the 2e-2 target: every board that flips no byte at an
    # e4m3 tie (test above) does; measured 61 % of these 64 boards on this per-layer-distinct network (88-89 % on
    # the seed-0 network), and two orderings of the torch emulation agree with each other on 84-93 %
    within = ((raw - emu[0]).abs().reshape(64, -1).amax(1) <= 2e-2).float().mean().item()
    print(f"\n  e4m3 at batch 4096: {within:.0%} of 64 sampled boards within 2e-2 of the emulation free-running")
    assert within >= 0.55
    assert (raw - f32[0]).abs().mean() < 1.15 * (emu[0] - f32[0]).abs().mean()
    assert (raw - emu[0]).abs().max() < (emu[0] - f32[0]).abs().max()
