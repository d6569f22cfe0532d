"""Pins the two CPU checkers before anything is compared with them.

``oracle/emulated.py`` (torch library calls) and ``oracle/bf_oracle.c`` (explicit fp32
operation order) restate the reference's int8-simulated forward.  What pins which part:

=====================  ==========================================================================
function               pinned by
=====================  ==========================================================================
activation quantiser   reference device KATs: round-half-even / tie cases (csrc/tests/tint8.cu:59-61
                       with the host rule :39-46), the formula input + expected scale (:190-227);
                       golden vectors written by the reference's own quantise_activations_int8
weight quantiser       golden checksums + scales written by the reference's quantise_weights_int8_bytes
int8_linear            exact-integer GEMM KAT (csrc/tests/tint8.cu:269-279, :319-323, rebuilt with
                       power-of-two scales so the expected value is an exact closed form); golden
                       outputs of the reference's int8_linear incl. the 4-chunk float64 path
forward composition    golden logits/value of the reference's BrokefishNet (fp32) and of its
                       emulated_forward (int8) on formula weights; reproduced BIT FOR BIT by the
                       library-stack route; fp32 functional route == torch nn.TransformerEncoder
explicit-order C file  stage-by-stage against the torch restatement: identical operand bytes at the
                       first quantiser of a layer up to near-ties, identical int32 accumulators given
                       identical operands, outputs equal to rounding noise on rows with no flipped byte
exp / tanh             float64 libm
mask AND / argmax      closed form (docs/reference/spec.md:141-143, :537-540), lowest index on ties
=====================  ==========================================================================

Free-running int8 forwards of two implementations that differ only in fp32 summation
order do NOT stay within 1e-3 of each other: one flipped operand byte (a quotient landing
the other side of .5) is amplified by the following quantisers.  ``test_free_running_
sensitivity`` records that this is a property of the algorithm -- the reference's own
emulation moved by a re-ordering of its attention arithmetic shows the same spread.
"""
import numpy as np
import pytest
import torch

import make_golden as mg
import reflayers
from brokefish_amd import positions
from brokefish_amd.net import BrokefishNet
from oracle import c_oracle, emulated


def _net(nv=1, distinct=True, seed=0):
    torch.manual_seed(seed)
    net = BrokefishNet(n_value=nv).eval()
    if distinct:
        net.randomise_layers_(seed=seed + 3)
    return net, {k: v.detach() for k, v in net.state_dict().items()}


# --------------------------------------------------------------------------- #
# quantisers and int8_linear: reference KATs and closed forms
# --------------------------------------------------------------------------- #

def test_round_half_even_and_ties_signed():
    # tint8.cu:59-61 cases that fit a row whose scale is exactly 1 (amax = 127)
    row = np.zeros(256, np.float32)
    vals = [0.0, 1.0, -1.0, 2.5, 3.5, -3.5, 126.6, -126.6, 0.4, -0.4, 127.0, -127.0, 0.5, 1.5, -2.5]
    want = [0, 1, -1, 2, 4, -4, 127, -127, 0, 0, 127, -127, 0, 2, -2]      # nearbyint, tint8.cu:39-46
    row[:len(vals)] = vals
    q, s = c_oracle.quantise_activations_int8(row[None], unsigned=False)
    assert s[0] == 1.0 and q[0, :len(vals)].tolist() == want
    qt, st = emulated.quantise_activations_int8(torch.from_numpy(row[None]))
    assert st.item() == 1.0 and qt[0, :len(vals)].tolist() == want


def test_round_half_even_and_ties_unsigned():
    row = np.zeros(256, np.float32)
    vals = [0.0, 1.0, 2.5, 3.5, 254.7, 0.5, 255.0, -7.0, 126.5]
    want = [0, 1, 2, 4, 255, 0, 255, 0, 126]
    row[:len(vals)] = vals
    q, s = c_oracle.quantise_activations_int8(row[None], unsigned=True)
    assert s[0] == 1.0 and q[0, :len(vals)].tolist() == want
    qt, st = emulated.quantise_activations_int8(torch.from_numpy(row[None]), unsigned=True)
    assert st.item() == 1.0 and qt[0, :len(vals)].tolist() == want


@pytest.mark.parametrize("unsigned", [False, True])
def test_quantiser_on_the_reference_formula_input(unsigned):
    # tint8.cu:190-227: v = (((r*31 + k*17) % 401) - 200) * 0.001 * (r+1); scale = amax / qmax.
    r, k = np.meshgrid(np.arange(32), np.arange(256), indexing="ij")
    v = (((r * 31 + k * 17) % 401) - 200).astype(np.float32) * (np.float32(0.001) * (r + 1).astype(np.float32))
    if unsigned:
        v = np.abs(v)
    qmax = np.float32(255.0 if unsigned else 127.0)
    amax = np.abs(v).max(axis=1)
    want_s = amax / qmax
    # independent statement of the rule: IEEE fp32 quotient, then round half to even
    want_q = np.rint(v / want_s[:, None]).astype(np.int64)
    q, s = c_oracle.quantise_activations_int8(v, unsigned)
    assert (s == want_s).all() and (q == want_q).all()
    qt, st = emulated.quantise_activations_int8(torch.from_numpy(v), unsigned)
    assert (st.numpy().reshape(-1) == want_s).all() and (qt.numpy() == want_q).all()
    assert q.max() == (255 if unsigned else 127)


@pytest.mark.parametrize("unsigned", [False, True])
def test_int8_linear_is_the_exact_integer_product(unsigned):
    # tint8.cu:269-279: A = ((m*13 + k*7) % 255) - 127 (or % 256 unsigned), W = ((n*11 + k*5) % 255) - 127.
    # Scales are powers of two here so the quantisers recover A and W exactly and the
    # expected output (float)dot * sa * sw (+ nothing) is a closed form (tint8.cu:319-323).
    M, K, N = 32, 512, 128
    m, k = np.meshgrid(np.arange(M), np.arange(K), indexing="ij")
    A = ((m * 13 + k * 7) % 256) if unsigned else (((m * 13 + k * 7) % 255) - 127)
    n, k2 = np.meshgrid(np.arange(N), np.arange(K), indexing="ij")
    W = ((n * 11 + k2 * 5) % 255) - 127
    sa = (2.0 ** -(np.arange(M) % 8 + 3)).astype(np.float32)
    sw = np.float32(2.0 ** -9)
    x = (A.astype(np.float32) * sa[:, None])
    w = W.astype(np.float32) * sw
    acc = np.stack([A[:, c:c + 256].astype(np.int64) @ W[:, c:c + 256].astype(np.int64).T for c in (0, 256)])
    want = ((acc[0].astype(np.float64) * sa[:, None].astype(np.float64)
             + acc[1].astype(np.float64) * sa[:, None].astype(np.float64)).astype(np.float32) * sw)
    got_c = c_oracle.int8_linear(x, w, None, unsigned)
    got_t = emulated.int8_linear(torch.from_numpy(x), torch.from_numpy(w), None, unsigned).numpy()
    assert (got_c == want).all() and (got_t == want).all()
    wq, ws = c_oracle.quantise_weights_int8(w)
    assert (wq == W).all() and (ws == sw).all()
    out, qa, sa_tap, acc_tap = c_oracle.int8_linear_q(x, wq, ws, None, unsigned)
    assert (qa == A).all() and (acc_tap == acc).all() and (sa_tap == np.stack([sa, sa], 1)).all()
    # the accumulator bound the reference asserts (brokefish/nn/quant.py:243)
    assert np.abs(acc).max() <= 255 * 127 * 256 < 2 ** 31 - 1


def test_golden_int8_linear_and_quantisers(golden):
    for name, x, w, bias, unsigned in mg.linear_cases():
        want = golden["lin_" + name]
        got_t = emulated.int8_linear(x, w, bias, unsigned).numpy()
        got_c = c_oracle.int8_linear(x.numpy(), w.numpy(), None if bias is None else bias.numpy(), unsigned)
        assert (got_t.view(np.int32) == want.view(np.int32)).all(), name
        assert (got_c.view(np.int32) == want.view(np.int32)).all(), name
        q, s = c_oracle.quantise_activations_int8(x[:, :256].numpy(), unsigned)
        assert (q == golden["qa_" + name]).all() and (s == golden["sa_" + name].reshape(-1)).all()
        wq, ws = c_oracle.quantise_weights_int8(w.numpy())
        wqt, wst = emulated.quantise_weights_int8(w)
        assert (mg.weight_checksum(wq) == golden["wqsum_" + name]).all() and (ws == golden["ws_" + name]).all()
        assert (wqt.numpy() == wq).all() and (wst.numpy() == ws).all()
    assert golden["sa_s8_zero_row"][3, 0] == 1.0          # an all-zero row takes scale 1


# --------------------------------------------------------------------------- #
# the forward composition
# --------------------------------------------------------------------------- #

def _golden_net(nv):
    torch.manual_seed(0)
    net = BrokefishNet(n_value=nv).eval()
    sd = mg.fill_state_dict(net.state_dict())
    b, c, r = mg.positions()
    if nv == 3:
        b, c, r = b[:3], c[:3], r[:3]
    return sd, b, c, r


@pytest.mark.parametrize("nv", [1, 3])
def test_golden_forward_fp32(golden, nv):
    sd, b, c, r = _golden_net(nv)
    with torch.no_grad():
        got = emulated.forward(sd, b, c, r, mode="fp32")
    for i, name in enumerate(("policy", "promo", "value")):
        assert np.abs(got[i].numpy() - golden[f"fp32_{name}_nv{nv}"]).max() < 2e-5
    if nv == 1:
        x, _ = emulated.embed(sd, b, c, r)
        y = torch.nn.functional.layer_norm(x, (256,), sd["encoder.layers.0.norm1.weight"],
                                           sd["encoder.layers.0.norm1.bias"], 1e-5)
        assert np.abs(y[:2].numpy() - golden["ln1_layer0"]).max() < 1e-5


@pytest.mark.parametrize("nv", [1, 3])
def test_golden_forward_int8_bit_exact_through_the_library_stack(golden, nv):
    sd, b, c, r = _golden_net(nv)
    got = emulated.forward_library_stack(sd, b, c, r, mode="int8")
    same_torch = str(golden["torch_version"]) == torch.__version__
    for i, name in enumerate(("policy", "promo", "value")):
        want = golden[f"int8_{name}_nv{nv}"]
        if same_torch:
            assert (got[i].numpy().view(np.int32) == want.view(np.int32)).all(), name
        else:   # another torch build may order its attention sums differently
            assert np.abs(got[i].numpy() - want).max() < 5e-2, name


@pytest.mark.parametrize("nv", [1, 3])
def test_golden_forward_int8_other_routes_within_the_algorithms_own_spread(golden, nv):
    # Same algorithm, different fp32 summation order inside attention / LayerNorm: agreement
    # only to the forward's own sensitivity (see test_free_running_sensitivity).
    sd, b, c, r = _golden_net(nv)
    with torch.no_grad():
        got_t = emulated.forward(sd, b, c, r, mode="int8")
    got_c = c_oracle.COracle(sd).forward(b.numpy(), c.numpy(), r.numpy())
    quant_noise = np.abs(golden[f"int8_policy_nv{nv}"] - golden[f"fp32_policy_nv{nv}"]).max()
    for got in (got_t[0].numpy(), got_c["policy"]):
        assert np.abs(got - golden[f"int8_policy_nv{nv}"]).max() < quant_noise
    assert np.abs(got_c["value"] - golden[f"int8_value_nv{nv}"]).max() < 2e-2


def test_fp32_restatement_equals_torch_transformer_encoder():
    net, sd = _net()
    b, c, r, _ = positions.random_positions(16, plies=80, seed=4, stamp_queen=True)
    with torch.no_grad():
        x, alive = emulated.embed(sd, b, c, r)
        h = net.norm_f(net.encoder(x, src_key_padding_mask=~alive))
        want = net.policy(h)
        got = emulated.forward(sd, b, c, r, mode="fp32")[0]
    assert (got - want).abs().max().item() < 2e-5


def test_c_checker_stage_by_stage_against_the_torch_restatement(capsys):
    net, sd = _net()
    n = 16
    b, c, r, _ = positions.random_positions(n, plies=80, seed=6, stamp_queen=True)
    taps = {}
    with torch.no_grad():
        emulated.forward(sd, b, c, r, mode="int8", taps=taps)
    co = c_oracle.COracle(sd)
    x_in = taps["embed"].numpy()
    total_rows, clean_rows = 0, 0
    n_flips, n_bytes, worst = 0, 0, 0.0
    for l in range(co.L):
        out = co.forward(b.numpy(), c.numpy(), r.numpy(), taps=True, x_in=x_in, layer_begin=l, layer_end=l + 1)
        bad_rows = np.zeros((n, 32), bool)
        for name in ("qkv", "out", "ff1", "ff2"):
            qt = taps["qa_" + name][l].numpy().reshape(n, 32, -1).astype(np.int32)
            qc = out["qa_" + name][:, 0]
            qc = (qc.view(np.uint8) if name == "ff2" else qc).astype(np.int32)
            mism = qt != qc
            clean = ~bad_rows                                           # rows with identical inputs so far
            assert np.abs(qt - qc)[clean].max() <= 1                    # a flip is one step, never more
            # ... and EVERY flip on a clean row is a provable tie: the quotient x / s (float64, from the
            # restatement's own fp32 x and s) sits within 2^-18 of full scale of a rounding boundary
            flips = mism & clean[..., None]
            dist = reflayers.tie_distance(taps["quot_" + name][l].numpy().reshape(n, 32, -1))
            tol = reflayers.TIE_TOL_U8 if name == "ff2" else reflayers.TIE_TOL
            assert (dist[flips] <= tol).all(), (l, name, int(flips.sum()), float(dist[flips].max()))
            n_flips += int(flips.sum())
            n_bytes += int(clean.sum()) * qt.shape[-1]
            worst = max(worst, float(dist[flips].max()) if flips.any() else 0.0)
            # exact integer GEMM: identical operand rows give identical accumulators
            at = taps["acc_" + name][l].numpy()
            at = at.reshape(at.shape[0], n, 32, -1).transpose(1, 0, 2, 3)
            ac = out["acc_" + name][:, 0]
            row_ok = ~mism.any(-1)
            assert (at.transpose(0, 2, 1, 3)[row_ok] == ac.transpose(0, 2, 1, 3)[row_ok]).all()
            bad_rows |= mism.any(-1)
            if name == "qkv":         # attention mixes the rows of a board
                bad_rows |= mism.any(-1).any(-1)[:, None]
        x_next = taps["resid"][l].numpy()
        d = np.abs(out["resid"][:, 0] - x_next).max(-1)
        scale = np.abs(x_next).max()
        assert d[~bad_rows].max() < 2e-5 * max(scale, 1.0)
        total_rows += bad_rows.size
        clean_rows += (~bad_rows).sum()
        x_in = x_next
    assert clean_rows > 0.5 * total_rows
    with capsys.disabled():
        print(f"\n  C checker vs torch restatement, teacher-forced: {n_flips} flipped bytes of {n_bytes} on clean rows, "
              f"every one within {worst:.2e} steps of a tie (allowed {reflayers.TIE_TOL:.2e}); {clean_rows}/{total_rows} rows clean")


def test_free_running_sensitivity_is_a_property_of_the_algorithm():
    # The torch restatement with its own attention arithmetic, and the same restatement
    # through torch's attention module, are the SAME algorithm in the same library and
    # differ only in fp32 operation order -- and already miss 1e-3 on some positions.
    net, sd = _net(distinct=False)
    b, c, r, _ = positions.random_positions(32, plies=80, seed=0)
    with torch.no_grad():
        a = emulated.forward(sd, b, c, r, mode="int8")[0]
    z = emulated.forward_library_stack(sd, b, c, r, mode="int8")[0]
    spread_torch = (a - z).abs().reshape(32, -1).max(1)[0]
    cc = c_oracle.COracle(sd).forward(b.numpy(), c.numpy(), r.numpy())["policy"]
    spread_c = np.abs(cc - z.numpy()).reshape(32, -1).max(1)
    assert spread_torch.max().item() > 1e-3          # the bar is not reachable by re-ordering alone
    assert spread_c.max() < 10 * max(spread_torch.max().item(), 1e-3)
    with torch.no_grad():
        fp32 = emulated.forward(sd, b, c, r, mode="fp32")[0]
    assert spread_c.max() < (z - fp32).abs().max().item()    # and stays below the quantisation noise itself


# --------------------------------------------------------------------------- #
# scalar functions, heads, mask
# --------------------------------------------------------------------------- #

def test_exp_and_tanh_against_libm():
    L = c_oracle.lib()
    xs = np.concatenate([-np.logspace(-6, np.log10(86.9), 4000), [0.0, -87.0, -1e-8]]).astype(np.float32)
    got = np.array([L.bfo_exp_neg(float(x)) for x in xs])
    want = np.exp(xs.astype(np.float64))
    assert (np.abs(got - want) / want).max() < 2.5e-7
    assert L.bfo_exp_neg(-88.0) == 0.0 and L.bfo_exp_neg(float("-inf")) == 0.0 and L.bfo_exp_neg(0.0) == 1.0
    ts = np.concatenate([np.linspace(-12, 12, 4001), [0.0, 1e-6, -1e-6]]).astype(np.float32)
    gt = np.array([L.bfo_tanh(float(x)) for x in ts])
    assert np.abs(gt - np.tanh(ts.astype(np.float64))).max() < 2e-7
    assert L.bfo_tanh(20.0) == 1.0 and L.bfo_tanh(-20.0) == -1.0 and L.bfo_tanh(0.0) == 0.0


def test_division_by_a_scale_constant_equals_ieee_division():
    # the kernels divide a row maximum by 127 or 255 as one multiply by the rounded reciprocal and
    # one residual correction; that equals the correctly rounded quotient for every positive
    # float (checked exhaustively once: 0 of 2,139,095,039), sampled here at every 997th value
    L = c_oracle.lib()
    for d in (127.0, 255.0):
        assert L.bfo_check_div_const(d, 997) == 0
    assert L.bfo_check_div_const(127.0, 1 << 20) == 0 and L.bfo_check_div_const(10.0, 997) > 0   # the check can fail: not every divisor has the property


def test_every_clock_sign_and_rep_reaches_its_table_row():
    # reference tests/test_b2.py:110-133: all 101 clocks x 2 signs x 3 reps
    net, sd = _net()
    co = c_oracle.COracle(sd)
    board = np.tile(positions.random_positions_np(1, plies=0)[0], (1, 1))
    ctrl, reps = [], []
    for mag in list(range(1, 103)) + [150]:
        for sign in (1, -1):
            for rp in (0, 1, 2, 7):
                ctrl.append(sign * mag)
                reps.append(rp)
    n = len(ctrl)
    b = np.repeat(board, n, axis=0)
    out = co.forward(b.view(np.int16), np.array(ctrl, np.int16), np.array(reps, np.uint8), taps=True,
                     layer_begin=0, layer_end=1)
    E = {k: sd[f"emb_{k}.weight"].numpy() for k in ("square", "type_special", "color_turn", "clock", "rep")}
    for i in (0, 5, 17, n - 1, n // 2):
        stm = int(ctrl[i] < 0)
        ck = min(abs(ctrl[i]) - 1, 100)
        rp = min(reps[i], 2)
        w = int(board[0, 20])
        want = ((E["square"][w & 63] + E["type_special"][((w >> 6) & 7) * 2 + ((w >> 9) & 1)])
                + E["color_turn"][((w >> 10) & 1) * 2 + stm]) + (E["clock"][ck] + E["rep"][rp])
        assert (out["embed"][i, 20] == want).all()
    with torch.no_grad():
        xt, _ = emulated.embed(sd, torch.from_numpy(b.view(np.int16)), torch.tensor(ctrl, dtype=torch.int16),
                               torch.tensor(reps, dtype=torch.uint8))
    assert (out["embed"] == xt.numpy()).all()


def test_dead_slots_are_inert():
    # reference tests/test_b2.py:270-293: garbage in the low bits of a captured slot changes
    # nothing any live token or the value can see.
    net, sd = _net()
    co = c_oracle.COracle(sd)
    b, c, r, _ = positions.random_positions_np(64, plies=120, seed=8)
    dead = (b & 0x800) != 0
    assert dead.any()
    b2 = b.copy()
    rng = np.random.default_rng(0)
    garbage = rng.integers(0, 0x600, size=b.shape).astype(np.uint16) & np.uint16(0x5FF)   # types 0..5 only
    garbage = (garbage & ~np.uint16(0x1C0)) | (rng.integers(0, 6, size=b.shape).astype(np.uint16) << 6)
    b2[dead] = 0x800 | garbage[dead]
    o1 = co.forward(b.view(np.int16), c, r)
    o2 = co.forward(b2.view(np.int16), c, r)
    live = ~dead
    assert (o1["policy"][live] == o2["policy"][live]).all()
    assert (o1["promo"][live] == o2["promo"][live]).all()
    assert (o1["value"] == o2["value"]).all()
    assert np.isfinite(o2["policy"]).all()


def test_value_head_rules():
    # king row select (reference tests/test_b2.py:185-209) and the win/draw/loss class order:
    # swapping the loss and win rows negates the value (tests/test_b2.py:417-446).
    net, sd = _net(nv=3)
    co = c_oracle.COracle(sd)
    b, c, r, _ = positions.random_positions_np(24, plies=60, seed=3)
    out = co.forward(b.view(np.int16), c, r, taps=True)
    king = np.where(c < 0, 31, 15)
    h = out["normed"][np.arange(24), king].astype(np.float64)
    raw = h @ sd["value.weight"].numpy().astype(np.float64).T
    p = np.exp(raw - raw.max(1, keepdims=True))
    p /= p.sum(1, keepdims=True)
    assert np.abs(out["value"] - (p[:, 2] - p[:, 0])).max() < 1e-5
    sd2 = dict(sd)
    sd2["value.weight"] = sd["value.weight"][[2, 1, 0]].clone()
    out2 = c_oracle.COracle(sd2).forward(b.view(np.int16), c, r)
    assert np.abs(out2["value"] + out["value"]).max() < 1e-6
    net1, sd1 = _net(nv=1)
    o1 = c_oracle.COracle(sd1).forward(b.view(np.int16), c, r, taps=True)
    raw1 = o1["normed"][np.arange(24), king].astype(np.float64) @ sd1["value.weight"].numpy()[0].astype(np.float64)
    assert np.abs(o1["value"] - np.tanh(raw1)).max() < 1e-5


@pytest.fixture(scope="module")
def golden_layers():
    import os
    return np.load(os.path.join(os.path.dirname(mg.__file__), "reference_vectors_layers.npz"))


def _golden_value_net(head, nv):
    torch.manual_seed(0)
    net = BrokefishNet(n_value=nv, value_head=head).eval()
    sd = mg.fill_state_dict(net.state_dict())
    return (sd,) + tuple(mg.positions())


@pytest.mark.parametrize("head", ["pooled", "prenorm"])
@pytest.mark.parametrize("nv", [1, 3])
def test_pooled_value_heads_against_the_reference(golden, golden_layers, head, nv):
    # the reference's own model with value_head="pooled" / "prenorm" (brokefish/nn/model.py:576-617;
    # its tests: tests/test_b2.py:520-650) wrote these values for the formula weights
    sd, b, c, r = _golden_value_net(head, nv)
    assert int(sd["value_mode"]) == {"pooled": 1, "prenorm": 2}[head]
    with torch.no_grad():
        got32 = emulated.forward(sd, b, c, r, mode="fp32")
    assert np.abs(got32[2].numpy() - golden_layers[f"fp32_value_{head}_nv{nv}"]).max() < 2e-6
    got8 = emulated.forward_library_stack(sd, b, c, r, mode="int8")
    if str(golden_layers["torch_version"]) == torch.__version__:
        assert (got8[2].numpy().view(np.int32) == golden_layers[f"int8_value_{head}_nv{nv}"].view(np.int32)).all()
        assert abs(got8[0].double().sum().item() - float(golden_layers[f"int8_policysum_{head}_nv{nv}"])) < 1e-9
    # the head changes the value only: the logits are the king net's
    nb = 3 if nv == 3 else 8
    assert np.abs(got32[0].numpy()[:nb] - golden[f"fp32_policy_nv{nv}"]).max() < 2e-5
    assert not np.allclose(got32[2].numpy()[:nb], golden[f"fp32_value_nv{nv}"], atol=1e-3)


@pytest.mark.parametrize("head", ["pooled", "prenorm"])
@pytest.mark.parametrize("nv", [1, 3])
def test_c_checker_pooled_value_heads_teacher_forced(head, nv):
    # the C checker's pooled heads (butterfly token sum, the token LayerNorm on the pooled row, the
    # value rows' fma chain, negation for Black) given the same residual stream as the torch
    # restatement: agreement to fp32 rounding, both colours, dead slots excluded from the mean
    torch.manual_seed(5)
    net = BrokefishNet(n_value=nv, value_head=head, n_layers=2).eval().randomise_layers_(seed=9)
    sd = {k: v.detach() for k, v in net.state_dict().items()}
    b, c, r, _ = positions.random_positions(48, plies=120, seed=7)
    assert (c < 0).any() and (c > 0).any()
    taps = {}
    with torch.no_grad():
        want = emulated.forward(sd, b, c, r, mode="int8", taps=taps)
    x_last = taps["resid"][-1].numpy()
    co = c_oracle.COracle(sd)
    assert co.value_mode == {"pooled": 1, "prenorm": 2}[head]
    got = co.forward(b.numpy(), c.numpy(), r.numpy(), x_in=x_last, layer_begin=2, layer_end=2)
    assert np.abs(got["value"] - want[2].numpy()).max() < 2e-6
    # closed form in float64 from the checker's own normed / residual stream
    alive = ((b.numpy().view(np.uint16) >> 11) & 1) == 0
    full = co.forward(b.numpy(), c.numpy(), r.numpy(), taps=True)
    src = full["normed"] if head == "pooled" else full["resid"][:, -1]
    pooled = (src.astype(np.float64) * alive[..., None]).sum(1) / np.maximum(alive.sum(1), 1)[:, None]
    if head == "prenorm":
        mu, var = pooled.mean(1, keepdims=True), pooled.var(1, keepdims=True)
        pooled = (pooled - mu) / np.sqrt(var + 1e-5) * sd["norm_f.weight"].numpy() + sd["norm_f.bias"].numpy()
    raw = pooled @ sd["value.weight"].numpy().astype(np.float64).T
    if nv == 1:
        val = np.tanh(raw[:, 0])
    else:
        p = np.exp(raw - raw.max(1, keepdims=True))
        p /= p.sum(1, keepdims=True)
        val = p[:, 2] - p[:, 0]
    val = np.where(c.numpy() > 0, val, -val)
    assert np.abs(full["value"] - val).max() < 2e-6


def test_c_checker_layer_by_layer_from_the_references_own_residual_stream(capsys):
    # The reference's emulated_forward wrote, for layers 0, 3, 7 of the golden network, the residual
    # stream entering the layer and every operand byte, scale and int32 accumulator inside it
    # (tests/golden/make_golden.py `layers`).  The C checker, run on that one layer from the
    # reference's stream, must give the reference's bytes (but for provable rounding ties) and the
    # reference's accumulators exactly.
    _, _, sd, b, c, r = reflayers.load()
    co = c_oracle.COracle(sd)

    def run_layer(l, x_in):
        return co.forward(b.numpy(), c.numpy(), r.numpy(), taps=True, x_in=x_in, layer_begin=l, layer_end=l + 1)

    stats = reflayers.check(run_layer)
    with capsys.disabled():
        print("\n  C checker vs the reference's per-layer data:", stats)


def test_mask_and_argmax_closed_form():
    net, sd = _net()
    co = c_oracle.COracle(sd)
    b, c, r, m = positions.random_positions_np(32, plies=100, seed=12)
    raw = co.forward(b.view(np.int16), c, r)
    out = co.forward(b.view(np.int16), c, r, mask=m.view(np.int64))
    legal = ((m[..., None] >> np.arange(64, dtype=np.uint64)) & np.uint64(1)).astype(bool)
    assert (out["policy"][legal] == raw["policy"][legal]).all()
    assert np.isneginf(out["policy"][~legal]).all()
    flat = np.where(legal, raw["policy"], -np.inf).reshape(32, -1)
    has = legal.reshape(32, -1).any(1)
    assert (out["best"][has] == flat.argmax(1)[has]).all()      # numpy argmax = first maximum
    assert (out["best"][~has] == -1).all()
    with torch.no_grad():
        t = emulated.forward(sd, torch.from_numpy(b.view(np.int16)), torch.from_numpy(c), torch.from_numpy(r),
                             mode="int8", mask=torch.from_numpy(m.view(np.int64)))
    assert (np.isneginf(t[0].numpy()) == np.isneginf(out["policy"])).all()
    # ties: all-zero heads give equal logits, the lowest legal index must win
    sd0 = dict(sd)
    sd0["policy.weight"] = torch.zeros_like(sd["policy.weight"])
    o0 = c_oracle.COracle(sd0).forward(b.view(np.int16), c, r, mask=m.view(np.int64))
    first = np.where(has, legal.reshape(32, -1).argmax(1), -1)
    assert (o0["best"] == first).all()
